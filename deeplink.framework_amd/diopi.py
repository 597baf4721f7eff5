"""ctypes view of the DIOPI C ABI (include/diopi/*.h) and of the diopirt objects of
include/dipu_amd/runtime.h.

This is the marshalling DIPU's generated wrappers do in C++
(dipu/scripts/autogen_diopi_wrapper/autogen_diopi_wrapper.py:878-961 and
dipu/torch_dipu/csrc_dipu/diopirt/diopi_helper.cpp:9-261): tensors become opaque handles,
Python numbers become diopiScalar_t with an int64 or float64 payload, int lists become
diopiSize_t by value, undefined tensors become NULL. torch is used only as the owner of
device memory: a handle carries the tensor's data pointer, shape, strides and dtype.
"""
import ctypes
from ctypes import POINTER, Structure, Union, byref, c_bool, c_char_p, c_double, c_int, c_int32, c_int64, c_uint64, c_void_p

import torch

from . import _native, runtime

MAX_DIMS = 8


class DiopiError(RuntimeError):
    pass


class dipuAmdTensor(Structure):
    _fields_ = [
        ("data", c_void_p),
        ("ndim", c_int64),
        ("shape", c_int64 * MAX_DIMS),
        ("stride", c_int64 * MAX_DIMS),
        ("dtype", c_int32),
        ("device", c_int32),
        ("device_index", c_int32),
        ("reserved", c_int32),
        ("storage_offset", c_int64),
        ("storage_ptr", c_void_p),
        ("storage_nbytes", c_uint64),
    ]


class _ScalarPayload(Union):
    _fields_ = [("fval", c_double), ("ival", c_int64)]


class diopiScalar_t(Structure):
    _anonymous_ = ("u",)
    _fields_ = [("stype", c_int32), ("u", _ScalarPayload)]


class diopiSize_t(Structure):
    _fields_ = [("data", POINTER(c_int64)), ("len", c_int64)]


# include/diopi/diopirt.h enumerators
DTYPE = {
    torch.int8: 0, torch.uint8: 1, torch.int16: 2, torch.int32: 4, torch.int64: 6,
    torch.float16: 8, torch.float32: 9, torch.float64: 10, torch.bool: 11, torch.bfloat16: 12,
}
DIOPI_HOST, DIOPI_DEVICE = 0, 1
ROUND_MODE = {None: 0, "floor": 1, "trunc": 2}
DIOPI_SUCCESS = 0


def scalar(value):
    """diopi_helper.cpp:74-97: bool/int -> int64 payload, float -> float64 payload."""
    s = diopiScalar_t()
    if isinstance(value, bool) or isinstance(value, int):
        s.stype = 6
        s.ival = int(value)
    elif isinstance(value, float):
        s.stype = 10
        s.fval = value
    else:
        raise TypeError(f"invalid scalar type {type(value)}")
    return s


def size(values):
    arr = (c_int64 * len(values))(*values)
    s = diopiSize_t(ctypes.cast(arr, POINTER(c_int64)), len(values))
    s._keepalive = arr
    return s


class Handle:
    """A diopiTensorHandle_t for a torch tensor. Keeps the tensor alive while the handle lives."""

    __slots__ = ("tensor", "desc", "ptr")

    def __init__(self, t):
        if t.dim() > MAX_DIMS:
            raise DiopiError(f"tensors of rank {t.dim()} are not supported (max {MAX_DIMS})")
        if t.dtype not in DTYPE:
            raise DiopiError(f"dtype {t.dtype} has no DIOPI equivalent on this backend")
        d = dipuAmdTensor()
        d.data = t.data_ptr()
        d.ndim = t.dim()
        for i, (n, s) in enumerate(zip(t.shape, t.stride())):
            d.shape[i] = n
            d.stride[i] = s
        d.dtype = DTYPE[t.dtype]
        d.device = DIOPI_HOST if t.device.type == "cpu" else DIOPI_DEVICE
        d.device_index = t.device.index if t.device.index is not None else -1
        d.storage_offset = t.storage_offset()
        st = t.untyped_storage()
        d.storage_ptr = st.data_ptr() if st.nbytes() else None
        d.storage_nbytes = st.nbytes()
        self.tensor = t
        self.desc = d
        self.ptr = ctypes.cast(ctypes.pointer(d), c_void_p)


def handle(t):
    """None (undefined tensor) -> NULL handle, as diopi_helper.cpp:13-34 does."""
    if t is None:
        return None, c_void_p(None)
    h = t if isinstance(t, Handle) else Handle(t)
    return h, h.ptr


class Generator:
    """The generator object behind the diopiGenerator* runtime callbacks (what vendorMakeGenerator returns in DIPU,
    runtime/core/DIPUGeneratorImpl.h:62): a Philox seed and offset, state = 16 host bytes (seed, offset)."""

    def __init__(self, device_index=0):
        self.ptr = c_void_p()
        if _native.runtime().dipuAmdGeneratorCreate(byref(self.ptr), c_int(device_index)) != 0:
            raise DiopiError("dipuAmdGeneratorCreate failed")

    def close(self):
        if self.ptr:
            _native.runtime().dipuAmdGeneratorDestroy(self.ptr)
            self.ptr = None

    def seed_and_offset(self):
        seed, off = c_uint64(), c_uint64()
        rc = _native.runtime().diopiGeneratorGetSeedAndOffset(self.ptr, byref(seed), byref(off))
        if rc != 0:
            raise DiopiError(f"diopiGeneratorGetSeedAndOffset returned {rc}")
        return seed.value, off.value

    def set_seed_and_offset(self, seed, offset):
        rc = _native.runtime().diopiGeneratorSetSeedAndOffset(self.ptr, c_uint64(seed), c_uint64(offset))
        if rc != 0:
            raise DiopiError(f"diopiGeneratorSetSeedAndOffset returned {rc} (the offset must be a multiple of 4)")

    def get_state(self):
        """The state as a uint8 CPU tensor of 16 bytes (copied out of the context's workspace before it closes)."""
        import torch
        with Context(0) as ctx:  # the state lives on the host: no stream is involved
            th = c_void_p()
            rc = _native.runtime().diopiGeneratorGetState(ctx.ptr, self.ptr, byref(th))
            if rc != 0:
                raise DiopiError(f"diopiGeneratorGetState returned {rc}")
            desc = ctypes.cast(th, POINTER(dipuAmdTensor)).contents
            raw = ctypes.string_at(desc.data, int(desc.shape[0]))
        return torch.frombuffer(bytearray(raw), dtype=torch.uint8)

    def set_state(self, state):
        h, p = handle(state)
        rc = _native.runtime().diopiGeneratorSetState(self.ptr, p)
        if rc != 0:
            raise DiopiError(f"diopiGeneratorSetState returned {rc} (state must be 16 or 8 host bytes, offset a multiple of 4)")


class Context:
    """diopiContext bound to a stream (diopirt_impl.h:19-26). Workspace the impl library
    requests lives until the context is closed; DIPU closes it when the wrapper returns."""

    def __init__(self, stream=None):
        rt = _native.runtime()
        if stream is None:
            stream = torch.cuda.current_stream().cuda_stream
        self.stream = stream
        p = c_void_p()
        if rt.dipuAmdContextCreate(c_void_p(stream), byref(p)) != 0:
            raise DiopiError(rt_error())
        self.ptr = p

    def workspace(self):
        n, b = c_uint64(), c_uint64()
        _native.runtime().dipuAmdContextWorkspace(self.ptr, byref(n), byref(b))
        return n.value, b.value

    def reset(self):
        _native.runtime().dipuAmdContextReset(self.ptr)

    def close(self):
        if self.ptr is not None:
            _native.runtime().dipuAmdContextDestroy(self.ptr)
            self.ptr = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def rt_error():
    f = _native.runtime().dipuAmdGetLastError
    f.restype = c_char_p
    return (f() or b"").decode()


def last_error():
    f = _native.impl().diopiGetLastErrorString
    f.restype = c_char_p
    return (f() or b"").decode()


_T, _S, _SZ = c_void_p, POINTER(diopiScalar_t), diopiSize_t
# name -> ctypes argument types after the leading context handle (include/diopi/functions*.h)
SIGNATURES = {
    "diopiAdd": [_T, _T, _T, _S],
    "diopiAddInp": [_T, _T, _S],
    "diopiAddScalar": [_T, _T, _S, _S],
    "diopiAddInpScalar": [_T, _S, _S],
    "diopiSub": [_T, _T, _T, _S],
    "diopiSubScalar": [_T, _T, _S, _S],
    "diopiMul": [_T, _T, _T],
    "diopiMulInp": [_T, _T],
    "diopiMulScalar": [_T, _T, _S],
    "diopiMulInpScalar": [_T, _S],
    "diopiDiv": [_T, _T, _T, c_int],
    "diopiDivScalar": [_T, _T, _S, c_int],
    "diopiSilu": [_T, _T],
    "diopiSiluInp": [_T],
    "diopiSigmoid": [_T, _T],
    "diopiRsqrt": [_T, _T],
    "diopiNeg": [_T, _T],
    "diopiSin": [_T, _T],
    "diopiCos": [_T, _T],
    "diopiExp": [_T, _T],
    "diopiPow": [_T, _T, _S],
    "diopiFill": [_T, _S],
    "diopiSoftmax": [_T, _T, c_int64],
    "diopiMean": [_T, _T, _SZ],
    "diopiCopyInp": [_T, _T],
    "diopiCat": [_T, POINTER(c_void_p), c_int64, c_int64],
    "diopiIndexPutInp": [_T, _T, POINTER(c_void_p), c_int64, c_bool],
    "diopiWhere": [_T, _T, _T, _T],
    "diopiMaskedFill": [_T, _T, _T, _T],
    "diopiMaskedFillInp": [_T, _T, _T],
    "diopiMaskedFillScalar": [_T, _T, _T, _S],
    "diopiMaskedFillInpScalar": [_T, _T, _S],
    "diopiTril": [_T, _T, c_int64],
    "diopiTriu": [_T, _T, c_int64],
    "diopiTriuInp": [_T, c_int64],
    "diopiArange": [_T, _S, _S, _S],
    "diopiIndexSelect": [_T, _T, c_int64, _T],
    "diopiGather": [_T, _T, c_int64, _T],
    "diopiEq": [_T, _T, _T],
    "diopiEqScalar": [_T, _T, _S],
    "diopiNe": [_T, _T, _T],
    "diopiNeScalar": [_T, _T, _S],
    "diopiLt": [_T, _T, _T],
    "diopiLtScalar": [_T, _T, _S],
    "diopiLe": [_T, _T, _T],
    "diopiLeScalar": [_T, _T, _S],
    "diopiGt": [_T, _T, _T],
    "diopiGtScalar": [_T, _T, _S],
    "diopiGe": [_T, _T, _T],
    "diopiGeScalar": [_T, _T, _S],
    "diopiMm": [_T, _T, _T],
    "diopiBmm": [_T, _T, _T],
    "diopiMatmul": [_T, _T, _T],
    "diopiAddmm": [_T, _T, _T, _T, _S, _S],
    "diopiBaddbmm": [_T, _T, _T, _T, c_double, c_double],
    "diopiLinear": [_T, _T, _T, _T],
    "diopiRMSNorm": [_T, _T, _T, _SZ, _T, _T, c_double],
    "diopiRotaryEmbedding": [_T, _T, _T, _T, c_bool, c_bool],
    "diopiDestIndexCopyKV": [_T, _T, _T],
    "diopiDestIndexCopyKVPair": [_T, _T, _T, _T, _T],
    "diopiTokenAttentionInference": [_T, _T, _T, _T, _T, _T, c_int],
    "diopiTokenSoftmaxReduceVInference": [_T, _T, _T, _T, _T, _T, c_int, c_int],
    "diopiContextAttentionInference": [_T, _T, _T, _T, _T, _T, c_int],
    "diopiTokenDecodeAttentionInference": [_T, _T, _T, _T, _T, _T, _T, c_int],
    "diopiTokenDecodeAttentionInferenceNoAlloc": [_T, _T, _T, _T, _T, _T, _T, c_int],
    "diopiWeightOnlyInt8Linear": [_T, _T, _T, _T, _T],
    "diopiSiluMul": [_T, _T, _T],
    "diopiLinearSiluMul": [_T, _T, _T],
    "diopiLinearRotary": [_T, _T, _T, _T, _T, _T, c_int64, c_int64, c_bool, c_bool],
}

_bound = {}


def fn(name):
    f = _bound.get(name)
    if f is None:
        f = getattr(_native.impl(), name)
        f.argtypes = [c_void_p] + SIGNATURES[name]
        f.restype = c_int
        _bound[name] = f
    return f


def call(name, ctx, *args):
    """Calls diopi<name>(ctx, *args) and raises with diopiGetLastErrorString() on failure,
    which is what the generated wrappers' TORCH_CHECK does (autogen_diopi_wrapper.py:1001)."""
    if runtime.profiler_on:
        # the generated wrapper's RecordBlockCreator dipuRecorder("<interface>") ... dipuRecorder.end()
        # around the call (autogen_diopi_wrapper.py:1013-1016): here a ROCTX range of that name
        rec = runtime.recordStart(name)
        try:
            ret = fn(name)(ctx.ptr, *args)
        finally:
            runtime.recordEnd(rec)
    else:
        ret = fn(name)(ctx.ptr, *args)
    if ret != DIOPI_SUCCESS:
        msg = last_error()
        if "runtime holds the cause" in msg:  # a workspace request failed: the runtime library knows why
            msg += f" [{rt_error()}]"
        raise DiopiError(f"{name} failed, ret = {ret}: {msg}")
