"""Op adapter: the Python mirror of torch_dipu's generated wrappers for the transformer
inference path. Each function does what the corresponding `dipu_<op>` wrapper does in
DIPU (dipu/scripts/autogen_diopi_wrapper/diopi_wrapper_template.py:100-141):

  1. infer and allocate the output (broadcast shape + promoted dtype, as
     dipu/torch_dipu/csrc_dipu/aten/ops/DIPUOpInferrer.cpp:62-245 does),
  2. open a diopiContext on the current stream,
  3. marshal tensors / scalars / sizes and call the diopi* entry point,
  4. raise on any return code other than diopiSuccess.

Nothing here computes: a missing libdiopi_impl.so raises, there is no torch fallback.
Names follow the aten op (or, for the ext ops, the lightllm op names the reference's
dicp/dicp/vendor/AscendGraph/ext_ops.py registers).
"""
import ctypes
from ctypes import byref, c_void_p

import torch

from . import diopi
from .diopi import Context, call, handle, scalar


def _is_number(x):
    return isinstance(x, (bool, int, float))


def _peel_cpu_scalar(x):
    """CPU 0-dim tensors are passed as scalars (dipu/torch_dipu/csrc_dipu/aten/ops/OpUtils.hpp:324-326)."""
    if isinstance(x, torch.Tensor) and x.device.type == "cpu" and x.dim() == 0:
        return x.item()
    return x


def _binary_out(a, b, out):
    if out is not None:
        return out
    shape = torch.broadcast_shapes(a.shape, b.shape) if isinstance(b, torch.Tensor) else a.shape
    dtype = torch.result_type(a, b)
    return torch.empty(shape, dtype=dtype, device=a.device)


_scope = None


class WorkspaceScope:
    """One diopiContext shared by every op called inside `with scope:`; the workspace those ops request stays
    allocated until close(), as a context keeps its arrays until it is destroyed (diopirt_impl.h:19-26). For work
    recorded into a HIP graph: the graph's kernels keep the workspace addresses they were recorded with, so the scope
    is created on the capturing stream and closed only after the last replay. Recording may not allocate device
    memory: run the same calls under a scope on that stream beforehand, and again until a pass leaves the
    allocator's num_device_malloc unchanged; the recording then finds every block in the cache."""

    def __init__(self, stream=None):
        self.ctx = Context(stream)

    def __enter__(self):
        global _scope
        self._outer, _scope = _scope, self
        return self

    def __exit__(self, *exc):
        global _scope
        _scope = self._outer

    def close(self):
        self.ctx.close()


def _call(name, *args, stream=None):
    if _scope is not None and stream is None:
        call(name, _scope.ctx, *args)
        return
    with Context(stream) as ctx:
        call(name, ctx, *args)


# ------------------------------------------------------------------ arithmetic
def add(self, other, *, alpha=1, out=None):
    """aten::add.Tensor / add.Scalar -> diopiAdd / diopiAddScalar (diopi_functions.yaml:31-63)."""
    other = _peel_cpu_scalar(other)
    out = _binary_out(self, other, out)
    ho, po = handle(out)
    hs, ps = handle(self)
    al = scalar(alpha)
    if _is_number(other):
        sc = scalar(other)
        _call("diopiAddScalar", po, ps, byref(sc), byref(al))
    else:
        hb, pb = handle(other)
        _call("diopiAdd", po, ps, pb, byref(al))
    return out


def add_(self, other, *, alpha=1):
    other = _peel_cpu_scalar(other)
    hs, ps = handle(self)
    al = scalar(alpha)
    if _is_number(other):
        sc = scalar(other)
        _call("diopiAddInpScalar", ps, byref(sc), byref(al))
    else:
        hb, pb = handle(other)
        _call("diopiAddInp", ps, pb, byref(al))
    return self


def sub(self, other, *, alpha=1, out=None):
    other = _peel_cpu_scalar(other)
    out = _binary_out(self, other, out)
    ho, po = handle(out)
    hs, ps = handle(self)
    al = scalar(alpha)
    if _is_number(other):
        sc = scalar(other)
        _call("diopiSubScalar", po, ps, byref(sc), byref(al))
    else:
        hb, pb = handle(other)
        _call("diopiSub", po, ps, pb, byref(al))
    return out


def mul(self, other, *, out=None):
    """aten::mul.Tensor / mul.Scalar -> diopiMul / diopiMulScalar (diopi_functions.yaml:159-196)."""
    other = _peel_cpu_scalar(other)
    out = _binary_out(self, other, out)
    ho, po = handle(out)
    hs, ps = handle(self)
    if _is_number(other):
        sc = scalar(other)
        _call("diopiMulScalar", po, ps, byref(sc))
    else:
        hb, pb = handle(other)
        _call("diopiMul", po, ps, pb)
    return out


def mul_(self, other):
    other = _peel_cpu_scalar(other)
    hs, ps = handle(self)
    if _is_number(other):
        sc = scalar(other)
        _call("diopiMulInpScalar", ps, byref(sc))
    else:
        hb, pb = handle(other)
        _call("diopiMulInp", ps, pb)
    return self


def div(self, other, *, rounding_mode=None, out=None):
    other = _peel_cpu_scalar(other)
    if out is None:
        shape = torch.broadcast_shapes(self.shape, other.shape) if isinstance(other, torch.Tensor) else self.shape
        dtype = torch.result_type(self, other)
        if rounding_mode is None and not dtype.is_floating_point:
            dtype = torch.get_default_dtype()
        out = torch.empty(shape, dtype=dtype, device=self.device)
    ho, po = handle(out)
    hs, ps = handle(self)
    mode = diopi.ROUND_MODE[rounding_mode]
    if _is_number(other):
        sc = scalar(other)
        _call("diopiDivScalar", po, ps, byref(sc), mode)
    else:
        hb, pb = handle(other)
        _call("diopiDiv", po, ps, pb, mode)
    return out


def _unary(name, self, out):
    if out is None:
        out = torch.empty_like(self, memory_format=torch.contiguous_format)
    ho, po = handle(out)
    hs, ps = handle(self)
    _call(name, po, ps)
    return out


def silu(self, *, out=None):
    """aten::silu -> diopiSilu (diopi_functions.yaml:1767-1775)."""
    return _unary("diopiSilu", self, out)


def silu_(self):
    hs, ps = handle(self)
    _call("diopiSiluInp", ps)
    return self


def sigmoid(self, *, out=None):
    return _unary("diopiSigmoid", self, out)


def rsqrt(self, *, out=None):
    return _unary("diopiRsqrt", self, out)


def neg(self, *, out=None):
    return _unary("diopiNeg", self, out)


def sin(self, *, out=None):
    return _unary("diopiSin", self, out)


def cos(self, *, out=None):
    return _unary("diopiCos", self, out)


def exp(self, *, out=None):
    return _unary("diopiExp", self, out)


def pow(self, exponent, *, out=None):
    """aten::pow.Tensor_Scalar -> diopiPow (diopi_functions.yaml:1306-1318)."""
    if out is None:
        dtype = torch.result_type(self, exponent)
        out = torch.empty(self.shape, dtype=dtype, device=self.device)
    ho, po = handle(out)
    hs, ps = handle(self)
    sc = scalar(exponent)
    _call("diopiPow", po, ps, byref(sc))
    return out


def fill_(self, value):
    hs, ps = handle(self)
    sc = scalar(value)
    _call("diopiFill", ps, byref(sc))
    return self


def silu_mul(gate, up, *, out=None):
    """silu(gate) * up in one pass (backend extension; see functions_ext.h)."""
    if out is None:
        out = torch.empty_like(gate, memory_format=torch.contiguous_format)
    ho, po = handle(out)
    hg, pg = handle(gate)
    hu, pu = handle(up)
    _call("diopiSiluMul", po, pg, pu)
    return out


def interleave_gate_up(w_gate, w_up):
    """The [2F, K] weight diopiLinearSiluMul expects: w_gate and w_up [F, K] interleaved in blocks of 32 rows
    (a load-time permutation of the checkpoint)."""
    f, k = w_gate.shape
    assert w_up.shape == (f, k) and f % 32 == 0
    return torch.stack([w_gate.reshape(f // 32, 32, k), w_up.reshape(f // 32, 32, k)], dim=1).reshape(2 * f, k).contiguous()


def linear_silu_mul(input, weight_gate_up, *, out=None):
    """silu(input @ w_gate^T) * (input @ w_up^T) in one launch (backend extension; see functions_ext.h).
    weight_gate_up = interleave_gate_up(w_gate, w_up)."""
    f = weight_gate_up.shape[0] // 2
    if out is None:
        out = torch.empty(*input.shape[:-1], f, dtype=input.dtype, device=input.device)
    ho, po = handle(out)
    hi, pi = handle(input)
    hw, pw = handle(weight_gate_up)
    _call("diopiLinearSiluMul", po, pi, pw)
    return out


def interleave_rotary_rows(w, head_dim):
    """Rows of a q or k projection weight [heads * head_dim, K] reordered inside every head from the half-split
    rotary convention to the interleaved one: row 2 i <- row i, row 2 i + 1 <- row i + head_dim / 2. q . k does
    not change when both are permuted this way, so attention is unaffected (a load-time permutation)."""
    n, k = w.shape
    assert n % head_dim == 0 and head_dim % 2 == 0
    return w.reshape(n // head_dim, 2, head_dim // 2, k).transpose(1, 2).reshape(n, k).contiguous()


def linear_rotary(input, weight, cos, sin, rotary_cols, head_dim, bias=None, *, conj=False, interleaved=True, out=None):
    """input @ weight^T (+ bias) with the rotary embedding applied to the first rotary_cols output columns
    (backend extension; see functions_ext.h). cos / sin: [rows, head_dim / 2]."""
    if out is None:
        out = torch.empty(*input.shape[:-1], weight.shape[0], dtype=input.dtype, device=input.device)
    ho, po = handle(out)
    hi, pi = handle(input)
    hw, pw = handle(weight)
    hb, pb = handle(bias)
    hc, pc = handle(cos)
    hs, ps = handle(sin)
    _call("diopiLinearRotary", po, pi, pw, pb, pc, ps, int(rotary_cols), int(head_dim), bool(conj), bool(interleaved))
    return out


# ------------------------------------------------------------------ reductions
def softmax(self, dim, *, out=None):
    """aten::_softmax.out -> diopiSoftmax (diopi_functions.yaml:1290-1292)."""
    if out is None:
        out = torch.empty_like(self, memory_format=torch.contiguous_format)
    ho, po = handle(out)
    hs, ps = handle(self)
    _call("diopiSoftmax", po, ps, int(dim))
    return out


def mean(self, dim, keepdim=False, *, out=None):
    """aten::mean.dim -> diopiMean (diopi_functions.yaml:830-842)."""
    dims = [dim] if isinstance(dim, int) else list(dim)
    dims = [d % self.dim() for d in dims]
    if out is None:
        shape = [(1 if i in dims else n) for i, n in enumerate(self.shape) if keepdim or i not in dims]
        out = torch.empty(shape, dtype=self.dtype, device=self.device)
    ho, po = handle(out)
    hs, ps = handle(self)
    sz = diopi.size(dims)
    _call("diopiMean", po, ps, sz)
    return out


# ------------------------------------------------------------------ movement
def copy_(self, src):
    """aten::copy_ on-device part -> diopiCopyInp(ctx, src, dest) (diopi_functions.yaml:2969-2973)."""
    hs, ps = handle(src)
    hd, pd = handle(self)
    _call("diopiCopyInp", ps, pd)
    return self


def cat(tensors, dim=0, *, out=None):
    tensors = list(tensors)
    if out is None:
        ref = next((t for t in tensors if not (t.dim() == 1 and t.numel() == 0)), tensors[0])  # all legacy-empty: the result is empty
        d = dim % ref.dim()
        shape = list(ref.shape)
        shape[d] = sum(t.shape[d] for t in tensors if not (t.dim() == 1 and t.numel() == 0))
        dtype = ref.dtype
        for t in tensors:
            dtype = torch.promote_types(dtype, t.dtype)
        out = torch.empty(shape, dtype=dtype, device=ref.device)
    hs = [handle(t) for t in tensors]
    arr = (c_void_p * len(hs))(*[p for _, p in hs])
    ho, po = handle(out)
    _call("diopiCat", po, arr, len(hs), int(dim))
    return out


def index_put_(self, indices, values, accumulate=False):
    """aten::_index_put_impl_ -> diopiIndexPutInp (diopi_functions.yaml:2370-2382)."""
    hs = [handle(t) for t in indices]
    arr = (c_void_p * len(hs))(*[p for _, p in hs])
    hd, pd = handle(self)
    hv, pv = handle(values)
    _call("diopiIndexPutInp", pd, pv, arr, len(hs), bool(accumulate))
    return self


# ------------------------------------------------- selection / masks / gathers
def where(condition, self, other, *, out=None):
    """aten::where.self -> diopiWhere (diopi_functions.yaml:1566-1571). Python numbers become
    0-d device tensors, which is what ATen hands the wrapper after its own scalar wrapping."""
    dev = condition.device
    if _is_number(self) and _is_number(other):
        dtype = torch.result_type(torch.tensor(self), torch.tensor(other))
        self, other = torch.tensor(self, dtype=dtype, device=dev), torch.tensor(other, dtype=dtype, device=dev)
    elif _is_number(self):
        self = torch.tensor(self, dtype=other.dtype, device=dev)
    elif _is_number(other):
        other = torch.tensor(other, dtype=self.dtype, device=dev)
    if out is None:
        shape = torch.broadcast_shapes(condition.shape, self.shape, other.shape)
        out = torch.empty(shape, dtype=torch.result_type(self, other), device=dev)
    hc, pc = handle(condition)
    ha, pa = handle(self)
    hb, pb = handle(other)
    ho, po = handle(out)
    _call("diopiWhere", po, pc, pa, pb)
    return out


def masked_fill(self, mask, value, *, out=None):
    """aten::masked_fill.Scalar / .Tensor -> diopiMaskedFillScalar / diopiMaskedFill
    (diopi_functions.yaml:1432-1453); a CPU value tensor is moved to the device first (:1436)."""
    if out is None:
        out = torch.empty(torch.broadcast_shapes(self.shape, mask.shape), dtype=self.dtype, device=self.device)
    ho, po = handle(out)
    hs, ps = handle(self)
    hm, pm = handle(mask)
    if _is_number(value):
        sc = scalar(value)
        _call("diopiMaskedFillScalar", po, ps, pm, byref(sc))
    else:
        hv, pv = handle(value.to(self.device))
        _call("diopiMaskedFill", po, ps, pm, pv)
    return out


def masked_fill_(self, mask, value):
    hs, ps = handle(self)
    hm, pm = handle(mask)
    if _is_number(value):
        sc = scalar(value)
        _call("diopiMaskedFillInpScalar", ps, pm, byref(sc))
    else:
        hv, pv = handle(value.to(self.device))
        _call("diopiMaskedFillInp", ps, pm, pv)
    return self


def tril(self, diagonal=0, *, out=None):
    """aten::tril -> diopiTril (diopi_functions.yaml:1191-1197)."""
    out = torch.empty_like(self) if out is None else out
    ho, po = handle(out)
    hs, ps = handle(self)
    _call("diopiTril", po, ps, int(diagonal))
    return out


def triu(self, diagonal=0, *, out=None):
    """aten::triu -> diopiTriu (diopi_functions.yaml:2505-2516)."""
    out = torch.empty_like(self) if out is None else out
    ho, po = handle(out)
    hs, ps = handle(self)
    _call("diopiTriu", po, ps, int(diagonal))
    return out


def triu_(self, diagonal=0):
    hs, ps = handle(self)
    _call("diopiTriuInp", ps, int(diagonal))
    return self


def arange(start, end=None, step=1, *, dtype=None, device=None, out=None):
    """aten::arange.start_out -> diopiArange (diopi_functions.yaml:2341-2347). The element count is
    ATen's ceil((end - start) / step); the wrapper only sizes `out` itself when it arrives empty."""
    import math
    if end is None:
        start, end = 0, start
    if out is None:
        if dtype is None:
            dtype = torch.get_default_dtype() if any(isinstance(v, float) for v in (start, end, step)) else torch.int64
        out = torch.empty(int(math.ceil((end - start) / step)), dtype=dtype, device=device)
    ho, po = handle(out)
    s0, s1, s2 = scalar(start), scalar(end), scalar(step)
    _call("diopiArange", po, byref(s0), byref(s1), byref(s2))
    return out


def index_select(self, dim, index, *, out=None):
    """aten::index_select -> diopiIndexSelect (diopi_functions.yaml:1926-1933)."""
    if out is None:
        shape = list(self.shape)
        shape[dim % self.dim()] = index.numel()
        out = torch.empty(shape, dtype=self.dtype, device=self.device)
    ho, po = handle(out)
    hs, ps = handle(self)
    hi, pi = handle(index)
    _call("diopiIndexSelect", po, ps, int(dim), pi)
    return out


def gather(self, dim, index, *, out=None):
    """aten::gather.out -> diopiGather (diopi_functions.yaml:1923-1924)."""
    if out is None:
        out = torch.empty(index.shape, dtype=self.dtype, device=self.device)
    ho, po = handle(out)
    hs, ps = handle(self)
    hi, pi = handle(index)
    _call("diopiGather", po, ps, int(dim), pi)
    return out


def _compare(name, self, other, out):
    other = _peel_cpu_scalar(other)
    if out is None:
        shape = torch.broadcast_shapes(self.shape, other.shape) if isinstance(other, torch.Tensor) else self.shape
        out = torch.empty(shape, dtype=torch.bool, device=self.device)
    ho, po = handle(out)
    hs, ps = handle(self)
    if _is_number(other):
        sc = scalar(other)
        _call(f"diopi{name}Scalar", po, ps, byref(sc))
    else:
        hb, pb = handle(other)
        _call(f"diopi{name}", po, ps, pb)
    return out


def eq(self, other, *, out=None):
    """aten::eq.Tensor_out / eq.Scalar_out -> diopiEq / diopiEqScalar (diopi_functions.yaml:409-420)."""
    return _compare("Eq", self, other, out)


def ne(self, other, *, out=None):
    return _compare("Ne", self, other, out)


def lt(self, other, *, out=None):
    return _compare("Lt", self, other, out)


def le(self, other, *, out=None):
    return _compare("Le", self, other, out)


def gt(self, other, *, out=None):
    return _compare("Gt", self, other, out)


def ge(self, other, *, out=None):
    return _compare("Ge", self, other, out)


# ------------------------------------------------------------------ contractions
def mm(self, mat2, *, out=None):
    """aten::mm -> diopiMm (diopi_functions.yaml:1829-1837)."""
    if out is None:
        out = torch.empty((self.shape[0], mat2.shape[1]), dtype=self.dtype, device=self.device)
    ho, po = handle(out)
    ha, pa = handle(self)
    hb, pb = handle(mat2)
    _call("diopiMm", po, pa, pb)
    return out


def bmm(self, mat2, *, out=None):
    """aten::bmm -> diopiBmm (diopi_functions.yaml:1755-1765)."""
    if out is None:
        out = torch.empty((self.shape[0], self.shape[1], mat2.shape[2]), dtype=self.dtype, device=self.device)
    ho, po = handle(out)
    ha, pa = handle(self)
    hb, pb = handle(mat2)
    _call("diopiBmm", po, pa, pb)
    return out


def _matmul_shape(a, b):
    if a.dim() == 1 and b.dim() == 1:
        return ()
    if a.dim() == 1:
        return tuple(b.shape[:-2]) + (b.shape[-1],)
    if b.dim() == 1:
        return tuple(a.shape[:-1])
    batch = torch.broadcast_shapes(a.shape[:-2], b.shape[:-2])
    return tuple(batch) + (a.shape[-2], b.shape[-1])


def matmul(self, other, *, out=None):
    """aten::matmul -> diopiMatmul (diopi_functions.yaml:1852-1893)."""
    if out is None:
        out = torch.empty(_matmul_shape(self, other), dtype=self.dtype, device=self.device)
    ho, po = handle(out)
    ha, pa = handle(self)
    hb, pb = handle(other)
    _call("diopiMatmul", po, pa, pb)
    return out


def addmm(self, mat1, mat2, *, beta=1, alpha=1, out=None):
    """aten::addmm -> diopiAddmm (diopi_functions.yaml:594-597)."""
    if out is None:
        out = torch.empty((mat1.shape[0], mat2.shape[1]), dtype=mat1.dtype, device=mat1.device)
    ho, po = handle(out)
    hi, pi = handle(self)
    ha, pa = handle(mat1)
    hb, pb = handle(mat2)
    sb, sa = scalar(beta), scalar(alpha)
    _call("diopiAddmm", po, pi, pa, pb, byref(sb), byref(sa))
    return out


def baddbmm(self, batch1, batch2, *, beta=1, alpha=1, out=None):
    """aten::baddbmm -> diopiBaddbmm, beta/alpha as doubles (diopi_functions.yaml:1534-1548)."""
    if out is None:
        out = torch.empty((batch1.shape[0], batch1.shape[1], batch2.shape[2]), dtype=batch1.dtype,
                          device=batch1.device)
    ho, po = handle(out)
    hi, pi = handle(self)
    ha, pa = handle(batch1)
    hb, pb = handle(batch2)
    _call("diopiBaddbmm", po, pi, pa, pb, float(beta), float(alpha))
    return out


def linear(input, weight, bias=None, *, out=None):
    """aten::linear -> diopiLinear, weight [N, K] (diopi_functions.yaml:902-909)."""
    if out is None:
        out = torch.empty(tuple(input.shape[:-1]) + (weight.shape[0],), dtype=input.dtype, device=input.device)
    ho, po = handle(out)
    hi, pi = handle(input)
    hw, pw = handle(weight)
    hb, pb = handle(bias)
    _call("diopiLinear", po, pi, pw, pb)
    return out


# ------------------------------------------------------------------ ext ops
def rms_norm(x, weight, eps, *, bias=None, out=None, inv_rms=None):
    """lightllm::rms_norm (ext_ops.py:36-49) -> diopiRMSNorm over the last dim."""
    if out is None:
        out = torch.empty_like(x, memory_format=torch.contiguous_format)
    ho, po = handle(out)
    hr, pr = handle(inv_rms)
    hx, px = handle(x)
    hw, pw = handle(weight)
    hb, pb = handle(bias)
    sz = diopi.size([x.shape[-1]])
    _call("diopiRMSNorm", po, pr, px, sz, pw, pb, float(eps))
    return out


def rotary_emb(x, cos, sin, *, conj=False, interleaved=False, out=None):
    """lightllm::rotary_emb (ext_ops.py:13-33; interleaved form model.py:58-69) -> diopiRotaryEmbedding."""
    if out is None:
        out = torch.empty_like(x, memory_format=torch.contiguous_format)
    ho, po = handle(out)
    hx, px = handle(x)
    hc, pc = handle(cos)
    hs, ps = handle(sin)
    _call("diopiRotaryEmbedding", po, px, pc, ps, bool(conj), bool(interleaved))
    return out


def dest_index_copy_kv(k, dest_loc, out):
    """out[dest_loc[i]] = k[i] -> diopiDestIndexCopyKV (bit-exact scatter into the KV pool)."""
    ho, po = handle(out)
    hk, pk = handle(k)
    hl, pl = handle(dest_loc)
    _call("diopiDestIndexCopyKV", po, pk, pl)
    return out


def dest_index_copy_kv_pair(k, v, dest_loc, out_k, out_v):
    """out_k[dest_loc[i]] = k[i] and out_v[dest_loc[i]] = v[i] in one launch (backend extension, functions_ext.h)."""
    hok, pok = handle(out_k)
    hk, pk = handle(k)
    hov, pov = handle(out_v)
    hv, pv = handle(v)
    hl, pl = handle(dest_loc)
    _call("diopiDestIndexCopyKVPair", pok, pk, pov, pv, pl)
    return out_k, out_v


def token_attention(q, k, attention_out, b_loc, b_start_loc, b_seq_len, max_input_len):
    ho, po = handle(attention_out)
    hq, pq = handle(q)
    hk, pk = handle(k)
    h1, p1 = handle(b_loc)
    h2, p2 = handle(b_start_loc)
    h3, p3 = handle(b_seq_len)
    _call("diopiTokenAttentionInference", po, pq, pk, p1, p2, p3, int(max_input_len))
    return attention_out


def token_softmax_reducev(logics, v, out, b_loc, b_start_loc, b_seq_len, max_input_len, other_kv_index=0):
    ho, po = handle(out)
    hl, pl = handle(logics)
    hv, pv = handle(v)
    h1, p1 = handle(b_loc)
    h2, p2 = handle(b_start_loc)
    h3, p3 = handle(b_seq_len)
    _call("diopiTokenSoftmaxReduceVInference", po, pl, pv, p1, p2, p3, int(max_input_len), int(other_kv_index))
    return out


def token_decode_attention(q, k, v, b_loc, b_start_loc, b_seq_len, max_input_len, *, out=None, no_alloc=False):
    """lightllm::flash_attention_inference (ext_ops.py:90-133) over a paged pool, fused. no_alloc selects the entry
    point whose partial results live in the library's own device array (the caller then passes `out`)."""
    if out is None:
        out = torch.empty_like(q)
    ho, po = handle(out)
    hq, pq = handle(q)
    hk, pk = handle(k)
    hv, pv = handle(v)
    h1, p1 = handle(b_loc)
    h2, p2 = handle(b_start_loc)
    h3, p3 = handle(b_seq_len)
    _call("diopiTokenDecodeAttentionInferenceNoAlloc" if no_alloc else "diopiTokenDecodeAttentionInference",
          po, pq, pk, pv, p1, p2, p3, int(max_input_len))
    return out


def context_attention(q, k, v, b_start_loc, b_seq_len, max_input_len, *, out=None):
    """lightllm::prompt_attention_inference (ext_ops.py:52-87) over packed sequences."""
    if out is None:
        out = torch.empty_like(q)
    ho, po = handle(out)
    hq, pq = handle(q)
    hk, pk = handle(k)
    hv, pv = handle(v)
    h2, p2 = handle(b_start_loc)
    h3, p3 = handle(b_seq_len)
    _call("diopiContextAttentionInference", po, pq, pk, pv, p2, p3, int(max_input_len))
    return out


def weight_only_int8_linear(input, weight, scale, bias=None, *, out=None):
    if out is None:
        out = torch.empty(tuple(input.shape[:-1]) + (weight.shape[0],), dtype=input.dtype, device=input.device)
    ho, po = handle(out)
    hi, pi = handle(input)
    hw, pw = handle(weight)
    hs, ps = handle(scale)
    hb, pb = handle(bias)
    _call("diopiWeightOnlyInt8Linear", po, pi, pw, ps, pb)
    return out
