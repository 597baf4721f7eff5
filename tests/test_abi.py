"""CPU-side checks of the drop-in boundary: both libraries load, every symbol declared in
include/ is exported, the ctypes signature table covers every declared DIOPI function, and
the shim's tensor struct matches the header layout. No compute is launched."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INC = os.path.join(ROOT, "include")


def _declared(path, macro):
    text = open(path).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.findall(macro + r"\s+[\w\s\*]+?\b(\w+)\s*\(", text)


def test_impl_exports_every_declared_function(pkg):
    lib = pkg._native.impl()
    names = _declared(os.path.join(INC, "diopi", "functions.h"), "DIOPI_API") + \
        _declared(os.path.join(INC, "diopi", "functions_ext.h"), "DIOPI_API")
    assert len(names) >= 40
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing
    unbound = [n for n in names if n != "diopiGetLastErrorString" and n not in pkg.diopi.SIGNATURES]
    assert not unbound, unbound


def test_runtime_exports_callbacks_and_facade(pkg):
    rt = pkg._native.runtime()
    cb = _declared(os.path.join(INC, "diopi", "diopirt.h"), "DIOPI_RT_API")
    assert "diopiRequireTensor" in cb and "diopiGetStream" in cb
    fac = _declared(os.path.join(INC, "dipu_amd", "runtime.h"), "DIPU_AMD_API")
    assert len(fac) >= 60
    missing = [n for n in cb + fac if not hasattr(rt, n)]
    assert not missing, missing


def test_impl_library_has_no_torch_dependency(pkg):
    # the boundary is plain C: the impl library must not link libtorch / libc10
    import subprocess
    out = subprocess.run(["ldd", pkg._native.IMPL_PATH], capture_output=True, text=True).stdout
    assert "libtorch" not in out and "libc10" not in out


def test_tensor_struct_layout_matches_header(pkg):
    d = pkg.diopi.dipuAmdTensor
    assert d.data.offset == 0 and d.ndim.offset == 8
    assert d.shape.offset == 16 and d.stride.offset == 16 + 64
    assert d.dtype.offset == 144 and d.device.offset == 148 and d.device_index.offset == 152
    assert d.storage_offset.offset == 160 and d.storage_ptr.offset == 168 and d.storage_nbytes.offset == 176
    assert ctypes.sizeof(d) == 184
    s = pkg.diopi.diopiScalar_t
    assert ctypes.sizeof(s) == 16 and s.u.offset == 8


def test_scalar_marshalling(pkg):
    # diopi_helper.cpp:74-97: bool/int -> int64 payload, float -> float64 payload
    s = pkg.diopi.scalar(3)
    assert (s.stype, s.ival) == (6, 3)
    s = pkg.diopi.scalar(True)
    assert (s.stype, s.ival) == (6, 1)
    s = pkg.diopi.scalar(0.5)
    assert (s.stype, s.fval) == (10, 0.5)
    with pytest.raises(TypeError):
        pkg.diopi.scalar("x")


def test_missing_library_fails_loudly(pkg, monkeypatch):
    monkeypatch.setattr(pkg._native, "_impl", None)
    monkeypatch.setattr(pkg._native, "IMPL_PATH", "/nonexistent/libdiopi_impl.so")
    with pytest.raises(pkg._native.NativeLibraryMissing):
        pkg._native.impl()


def test_version_and_error_string(pkg):
    rt = pkg._native.runtime()
    rt.diopiGetVersion.restype = ctypes.c_char_p
    assert rt.diopiGetVersion().startswith(b"DIOPI Version: ")
    assert isinstance(pkg.diopi.last_error(), str)


def test_profiler_hooks_count_ranges_only_while_enabled(pkg):
    """devapis::enableProfiler / disableProfiler and the diopiRecordStart/End pair
    (dipu/torch_dipu/csrc_dipu/runtime/device/profilerapis.h:12-14, diopirt/diopirt_impl.cpp:224-237):
    disabled -> null record, nothing counted; enabled -> one range started and ended per pair."""
    rt = pkg.runtime
    rt.disableProfiler()
    s0, e0, _ = rt.profilerCounts()
    rec = rt.recordStart("idle")
    assert not rec.value
    rt.recordEnd(rec)
    assert rt.profilerCounts()[:2] == (s0, e0)
    rt.enableProfiler("/tmp/unused")
    try:
        recs = [rt.recordStart(f"diopiOp{i}") for i in range(3)]
        assert all(r.value for r in recs)
        s1, e1, _ = rt.profilerCounts()
        assert (s1 - s0, e1 - e0) == (3, 0)
        for r in reversed(recs):
            rt.recordEnd(r)
            assert not r.value
        s2, e2, _ = rt.profilerCounts()
        assert (s2 - s0, e2 - e0) == (3, 3)
    finally:
        rt.disableProfiler()


def test_generator_state_round_trip(pkg):
    """The diopiGenerator* runtime callbacks with the CUDA vendor's state layout
    (dipu/torch_dipu/csrc_dipu/vendor/cuda/CudaGeneratorImpl.cpp:17-76; callbacks diopirt_impl.cpp:175-226): 16 host
    bytes = seed then Philox offset, an 8-byte state sets offset 0, offsets must be multiples of 4."""
    import struct
    import torch
    d = pkg.diopi
    g = d.Generator()
    try:
        assert g.seed_and_offset() == (67280421310721, 0)          # torch's default seed
        g.set_seed_and_offset(1234, 8)
        assert g.seed_and_offset() == (1234, 8)
        st = g.get_state()
        assert st.dtype == torch.uint8 and st.numel() == 16
        assert struct.unpack("<QQ", bytes(st.tolist())) == (1234, 8)
        h = d.Generator()
        h.set_state(st)
        assert h.seed_and_offset() == (1234, 8)
        h.set_state(torch.tensor(list(struct.pack("<Q", 99)), dtype=torch.uint8))   # seed only
        assert h.seed_and_offset() == (99, 0)
        with pytest.raises(d.DiopiError):
            g.set_seed_and_offset(1, 6)                               # offset not a multiple of 4
        with pytest.raises(d.DiopiError):
            h.set_state(torch.zeros(12, dtype=torch.uint8))           # wrong size
        h.close()
    finally:
        g.close()


def test_allocator_metrics_labels_events_and_histogram(pkg):
    """Label sets and event rules of dipu/torch_dipu/csrc_dipu/runtime/core/allocator/allocator_metrics.h:17-120, fed
    through the same call the allocators make (no device needed)."""
    rt = pkg.runtime
    assert rt.metricsEnable() is True                       # on by default (metrics/metrics.cpp:5-11)
    t, dev = "unit_test", 3
    key = lambda name, **kw: (name, frozenset({("type", t), ("device", str(dev))} | set(kw.items())))
    rt.metricsRecord(t, dev, 0x1000, 16)                    # <= 2^4: first bucket
    rt.metricsRecord(t, dev, 0x2000, 17)                    # second bucket
    rt.metricsRecord(t, dev, 0x3000, 1 << 31)               # last finite bucket
    rt.metricsRecord(t, dev, 0x4000, (1 << 31) + 1)         # +Inf
    rt.metricsRecord(t, dev, 0x5000, 0)                     # size 0: ignored
    rt.metricsRecord(t, dev, 0, 64)                         # null pointer
    rt.metricsRecord(t, dev, 0x1000, 32)                    # already live
    m = rt.metrics()
    assert m[key("allocator_event_count", method="allocate", event="nullptr")] == 1
    assert m[key("allocator_event_count", method="allocate", event="duplicated")] == 1
    assert m[key("allocator_size_bucket", method="allocate", le="16")] == 1
    assert m[key("allocator_size_bucket", method="allocate", le="32")] == 2
    assert m[key("allocator_size_bucket", method="allocate", le=str(1 << 30))] == 2
    assert m[key("allocator_size_bucket", method="allocate", le=str(1 << 31))] == 3
    assert m[key("allocator_size_bucket", method="allocate", le="+Inf")] == 4
    assert m[key("allocator_size_count", method="allocate")] == 4
    assert m[key("allocator_size_sum", method="allocate")] == 16 + 17 + (1 << 31) + (1 << 31) + 1
    rt.metricsRecord(t, dev, 0x2000, deallocate=True)       # records the size it was allocated with
    rt.metricsRecord(t, dev, 0x2000, deallocate=True)       # no longer live
    rt.metricsRecord(t, dev, 0, deallocate=True)
    m = rt.metrics()
    assert m[key("allocator_size_sum", method="deallocate")] == 17 and m[key("allocator_size_count", method="deallocate")] == 1
    assert m[key("allocator_event_count", method="deallocate", event="unexpected")] == 1
    assert m[key("allocator_event_count", method="deallocate", event="nullptr")] == 1
    # switched off nothing is recorded
    assert rt.metricsEnable(False) is False
    rt.metricsRecord(t, dev, 0x9000, 64)
    assert rt.metrics()[key("allocator_size_count", method="allocate")] == 4
    assert rt.metricsEnable(True) is True


def test_generated_gemm_loop_is_current(tmp_path):
    """The committed K loop of the 4-wave GEMM kernel is what its generator writes."""
    import subprocess
    import sys
    d = os.path.join(ROOT, "deeplink.framework_amd", "csrc", "diopi_impl")
    out = tmp_path / "loop.inc"
    subprocess.run([sys.executable, os.path.join(d, "gen_gemm_loop_4wave.py"), str(out)], check=True)
    assert out.read_text() == open(os.path.join(d, "gemm_loop_4wave.inc")).read()
