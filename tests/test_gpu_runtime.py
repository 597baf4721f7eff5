"""GPU checks of the host runtime (devapis over HIP, pools, caching allocators, diopirt shim).
Behaviours asserted are those the reference's runtime tests assert (cited per test)."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def rt(pkg):
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return pkg.runtime


def test_device_queries(rt):
    # dipu/tests/python/individual_scripts/test_get_device_properties.py:5-13
    n = rt.getDeviceCount()
    assert n >= 1
    for i in range(n):
        p = rt.getDeviceProperties(i)
        assert p["totalGlobalMem"] >= 256 << 20 and p["multiProcessorCount"] > 0 and p["major"] >= 0
    assert rt.current_device() == 0
    st = rt.getDeviceStatus(0)
    assert 0 < st["freeGlobalMem"] <= st["totalGlobalMem"]
    assert rt.getDriverVersion() > 0 and rt.getRuntimeVersion() > 0
    rt.checkLastError()


def test_streams_events_and_copies(rt):
    # dipu/tests/python/individual_scripts/test_rt_tensor.py:76-128
    s = rt.getStreamFromPool()
    assert s != 0 and s != rt.getDefaultStream()
    seen = {rt.getStreamFromPool() for _ in range(16)}
    assert len(seen) == 8                                  # 8 pooled streams, round robin
    assert rt.getCurrentStream() == rt.getDefaultStream()
    rt.setCurrentStream(s)
    assert rt.getCurrentStream() == s
    rt.setCurrentStream(rt.getDefaultStream())
    n = 1 << 24
    d1, st1 = rt.mallocDevice(n)
    d2, _ = rt.mallocDevice(n)
    assert st1 == "SUCCESS"
    h = rt.mallocHost(n)
    assert rt.isPinnedPtr(h)
    buf = ctypes.create_string_buffer(64)
    assert not rt.isPinnedPtr(ctypes.addressof(buf))      # pageable memory: test_pin_memory.py:9-32
    ctypes.memset(h, 0x5A, n)
    e0, e1 = rt.createEvent(), rt.createEvent()
    rt.recordEvent(e0, s)
    rt.memCopyH2DAsync(s, n, d1, h)
    rt.memCopyD2DAsync(s, n, 0, d2, 0, d1)
    rt.memSetAsync(s, d1, 0, n)
    ctypes.memset(h, 0, n)
    rt.recordEvent(e1, s)
    rt.waitEvent(e1)
    assert rt.getEventStatus(e1) == "READY" and rt.isStreamEmpty(s)
    assert rt.eventElapsedTime(e0, e1) >= 0.0
    out = (ctypes.c_ubyte * 16)()
    rt.memCopyD2H(16, ctypes.addressof(out), d2)
    assert bytes(out) == b"\x5a" * 16
    rt.memCopyD2H(16, ctypes.addressof(out), d1)
    assert bytes(out) == b"\x00" * 16
    s2 = rt.getStreamFromPool()
    rt.streamWaitEvent(s2, e1)
    rt.syncStream(s2)
    rt.destroyEvent(e0)
    rt.destroyEvent(e1)
    assert rt.createEvent() in (e0, e1)                    # events come back from the pool
    rt.freeDevice(d1)
    rt.freeDevice(d2)
    rt.freeHost(h)
    rt.syncDevice()


def test_malloc_device_reports_nomem_without_throwing(rt):
    # deviceapis contract: throwExcepion=false returns ERR_NOMEM and clears the error
    p, status = rt.mallocDevice(1 << 50, throw_on_oom=False)
    assert status == "ERR_NOMEM" and p == 0
    rt.checkLastError()
    with pytest.raises(rt.RuntimeError_):
        rt.mallocDevice(1 << 50, throw_on_oom=True)
    rt.checkLastError() if False else None


def test_caching_allocator_on_device(rt):
    # dipu/tests/python/individual_scripts/test_memory_stats.py:29-45, test_allocator.py:24-74
    base = rt.cachingStats()["allocated_bytes"]
    ptrs, want = [], 0
    for n in list(range(1, 32768, 997)) + [1 << 20, (1 << 20) + 1, 64 << 20]:
        p = rt.cachingMalloc(n)
        assert p % 512 == 0
        ptrs.append(p)
        want += rt.roundSize(n)
    st = rt.cachingStats()
    assert st["allocated_bytes"] - base >= want and st["reserved_bytes"] >= st["allocated_bytes"]
    # the memory is real: fill one block and read it back
    rt.memSetAsync(0, ptrs[-1], 0x11, 64 << 20)
    rt.syncDevice()
    out = (ctypes.c_ubyte * 8)()
    rt.memCopyD2H(8, ctypes.addressof(out), ptrs[-1] + (64 << 20) - 8)
    assert bytes(out) == b"\x11" * 8
    for p in ptrs:
        rt.cachingFree(p)
    assert rt.cachingStats()["allocated_bytes"] == base
    q = rt.cachingMalloc(64 << 20)
    assert q == ptrs[-1]                                   # served from the cache
    rt.cachingFree(q)
    rt.cachingEmptyCache()
    assert rt.cachingStats()["reserved_bytes"] == rt.cachingStats()["allocated_bytes"] or base > 0
    hp = rt.cachingHostMalloc(1000)
    assert rt.isPinnedPtr(hp)
    rt.cachingHostRecordStream(hp, rt.getDefaultStream())
    rt.cachingHostFree(hp)
    rt.syncDevice()
    assert rt.cachingHostMalloc(1024) == hp                # power-of-two block reused after its event


def test_caching_allocator_history_on_device(rt):
    # recordHistory / trace of the TORCH allocator: DIPUCachingDeviceAllocator.cpp:555-566, 1017-1027
    rt.cachingEmptyCache()
    rt.cachingRecordHistory(True, 16)
    stream = rt.getDefaultStream()
    p = rt.cachingMalloc(48 << 20, stream)
    rt.cachingFree(p)
    rt.cachingEmptyCache()
    steps = [(e["action"], e["addr"], e["size"], e["stream"]) for e in rt.cachingTrace()]
    rt.cachingRecordHistory(False)
    assert steps == [("SEGMENT_ALLOC", p, 48 << 20, stream), ("ALLOC", p, 48 << 20, stream),
                     ("FREE_REQUESTED", p, 48 << 20, stream), ("FREE_COMPLETED", p, 48 << 20, stream),
                     ("SEGMENT_FREE", p, 48 << 20, stream)]
    assert rt.cachingTrace() == []


def test_context_workspace_lifetime(pkg, ops, dev):
    # workspace requested by the impl library lives until the context closes
    # (diopirt_impl.h:19-26), then returns to the caching allocator
    x = torch.randn(64, 48, device=dev).t()                # non-contiguous -> softmax makes a dense copy
    out = torch.empty(48, 64, device=dev)
    with pkg.diopi.Context() as ctx:
        ho, po = pkg.diopi.handle(out)
        hx, px = pkg.diopi.handle(x)
        pkg.diopi.call("diopiSoftmax", ctx, po, px, 1)
        n, b = ctx.workspace()
        assert n >= 1 and b >= 48 * 64 * 4
        ctx.reset()
        assert ctx.workspace() == (0, 0)
    torch.cuda.synchronize()
    assert torch.allclose(out.cpu(), torch.softmax(x.cpu(), 1), atol=1e-6)


def test_errors_are_reported_not_thrown(pkg, ops, dev):
    a = torch.randn(4, 5, device=dev)
    b = torch.randn(4, 6, device=dev)
    with pytest.raises(pkg.diopi.DiopiError, match="broadcast"):
        ops.add(a, b, out=torch.empty(4, 5, device=dev))
    with pytest.raises(pkg.diopi.DiopiError, match="inner dims"):
        ops.mm(a, b, out=torch.empty(4, 6, device=dev))
    with pytest.raises(pkg.diopi.DiopiError, match="host"):
        ops.add(a, torch.randn(4, 5), out=torch.empty(4, 5, device=dev))


@pytest.mark.parametrize("algorithm", ["BF", "BS"])
def test_other_caching_algorithms_on_device_in_a_fresh_process(pkg, algorithm):
    """DIPU_DEVICE_MEMCACHING_ALGORITHM is read once per process (dipu/torch_dipu/csrc_dipu/base/environ.hpp:88-92),
    so the BF and BS allocators each get a process of their own: accounting invariant of test_memory_stats.py:29-45, real memory,
    reuse after the stream's work is done, workspace of an op (a transposed GEMM operand) served by it."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = r'''
import ctypes, sys
sys.path.insert(0, %r)
import torch
from __graft_entry__ import load_package
pkg = load_package(); rt = pkg.runtime; ops = pkg.ops
ptrs, want = [], 0
for n in list(range(1, 32768, 997)) + [1 << 20, (1 << 20) + 1, 64 << 20]:
    p = rt.cachingMalloc(n); assert p %% 512 == 0
    ptrs.append(p); want += ((n - 1) | 511) + 1
st = rt.cachingStats()
assert st["allocated_bytes"] == want and st["reserved_bytes"] >= want, st
rt.memSetAsync(0, ptrs[-1], 0x22, 64 << 20); rt.syncDevice()
out = (ctypes.c_ubyte * 8)(); rt.memCopyD2H(8, ctypes.addressof(out), ptrs[-1] + (64 << 20) - 8)
assert bytes(out) == b"\x22" * 8
for p in ptrs: rt.cachingFree(p)
rt.syncDevice()
assert rt.cachingStats()["allocated_bytes"] == 0
q = rt.cachingMalloc(64 << 20); assert q == ptrs[-1], "not served from the cache"
rt.cachingFree(q)
dev = torch.device("cuda:0")
a = torch.randn(300, 200, device=dev).bfloat16(); b = torch.randn(200, 136, device=dev).bfloat16()
got = ops.mm(a, b).float().cpu(); ref = a.float().cpu() @ b.float().cpu()
assert float((got - ref).abs().max()) < 0.5
rt.syncDevice(); rt.cachingEmptyCache()
assert rt.cachingStats()["reserved_bytes"] == 0
print("allocator ok")
''' % root
    env = dict(os.environ, DIPU_DEVICE_MEMCACHING_ALGORITHM=algorithm)
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300, env=env)
    assert out.returncode == 0 and "allocator ok" in out.stdout, out.stderr[-2000:]


def test_torch_algorithm_with_expandable_segments_on_device_in_a_fresh_process(pkg):
    """DIPU_TORCH_ALLOCATOR_CONF=expandable_segments:True (DIPUCachingDeviceAllocator.cpp:1086-1215) over HIP virtual
    memory: blocks are contiguous in one growing range, a large request is assembled from freed small ones without
    new memory, contents survive, empty_cache gives everything back, an op's workspace is served by it."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = r"""
import ctypes, sys
sys.path.insert(0, %r)
import torch
from __graft_entry__ import load_package
pkg = load_package(); rt = pkg.runtime; ops = pkg.ops
MiB = 1 << 20
ps = [rt.cachingMalloc(18 * MiB) for _ in range(10)]
assert ps == [ps[0] + i * 18 * MiB for i in range(10)], ps
st = rt.cachingStats()
assert st["reserved_bytes"] == 180 * MiB and st["segments"] == 1 and st["allocated_bytes"] == 180 * MiB, st
for i, p in enumerate(ps): rt.memSetAsync(0, p, 0x30 + i, 18 * MiB)
rt.syncDevice()
for p in ps: rt.cachingFree(p)
big = rt.cachingMalloc(170 * MiB)
assert big == ps[0]
st = rt.cachingStats()
assert st["reserved_bytes"] == 180 * MiB and st["num_device_malloc"] == 0, st
out = (ctypes.c_ubyte * 4)()
for i in (0, 3, 9):
    rt.memCopyD2H(4, ctypes.addressof(out), big + i * 18 * MiB + 12345)
    assert bytes(out) == bytes([0x30 + i]) * 4, (i, bytes(out))
small = rt.cachingMalloc(1000)
rt.cachingFree(big)
rt.cachingEmptyCache()
st = rt.cachingStats()
assert st["reserved_bytes"] == 2 * MiB and st["segments"] == 1, st   # only the small pool's range is left
again = rt.cachingMalloc(170 * MiB)
rt.memSetAsync(0, again, 0x11, 170 * MiB); rt.syncDevice()
rt.cachingFree(again); rt.cachingFree(small)
dev = torch.device("cuda:0")
a = torch.randn(300, 200, device=dev).bfloat16(); b = torch.randn(200, 136, device=dev).bfloat16()
got = ops.mm(a, b).float().cpu(); ref = a.float().cpu() @ b.float().cpu()
assert float((got - ref).abs().max()) < 0.5
rt.syncDevice(); rt.cachingEmptyCache()
st = rt.cachingStats()
assert st["reserved_bytes"] == 0 and st["segments"] == 0, st
print("allocator ok")
""" % root
    env = dict(os.environ, DIPU_TORCH_ALLOCATOR_CONF="expandable_segments:True")
    env.pop("DIPU_DEVICE_MEMCACHING_ALGORITHM", None)
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300, env=env)
    assert out.returncode == 0 and "allocator ok" in out.stdout, out.stderr[-2000:]


def test_expandable_segment_over_hip_virtual_memory(rt):
    """The vendor half of expandable segments (runtime/core/allocator/ExpandableSegment.h:114-136): map backs whole
    segments, the memory is real and keeps its contents while neighbours come and go, unmap releases only the
    segments entirely inside the range, misuse raises."""
    MiB = 1 << 20
    seg = rt.ExpandableSegment(2 * MiB)
    try:
        base, reserved, mapped = seg.info()
        assert base and reserved >= rt.getDeviceProperties(0)["totalGlobalMem"] and mapped == 0
        assert seg.map(0, 5 * MiB) == (0, 6 * MiB)              # three segments cover 5 MiB
        assert seg.info()[2] == 6 * MiB
        rt.memSetAsync(0, base, 0x5a, 6 * MiB)
        rt.syncDevice()
        out = (ctypes.c_ubyte * 8)()
        rt.memCopyD2H(8, ctypes.addressof(out), base + 6 * MiB - 8)
        assert bytes(out) == b"\x5a" * 8
        assert seg.unmap(1 * MiB, 4 * MiB) == (2 * MiB, 2 * MiB)   # only the middle segment lies inside [1, 5) MiB
        assert seg.info()[2] == 4 * MiB
        assert seg.unmap(3 * MiB, 512) == (3 * MiB, 0)              # nothing entirely inside
        assert seg.map(2 * MiB, 2 * MiB) == (2 * MiB, 2 * MiB)      # the hole is filled again
        rt.memCopyD2H(8, ctypes.addressof(out), base + 8)           # the first segment kept its contents
        assert bytes(out) == b"\x5a" * 8
        assert seg.map(6 * MiB, 1) == (6 * MiB, 2 * MiB)            # grows at the end
        with pytest.raises(RuntimeError, match="already mapped"):
            seg.map(0, 2 * MiB)
        with pytest.raises(RuntimeError, match="segment boundary"):
            seg.map(8 * MiB + 4096, 2 * MiB)
        assert seg.unmap(0, 8 * MiB) == (0, 8 * MiB) and seg.info()[2] == 0
    finally:
        seg.close()
    with pytest.raises(RuntimeError, match="granularity"):
        rt.ExpandableSegment(3000)


def test_ops_emit_roctx_ranges_while_the_profiler_is_on(pkg, ops, dev):
    """devapis::enableProfiler switches named ranges on around every op call, as the generated wrappers'
    RecordBlockCreator does (dipu/scripts/autogen_diopi_wrapper/autogen_diopi_wrapper.py:1013-1016), and on a ROCm
    machine they reach the ROCTX library (what rocprofv3 --marker-trace reads)."""
    rt = pkg.runtime
    a = torch.randn(64, 64, device=dev)
    s0, e0, _ = rt.profilerCounts()
    ops.add(a, a)
    assert rt.profilerCounts()[:2] == (s0, e0)              # off: nothing recorded
    rt.enableProfiler("")
    try:
        ops.add(a, a)
        ops.softmax(a, -1)
        with pytest.raises(pkg.diopi.DiopiError):
            ops.mm(a, torch.randn(3, 3, device=dev), out=torch.empty(64, 3, device=dev))   # a failing op still ends its range
        s1, e1, bound = rt.profilerCounts()
        assert (s1 - s0, e1 - e0) == (3, 3)
        assert bound, "no ROCTX library could be bound on a ROCm machine"
    finally:
        rt.disableProfiler()
    ops.add(a, a)
    assert rt.profilerCounts()[:2] == (s1, e1)
    torch.cuda.synchronize()


def test_allocator_metrics_through_the_caching_allocator(pkg, dev):
    """dipu/tests/python/individual_scripts/test_metrics.py:41-68: 100 allocations of random size show up as 100 more
    entries of allocator_size{type="caching", device, method="allocate"} and at least their bytes in its sum."""
    import random
    rt = pkg.runtime
    rnd = random.Random(0)
    d = str(rt.current_device())
    key = lambda name, **kw: (name, frozenset({("type", "caching"), ("device", d)} | set(kw.items())))
    p = rt.cachingMalloc(1000)                              # preheat
    before = rt.metrics()
    sizes = [rnd.randrange(1, 100000) for _ in range(100)]
    ptrs = [rt.cachingMalloc(n) for n in sizes]
    after = rt.metrics()
    count = after[key("allocator_size_count", method="allocate")] - before[key("allocator_size_count", method="allocate")]
    total = after[key("allocator_size_sum", method="allocate")] - before[key("allocator_size_sum", method="allocate")]
    assert count == 100 and total >= sum(sizes)
    for q in ptrs + [p]:
        rt.cachingFree(q)
    done = rt.metrics()
    assert done[key("allocator_size_count", method="deallocate")] - before.get(key("allocator_size_count", method="deallocate"), 0) == 101
    assert done[key("allocator_event_count", method="deallocate", event="unexpected")] == before[key("allocator_event_count", method="deallocate", event="unexpected")]
    # the raw vendor calls underneath are counted under type "device"
    dkey = ("allocator_size_count", frozenset({("type", "device"), ("device", d), ("method", "allocate")}))
    assert done[dkey] >= 1
