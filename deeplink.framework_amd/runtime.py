"""Python facade of libdipu_amd_rt.so (include/dipu_amd/runtime.h): the devapis functions,
stream/event pools and caching allocators, with names following the contract in
dipu/torch_dipu/csrc_dipu/runtime/device/deviceapis.h:23-124."""
import ctypes
from ctypes import byref, c_char_p, c_float, c_int, c_int32, c_int64, c_size_t, c_uint64, c_void_p

from . import _native


class RuntimeError_(RuntimeError):
    pass


def _rt():
    return _native.runtime()


def _check(rc):
    if rc != 0:
        f = _rt().dipuAmdGetLastError
        f.restype = c_char_p
        raise RuntimeError_((f() or b"").decode())


class DeviceProperties(ctypes.Structure):
    _fields_ = [("name", ctypes.c_char * 256), ("totalGlobalMem", c_uint64), ("major", c_int32),
                ("minor", c_int32), ("multiProcessorCount", c_int32)]


class MemoryStats(ctypes.Structure):
    _fields_ = [(n, c_int64) for n in (
        "allocated_bytes", "allocated_bytes_peak", "reserved_bytes", "reserved_bytes_peak", "active_bytes",
        "inactive_split_bytes", "requested_bytes", "allocations", "segments", "num_alloc_retries", "num_ooms",
        "num_device_malloc", "num_device_free")]

    def as_dict(self):
        return {n: getattr(self, n) for n, _ in self._fields_}


# ---- device ----
def getDeviceCount():
    n = c_int()
    _check(_rt().dipuAmdGetDeviceCount(byref(n)))
    return n.value


def current_device():
    n = c_int()
    _check(_rt().dipuAmdCurrentDevice(byref(n)))
    return n.value


def setDevice(dev):
    _check(_rt().dipuAmdSetDevice(c_int(dev)))


def syncDevice():
    _check(_rt().dipuAmdSyncDevice())


def checkLastError():
    _check(_rt().dipuAmdCheckLastError())


def getDriverVersion():
    v = c_int()
    _check(_rt().dipuAmdGetDriverVersion(byref(v)))
    return v.value


def getRuntimeVersion():
    v = c_int()
    _check(_rt().dipuAmdGetRuntimeVersion(byref(v)))
    return v.value


def getDeviceProperties(dev):
    p = DeviceProperties()
    _check(_rt().dipuAmdGetDeviceProperties(c_int(dev), byref(p)))
    return {"name": p.name.decode(), "totalGlobalMem": p.totalGlobalMem, "major": p.major, "minor": p.minor,
            "multiProcessorCount": p.multiProcessorCount}


def getDeviceStatus(dev):
    f, t = c_uint64(), c_uint64()
    _check(_rt().dipuAmdGetDeviceStatus(c_int(dev), byref(f), byref(t)))
    return {"freeGlobalMem": f.value, "totalGlobalMem": t.value}


# ---- streams ----
def _out_ptr(fn, *args):
    p = c_void_p()
    _check(fn(*args, byref(p)))
    return p.value or 0


def createStream():
    return _out_ptr(_rt().dipuAmdCreateStream)


def destroyStream(s):
    _check(_rt().dipuAmdDestroyStream(c_void_p(s)))


def syncStream(s):
    _check(_rt().dipuAmdSyncStream(c_void_p(s)))


def isStreamEmpty(s):
    e = c_int()
    _check(_rt().dipuAmdIsStreamEmpty(c_void_p(s), byref(e)))
    return bool(e.value)


def streamWaitEvent(s, e):
    _check(_rt().dipuAmdStreamWaitEvent(c_void_p(s), c_void_p(e)))


def getDefaultStream(dev=-1):
    return _out_ptr(_rt().dipuAmdGetDefaultStream, c_int(dev))


def getStreamFromPool(dev=-1):
    return _out_ptr(_rt().dipuAmdGetStreamFromPool, c_int(dev))


def getCurrentStream(dev=-1):
    return _out_ptr(_rt().dipuAmdGetCurrentStream, c_int(dev))


def setCurrentStream(s, dev=-1):
    _check(_rt().dipuAmdSetCurrentStream(c_int(dev), c_void_p(s)))


# ---- events ----
def createEvent():
    return _out_ptr(_rt().dipuAmdCreateEvent)


def destroyEvent(e):
    _check(_rt().dipuAmdDestroyEvent(c_void_p(e)))


def recordEvent(e, s):
    _check(_rt().dipuAmdRecordEvent(c_void_p(e), c_void_p(s)))


def waitEvent(e):
    _check(_rt().dipuAmdWaitEvent(c_void_p(e)))


def eventElapsedTime(start, end):
    ms = c_float()
    _check(_rt().dipuAmdEventElapsedTime(byref(ms), c_void_p(start), c_void_p(end)))
    return ms.value


EVENT_STATUS = ("PENDING", "RUNNING", "DEFERRED", "READY")


def getEventStatus(e):
    st = c_int()
    _check(_rt().dipuAmdGetEventStatus(c_void_p(e), byref(st)))
    return EVENT_STATUS[st.value]


# ---- raw memory ----
def mallocHost(n):
    p = c_void_p()
    _check(_rt().dipuAmdMallocHost(byref(p), c_size_t(n)))
    return p.value or 0


def freeHost(p):
    _check(_rt().dipuAmdFreeHost(c_void_p(p)))


def mallocDevice(n, throw_on_oom=True):
    p, st = c_void_p(), c_int()
    _check(_rt().dipuAmdMallocDevice(byref(p), c_size_t(n), c_int(1 if throw_on_oom else 0), byref(st)))
    return (p.value or 0), ("SUCCESS", "ERR_UNKNOWN", "ERR_NOMEM")[st.value]


def freeDevice(p):
    _check(_rt().dipuAmdFreeDevice(c_void_p(p)))


def isPinnedPtr(p):
    r = c_int()
    _check(_rt().dipuAmdIsPinnedPtr(c_void_p(p), byref(r)))
    return bool(r.value)


def memSetAsync(stream, ptr, val, size):
    _check(_rt().dipuAmdMemSetAsync(c_void_p(stream), c_void_p(ptr), c_int(val), c_size_t(size)))


def memCopyD2D(n, dst_dev, dst, src_dev, src):
    _check(_rt().dipuAmdMemCopyD2D(c_size_t(n), c_int(dst_dev), c_void_p(dst), c_int(src_dev), c_void_p(src)))


def memCopyH2D(n, dst, src):
    _check(_rt().dipuAmdMemCopyH2D(c_size_t(n), c_void_p(dst), c_void_p(src)))


def memCopyD2H(n, dst, src):
    _check(_rt().dipuAmdMemCopyD2H(c_size_t(n), c_void_p(dst), c_void_p(src)))


def memCopyD2DAsync(stream, n, dst_dev, dst, src_dev, src):
    _check(_rt().dipuAmdMemCopyD2DAsync(c_void_p(stream), c_size_t(n), c_int(dst_dev), c_void_p(dst), c_int(src_dev),
                                        c_void_p(src)))


def memCopyH2DAsync(stream, n, dst, src):
    _check(_rt().dipuAmdMemCopyH2DAsync(c_void_p(stream), c_size_t(n), c_void_p(dst), c_void_p(src)))


def memCopyD2HAsync(stream, n, dst, src):
    _check(_rt().dipuAmdMemCopyD2HAsync(c_void_p(stream), c_size_t(n), c_void_p(dst), c_void_p(src)))


# ---- caching allocators ----
def cachingMalloc(n, stream=0):
    p = c_void_p()
    _check(_rt().dipuAmdCachingMalloc(byref(p), c_size_t(n), c_void_p(stream)))
    return p.value or 0


def cachingFree(p):
    _check(_rt().dipuAmdCachingFree(c_void_p(p)))


def cachingRecordStream(p, stream):
    _check(_rt().dipuAmdCachingRecordStream(c_void_p(p), c_void_p(stream)))


def cachingEmptyCache():
    _check(_rt().dipuAmdCachingEmptyCache())


def cachingStats(dev=-1):
    s = MemoryStats()
    _check(_rt().dipuAmdCachingStats(c_int(dev), byref(s)))
    return s.as_dict()


TRACE_ACTIONS = ("ALLOC", "FREE_REQUESTED", "FREE_COMPLETED", "SEGMENT_ALLOC", "SEGMENT_FREE", "SEGMENT_MAP",
                 "SEGMENT_UNMAP", "SNAPSHOT", "OOM")   # DIPUCachingDeviceAllocator.h:135-153


class TraceEntry(ctypes.Structure):
    _fields_ = [("action", ctypes.c_int32), ("reserved", ctypes.c_int32), ("addr", ctypes.c_int64),
                ("size", c_uint64), ("stream", c_void_p)]


def _read_trace(fn, *head):
    n = c_uint64()
    _check(fn(*head, None, c_uint64(0), byref(n)))
    buf = (TraceEntry * max(1, n.value))()
    _check(fn(*head, buf, c_uint64(n.value), byref(n)))
    return [{"action": TRACE_ACTIONS[e.action], "addr": e.addr, "size": e.size, "stream": e.stream or 0}
            for e in buf[:min(n.value, len(buf))]]


def cachingRecordHistory(enabled, max_entries=2 ** 20, dev=-1):
    """recordHistory of the TORCH allocator (DIPUCachingDeviceAllocator.cpp:555-566): keep its last max_entries steps."""
    _check(_rt().dipuAmdCachingRecordHistory(c_int(dev), c_int(int(bool(enabled))), c_uint64(max_entries)))


def cachingTrace(dev=-1):
    return _read_trace(_rt().dipuAmdCachingTrace, c_int(dev))


def cachingHostMalloc(n):
    p = c_void_p()
    _check(_rt().dipuAmdCachingHostMalloc(byref(p), c_size_t(n)))
    return p.value or 0


def cachingHostFree(p):
    _check(_rt().dipuAmdCachingHostFree(c_void_p(p)))


def cachingHostRecordStream(p, stream):
    _check(_rt().dipuAmdCachingHostRecordStream(c_void_p(p), c_void_p(stream)))


def roundSize(n, conf=""):
    f = _rt().dipuAmdRoundSize
    f.restype = c_uint64
    return f(c_uint64(n), conf.encode())


def segmentSize(n, conf=""):
    f = _rt().dipuAmdSegmentSize
    f.restype = c_uint64
    return f(c_uint64(n), conf.encode())


class SimAllocator:
    """The caching allocator's state machine over a capacity-limited host stand-in for the
    device, with events that complete only on request. Needs no GPU."""

    def __init__(self, capacity, conf="", algorithm="TORCH", max_extend=0, min_allocate=0, power_of_two=False):
        self.h = c_void_p()
        if algorithm == "BF":
            _check(_rt().dipuAmdSimAllocatorCreateBF(byref(self.h), c_uint64(capacity), c_uint64(max_extend)))
        elif algorithm == "BS":
            _check(_rt().dipuAmdSimAllocatorCreateBS(byref(self.h), c_uint64(capacity), c_uint64(min_allocate), c_int(int(power_of_two))))
        else:
            _check(_rt().dipuAmdSimAllocatorCreate(byref(self.h), c_uint64(capacity), conf.encode()))

    def close(self):
        if self.h:
            _check(_rt().dipuAmdSimAllocatorDestroy(self.h))
            self.h = None

    def malloc(self, n, stream=0):
        p = c_void_p()
        _check(_rt().dipuAmdSimAllocatorMalloc(self.h, byref(p), c_size_t(n), c_void_p(stream)))
        return p.value or 0

    def malloc_from_cache(self, n, stream=0):
        p = c_void_p()
        _check(_rt().dipuAmdSimAllocatorMallocFromCache(self.h, byref(p), c_size_t(n), c_void_p(stream)))
        return p.value or 0

    def event_queries(self):
        n = c_uint64()
        _check(_rt().dipuAmdSimAllocatorEventQueries(self.h, byref(n)))
        return n.value

    def free(self, p):
        _check(_rt().dipuAmdSimAllocatorFree(self.h, c_void_p(p)))

    def record_stream(self, p, stream):
        _check(_rt().dipuAmdSimAllocatorRecordStream(self.h, c_void_p(p), c_void_p(stream)))

    def empty_cache(self):
        _check(_rt().dipuAmdSimAllocatorEmptyCache(self.h))

    def complete_events(self, stream=0):
        _check(_rt().dipuAmdSimAllocatorCompleteEvents(self.h, c_void_p(stream)))

    def stats(self):
        s = MemoryStats()
        _check(_rt().dipuAmdSimAllocatorStats(self.h, byref(s)))
        return s.as_dict()

    def record_history(self, enabled, max_entries=2 ** 20):
        _check(_rt().dipuAmdSimAllocatorRecordHistory(self.h, c_int(int(bool(enabled))), c_uint64(max_entries)))

    def trace(self):
        return _read_trace(_rt().dipuAmdSimAllocatorTrace, self.h)

    def backend_usage(self):
        b, n = c_uint64(), c_uint64()
        _check(_rt().dipuAmdSimAllocatorBackendUsage(self.h, byref(b), byref(n)))
        return b.value, n.value


# ---- profiler hooks (runtime/device/profilerapis.h:12-14; diopirt_impl.cpp:224-237) ----
profiler_on = False   # read by diopi.call on every op: a plain attribute, no C call while the profiler is off


def enableProfiler(dump_path=""):
    global profiler_on
    _check(_rt().dipuAmdProfilerEnable(dump_path.encode()))
    profiler_on = True


def disableProfiler():
    global profiler_on
    profiler_on = False
    _check(_rt().dipuAmdProfilerDisable())


def profilerCounts():
    """(ranges started, ranges ended, whether a ROCTX library is bound)."""
    a, b, r = c_uint64(), c_uint64(), c_int()
    _check(_rt().dipuAmdProfilerCounts(byref(a), byref(b), byref(r)))
    return a.value, b.value, bool(r.value)


def recordStart(name):
    """diopiRecordStart as an operator library would call it; returns the opaque record."""
    rec = c_void_p()
    f = _rt().diopiRecordStart
    f.argtypes = [c_char_p, ctypes.POINTER(c_void_p)]
    if f(name.encode(), byref(rec)) != 0:
        raise RuntimeError_("diopiRecordStart failed")
    return rec


def recordEnd(rec):
    f = _rt().diopiRecordEnd
    f.argtypes = [ctypes.POINTER(c_void_p)]
    if f(byref(rec)) != 0:
        raise RuntimeError_("diopiRecordEnd failed")


class ExpandableSegment:
    """An address range backed segment by segment through HIP virtual memory management (the vendor half of DIPU's
    expandable segments, runtime/core/allocator/ExpandableSegment.h:114-136). Offsets are relative to `base`."""

    def __init__(self, segment_bytes, device=0, stream=0):
        self.h = c_void_p()
        _check(_rt().dipuAmdExpandableSegmentCreate(byref(self.h), c_int(device), c_void_p(stream), c_uint64(segment_bytes)))

    def close(self):
        if self.h:
            _check(_rt().dipuAmdExpandableSegmentDestroy(self.h))
            self.h = None

    def info(self):
        base, res, mapped = c_void_p(), c_uint64(), c_uint64()
        _check(_rt().dipuAmdExpandableSegmentInfo(self.h, byref(base), byref(res), byref(mapped)))
        return base.value, res.value, mapped.value

    def map(self, offset, nbytes):
        o, n = c_uint64(), c_uint64()
        _check(_rt().dipuAmdExpandableSegmentMap(self.h, c_uint64(offset), c_uint64(nbytes), byref(o), byref(n)))
        return o.value, n.value

    def unmap(self, offset, nbytes):
        o, n = c_uint64(), c_uint64()
        _check(_rt().dipuAmdExpandableSegmentUnmap(self.h, c_uint64(offset), c_uint64(nbytes), byref(o), byref(n)))
        return o.value, n.value


# ---- allocator metrics ----
def metricsEnable(update=None):
    """torch_dipu._C.enable_metrics / is_metrics_enabled (binding/ExportRT.cpp:345-346): returns the setting."""
    on = c_int()
    _check(_rt().dipuAmdMetricsEnable(c_int(-1 if update is None else int(bool(update))), byref(on)))
    return bool(on.value)


def metricsText():
    need = ctypes.c_size_t()
    _check(_rt().dipuAmdMetricsText(None, ctypes.c_size_t(0), byref(need)))
    buf = ctypes.create_string_buffer(need.value + 4096)
    _check(_rt().dipuAmdMetricsText(buf, ctypes.c_size_t(len(buf)), byref(need)))
    return buf.value.decode()


def metrics():
    """{(name, frozenset of (label, value) pairs): value} of every exported line, the lookup
    dipu/tests/python/individual_scripts/test_metrics.py:22-26 does on torch_dipu._C.metrics()."""
    out = {}
    for line in metricsText().splitlines():
        head, value = line.rsplit(" ", 1)
        name, labels = head.split("{", 1)
        pairs = frozenset(tuple(kv.split("=", 1)) for kv in labels.rstrip("}").split(","))
        out[(name, frozenset((k, v.strip('"')) for k, v in pairs))] = int(value)
    return out


def metricsRecord(type_, device, data, size=0, deallocate=False):
    _check(_rt().dipuAmdMetricsRecord(type_.encode(), c_int(device), c_int(1 if deallocate else 0), c_void_p(data), ctypes.c_size_t(size)))
