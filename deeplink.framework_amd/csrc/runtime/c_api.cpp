// C facade over the C++ runtime: turns exceptions into return codes so callers
// in any language (ctypes here, a C harness, DIPU glue) never see a C++ exception.
#include <cstdlib>
#include <cstring>
#include <map>

#include <dipu_amd/runtime.h>

#include "expandable_segment.h"
#include "runtime_core.h"
#include "allocator_metrics.h"

using namespace dipu;
using namespace dipu::amdrt;

namespace dipu {
namespace amdrt {
void* contextCreate(deviceStream_t s);
void contextDestroy(void* c);
void contextReset(void* c);
void contextWorkspace(void* c, uint64_t* tensors, uint64_t* bytes);
void noteError(const char* what);
}  // namespace amdrt
}  // namespace dipu

namespace {
thread_local std::string g_err;

template <typename F>
int guarded(F&& f) {
  try {
    f();
    return 0;
  } catch (const std::exception& e) {
    g_err = e.what();
    return 1;
  } catch (...) {
    g_err = "unknown C++ exception";
    return 1;
  }
}

deviceStream_t S(void* s) { return static_cast<deviceStream_t>(s); }
deviceEvent_t E(void* e) { return static_cast<deviceEvent_t>(e); }
devapis::deviceId_t D(int d) { return static_cast<devapis::deviceId_t>(d); }

void fillStats(const DeviceStats& s, dipuAmdMemoryStats* o) {
  o->allocated_bytes = s.allocatedBytes.current;
  o->allocated_bytes_peak = s.allocatedBytes.peak;
  o->reserved_bytes = s.reservedBytes.current;
  o->reserved_bytes_peak = s.reservedBytes.peak;
  o->active_bytes = s.activeBytes.current;
  o->inactive_split_bytes = s.inactiveSplitBytes.current;
  o->requested_bytes = s.requestedBytes.current;
  o->allocations = s.allocation.current;
  o->segments = s.segment.current;
  o->num_alloc_retries = s.numAllocRetries;
  o->num_ooms = s.numOoms;
  o->num_device_malloc = s.numDeviceMalloc;
  o->num_device_free = s.numDeviceFree;
}

// Host-memory stand-in for the device: capacity-limited malloc, events that complete
// only when the test says so.
struct SimBackend {
  uint64_t capacity = 0, inUse = 0, segments = 0, eventQueries = 0;
  uintptr_t nextAddr = uintptr_t(1) << 44;
  std::map<void*, size_t> live;
  struct SimEvent {
    void* stream = nullptr;
    bool ready = true;
  };
  std::vector<SimEvent*> events;
  ~SimBackend() {
    for (auto* e : events) delete e;
  }
};

// A 1 GiB synthetic address range whose segments count against the simulated capacity while mapped.
struct SimExpandableRange final : ExpandableRange {
  SimBackend* sb;
  size_t segmentSize;
  char* base;
  std::vector<bool> mapped;
  SimExpandableRange(SimBackend* b, size_t segSize) : sb(b), segmentSize(segSize), mapped((size_t(1) << 30) / segSize, false) {
    base = reinterpret_cast<char*>(sb->nextAddr);
    sb->nextAddr += size_t(1) << 30;
  }
  ~SimExpandableRange() override {
    for (bool m : mapped)
      if (m) sb->inUse -= segmentSize, --sb->segments;
  }
  void map(char* p, size_t n, char** mp, size_t* ms) override {
    const size_t begin = static_cast<size_t>(p - base) / segmentSize;
    const size_t end = std::min(mapped.size(), (static_cast<size_t>(p - base) + n + segmentSize - 1) / segmentSize);
    if (static_cast<size_t>(p - base) % segmentSize) throw std::invalid_argument("sim expandable range: map must start at a segment");
    *mp = p, *ms = 0;
    if (sb->inUse + (end - begin) * segmentSize > sb->capacity) return;
    for (size_t i = begin; i < end; ++i) {
      if (mapped[i]) throw std::invalid_argument("sim expandable range: segment mapped twice");
      mapped[i] = true, sb->inUse += segmentSize, ++sb->segments;
    }
    *ms = (end - begin) * segmentSize;
  }
  void unmap(char* p, size_t n, char** up, size_t* us) override {
    const size_t begin = (static_cast<size_t>(p - base) + segmentSize - 1) / segmentSize;
    const size_t end = std::min(mapped.size(), (static_cast<size_t>(p - base) + n) / segmentSize);
    *up = base + begin * segmentSize, *us = 0;
    if (begin >= end) return;
    for (size_t i = begin; i < end; ++i) {
      if (!mapped[i]) throw std::invalid_argument("sim expandable range: segment was not mapped");
      mapped[i] = false, sb->inUse -= segmentSize, --sb->segments;
    }
    *us = (end - begin) * segmentSize;
  }
  char* ptr() const override { return base; }
  size_t size() const override { return mapped.size() * segmentSize; }
};

struct SimAllocator {
  SimBackend backend;
  std::unique_ptr<DeviceAllocator> alloc;
};

RawBackend makeSimBackend(SimBackend* sb) {
  RawBackend b;
  b.createExpandable = [sb](StreamHandle, size_t segmentSize) -> ExpandableRange* { return new SimExpandableRange(sb, segmentSize); };
  b.mallocDevice = [sb](void** p, size_t n) {
    if (sb->inUse + n > sb->capacity) return false;
    // Addresses are synthetic and never dereferenced: a monotonically growing, 2 MiB
    // aligned range per segment, so split blocks of different segments never collide.
    uintptr_t base = sb->nextAddr;
    sb->nextAddr += (n + (size_t(2) << 20) - 1) & ~((size_t(2) << 20) - 1);
    void* q = reinterpret_cast<void*>(base);
    sb->live[q] = n;
    sb->inUse += n;
    ++sb->segments;
    *p = q;
    return true;
  };
  b.freeDevice = [sb](void* p) {
    auto it = sb->live.find(p);
    if (it == sb->live.end()) throw std::invalid_argument("sim backend: double free");
    sb->inUse -= it->second;
    --sb->segments;
    sb->live.erase(it);
  };
  b.createEvent = [sb]() {
    auto* e = new SimBackend::SimEvent();
    sb->events.push_back(e);
    return static_cast<EventHandle>(e);
  };
  b.destroyEvent = [](EventHandle) {};
  b.recordEvent = [](EventHandle e, StreamHandle s) {
    auto* ev = static_cast<SimBackend::SimEvent*>(e);
    ev->stream = s;
    ev->ready = false;
  };
  b.eventReady = [sb](EventHandle e) {
    ++sb->eventQueries;
    return static_cast<SimBackend::SimEvent*>(e)->ready;
  };
  b.syncDevice = [sb]() {
    for (auto* e : sb->events) e->ready = true;
  };
  return b;
}
}  // namespace

extern "C" {

const char* dipuAmdGetLastError(void) { return g_err.c_str(); }
}
// what a diopirt callback could not report through its return code (it has no message channel of its own)
void dipu::amdrt::noteError(const char* what) { g_err = what; }
extern "C" {

int dipuAmdInitializeVendor(void) { return guarded([] { devapis::initializeVendor(); }); }
int dipuAmdFinalizeVendor(void) {
  return guarded([] {
    Runtime::get().shutdown();
    devapis::finalizeVendor();
  });
}
int dipuAmdGetDeviceCount(int* count) { return guarded([&] { *count = devapis::getDeviceCount(); }); }
int dipuAmdCurrentDevice(int* device) { return guarded([&] { *device = devapis::current_device(); }); }
int dipuAmdSetDevice(int device) { return guarded([&] { devapis::setDevice(D(device)); }); }
int dipuAmdSyncDevice(void) { return guarded([] { devapis::syncDevice(); }); }
int dipuAmdCheckLastError(void) { return guarded([] { devapis::checkLastError(); }); }
int dipuAmdGetDriverVersion(int* v) { return guarded([&] { devapis::getDriverVersion(v); }); }
int dipuAmdGetRuntimeVersion(int* v) { return guarded([&] { devapis::getRuntimeVersion(v); }); }
int dipuAmdGetDeviceProperties(int device, dipuAmdDeviceProperties* props) {
  return guarded([&] {
    auto p = devapis::getDeviceProperties(device);
    std::memset(props, 0, sizeof(*props));
    std::strncpy(props->name, p.name.c_str(), sizeof(props->name) - 1);
    props->totalGlobalMem = p.totalGlobalMem;
    props->major = p.major;
    props->minor = p.minor;
    props->multiProcessorCount = p.multiProcessorCount;
  });
}
int dipuAmdGetDeviceStatus(int device, uint64_t* free_bytes, uint64_t* total_bytes) {
  return guarded([&] {
    auto s = devapis::getDeviceStatus(device);
    *free_bytes = s.freeGlobalMem;
    *total_bytes = s.totalGlobalMem;
  });
}

int dipuAmdCreateStream(void** stream) {
  return guarded([&] {
    deviceStream_t s;
    devapis::createStream(&s);
    *stream = s;
  });
}
int dipuAmdDestroyStream(void* stream) { return guarded([&] { devapis::destroyStream(S(stream)); }); }
int dipuAmdSyncStream(void* stream) { return guarded([&] { devapis::syncStream(S(stream)); }); }
int dipuAmdIsStreamEmpty(void* stream, int* empty) {
  return guarded([&] { *empty = devapis::isStreamEmpty(S(stream)) ? 1 : 0; });
}
int dipuAmdStreamWaitEvent(void* stream, void* event) {
  return guarded([&] { devapis::streamWaitEvent(S(stream), E(event)); });
}
int dipuAmdGetDefaultStream(int device, void** stream) {
  return guarded([&] { *stream = Runtime::get().streams.defaultStream(device); });
}
int dipuAmdGetStreamFromPool(int device, void** stream) {
  return guarded([&] { *stream = Runtime::get().streams.fromPool(device); });
}
int dipuAmdGetCurrentStream(int device, void** stream) {
  return guarded([&] { *stream = Runtime::get().streams.current(device); });
}
int dipuAmdSetCurrentStream(int device, void* stream) {
  return guarded([&] { Runtime::get().streams.setCurrent(device, S(stream)); });
}

int dipuAmdCreateEvent(void** event) {
  return guarded([&] { *event = Runtime::get().events.get(-1); });
}
int dipuAmdDestroyEvent(void* event) {
  return guarded([&] { Runtime::get().events.put(-1, E(event)); });
}
int dipuAmdRecordEvent(void* event, void* stream) { return guarded([&] { devapis::recordEvent(E(event), S(stream)); }); }
int dipuAmdWaitEvent(void* event) { return guarded([&] { devapis::waitEvent(E(event)); }); }
int dipuAmdEventElapsedTime(float* ms, void* start, void* end) {
  return guarded([&] { devapis::eventElapsedTime(ms, E(start), E(end)); });
}
int dipuAmdGetEventStatus(void* event, int* status) {
  return guarded([&] { *status = static_cast<int>(devapis::getEventStatus(E(event))); });
}

int dipuAmdMallocHost(void** p, size_t n) { return guarded([&] { devproxy::mallocHost(p, n); }); }
int dipuAmdFreeHost(void* p) { return guarded([&] { devproxy::freeHost(p); }); }
int dipuAmdMallocDevice(void** p, size_t n, int throw_on_oom, int* status) {
  return guarded([&] { *status = static_cast<int>(devproxy::mallocDevice(p, n, throw_on_oom != 0)); });
}
int dipuAmdFreeDevice(void* p) { return guarded([&] { devproxy::freeDevice(p); }); }
int dipuAmdIsPinnedPtr(const void* p, int* pinned) {
  return guarded([&] { *pinned = devapis::isPinnedPtr(p) ? 1 : 0; });
}
int dipuAmdMemSetAsync(void* stream, void* ptr, int val, size_t size) {
  return guarded([&] { devapis::memSetAsync(S(stream), ptr, val, size); });
}
int dipuAmdMemCopyD2D(size_t n, int dd, void* dst, int sd, const void* src) {
  return guarded([&] { devapis::memCopyD2D(n, D(dd), dst, D(sd), src); });
}
int dipuAmdMemCopyH2D(size_t n, void* dst, const void* src) { return guarded([&] { devapis::memCopyH2D(n, dst, src); }); }
int dipuAmdMemCopyD2H(size_t n, void* dst, const void* src) { return guarded([&] { devapis::memCopyD2H(n, dst, src); }); }
int dipuAmdMemCopyD2DAsync(void* stream, size_t n, int dd, void* dst, int sd, const void* src) {
  return guarded([&] { devapis::memCopyD2DAsync(S(stream), n, D(dd), dst, D(sd), src); });
}
int dipuAmdMemCopyH2DAsync(void* stream, size_t n, void* dst, const void* src) {
  return guarded([&] { devapis::memCopyH2DAsync(S(stream), n, dst, src); });
}
int dipuAmdMemCopyD2HAsync(void* stream, size_t n, void* dst, const void* src) {
  return guarded([&] { devapis::memCopyD2HAsync(S(stream), n, dst, src); });
}

int dipuAmdCachingMalloc(void** p, size_t n, void* stream) {
  return guarded([&] { *p = Runtime::get().deviceMalloc(n, S(stream)); });
}
int dipuAmdCachingFree(void* p) { return guarded([&] { Runtime::get().deviceFree(p); }); }
int dipuAmdCachingRecordStream(void* p, void* stream) {
  return guarded([&] {
    if (!Runtime::get().useRaw()) Runtime::get().caching(-1)->recordStream(p, stream);
  });
}
int dipuAmdCachingEmptyCache(void) {
  return guarded([&] {
    if (!Runtime::get().useRaw()) Runtime::get().caching(-1)->emptyCache();
  });
}
int dipuAmdCachingStats(int device, dipuAmdMemoryStats* stats) {
  return guarded([&] {
    Runtime& rt = Runtime::get();
    fillStats(rt.useRaw() ? rt.raw(device)->stats() : rt.caching(device)->stats(), stats);
  });
}
int dipuAmdCachingResetPeakStats(int device) {
  return guarded([&] {
    if (!Runtime::get().useRaw()) Runtime::get().caching(device)->resetPeakStats();
  });
}
namespace {
void copyTrace(const std::vector<TraceEntry>& t, dipuAmdTraceEntry* entries, uint64_t capacity, uint64_t* count) {
  *count = t.size();
  for (size_t i = 0; i < t.size() && i < capacity; ++i)
    entries[i] = dipuAmdTraceEntry{t[i].action, 0, t[i].addr, t[i].size, t[i].stream};
}
}  // namespace
int dipuAmdCachingRecordHistory(int device, int enabled, uint64_t max_entries) {
  return guarded([&] {
    if (!Runtime::get().useRaw()) Runtime::get().caching(device)->recordHistory(enabled != 0, max_entries);
  });
}
int dipuAmdCachingTrace(int device, dipuAmdTraceEntry* entries, uint64_t capacity, uint64_t* count) {
  return guarded([&] {
    *count = 0;
    if (!Runtime::get().useRaw()) copyTrace(Runtime::get().caching(device)->trace(), entries, capacity, count);
  });
}
int dipuAmdCachingHostMalloc(void** p, size_t n) { return guarded([&] { *p = Runtime::get().host.malloc(n); }); }
int dipuAmdCachingHostFree(void* p) { return guarded([&] { Runtime::get().host.free(p); }); }
int dipuAmdCachingHostRecordStream(void* p, void* stream) {
  return guarded([&] { Runtime::get().host.recordStream(p, S(stream)); });
}
int dipuAmdCachingHostEmptyCache(void) { return guarded([&] { Runtime::get().host.emptyCache(); }); }

int dipuAmdSimAllocatorCreate(void** handle, uint64_t capacity_bytes, const char* conf) {
  return guarded([&] {
    auto sim = std::make_unique<SimAllocator>();
    sim->backend.capacity = capacity_bytes;
    AllocatorConfig cfg = AllocatorConfig::parse(conf ? conf : "");
    cfg.deviceCapacity = capacity_bytes;
    sim->alloc = std::make_unique<DeviceCachingAllocator>(makeSimBackend(&sim->backend), cfg);
    *handle = sim.release();
  });
}
int dipuAmdSimAllocatorCreateBF(void** handle, uint64_t capacity_bytes, uint64_t max_extend_bytes) {
  return guarded([&] {
    auto sim = std::make_unique<SimAllocator>();
    sim->backend.capacity = capacity_bytes;
    sim->alloc = std::make_unique<BFCachingAllocator>(makeSimBackend(&sim->backend), max_extend_bytes);
    *handle = sim.release();
  });
}
int dipuAmdExpandableSegmentCreate(void** handle, int device, void* stream, uint64_t segment_bytes) {
  return guarded([&] { *handle = new HipExpandableSegment(device, S(stream), segment_bytes); });
}
int dipuAmdExpandableSegmentDestroy(void* handle) {
  return guarded([&] { delete static_cast<HipExpandableSegment*>(handle); });
}
int dipuAmdExpandableSegmentInfo(void* handle, void** base, uint64_t* reserved_bytes, uint64_t* mapped_bytes) {
  return guarded([&] {
    auto* s = static_cast<HipExpandableSegment*>(handle);
    *base = s->ptr(), *reserved_bytes = s->size(), *mapped_bytes = s->mappedBytes();
  });
}
int dipuAmdExpandableSegmentMap(void* handle, uint64_t offset, uint64_t nbytes, uint64_t* mapped_offset, uint64_t* mapped_bytes) {
  return guarded([&] {
    auto* s = static_cast<HipExpandableSegment*>(handle);
    const SegmentRange r = s->map({s->ptr() + offset, nbytes});
    *mapped_offset = static_cast<uint64_t>(r.ptr - s->ptr()), *mapped_bytes = r.size;
  });
}
int dipuAmdExpandableSegmentUnmap(void* handle, uint64_t offset, uint64_t nbytes, uint64_t* unmapped_offset, uint64_t* unmapped_bytes) {
  return guarded([&] {
    auto* s = static_cast<HipExpandableSegment*>(handle);
    const SegmentRange r = s->unmap({s->ptr() + offset, nbytes});
    *unmapped_offset = static_cast<uint64_t>(r.ptr - s->ptr()), *unmapped_bytes = r.size;
  });
}
int dipuAmdSimAllocatorCreateBS(void** handle, uint64_t capacity_bytes, uint64_t min_allocate_bytes, int power_of_two) {
  return guarded([&] {
    auto sim = std::make_unique<SimAllocator>();
    sim->backend.capacity = capacity_bytes;
    sim->alloc = std::make_unique<BSCachingAllocator>(makeSimBackend(&sim->backend), min_allocate_bytes, power_of_two ? 1 : 0);
    *handle = sim.release();
  });
}
int dipuAmdSimAllocatorDestroy(void* handle) {
  return guarded([&] {
    auto* sim = static_cast<SimAllocator*>(handle);
    sim->alloc.reset();
    delete sim;
  });
}
int dipuAmdSimAllocatorMalloc(void* handle, void** p, size_t n, void* stream) {
  return guarded([&] { *p = static_cast<SimAllocator*>(handle)->alloc->malloc(n, stream); });
}
int dipuAmdSimAllocatorMallocFromCache(void* handle, void** p, size_t n, void* stream) {
  return guarded([&] { *p = static_cast<SimAllocator*>(handle)->alloc->mallocFromCache(n, stream); });
}
int dipuAmdSimAllocatorEventQueries(void* handle, uint64_t* queries) {
  return guarded([&] { *queries = static_cast<SimAllocator*>(handle)->backend.eventQueries; });
}
int dipuAmdSimAllocatorFree(void* handle, void* p) {
  return guarded([&] { static_cast<SimAllocator*>(handle)->alloc->free(p); });
}
int dipuAmdSimAllocatorRecordStream(void* handle, void* p, void* stream) {
  return guarded([&] { static_cast<SimAllocator*>(handle)->alloc->recordStream(p, stream); });
}
int dipuAmdSimAllocatorEmptyCache(void* handle) {
  return guarded([&] { static_cast<SimAllocator*>(handle)->alloc->emptyCache(); });
}
int dipuAmdSimAllocatorStats(void* handle, dipuAmdMemoryStats* stats) {
  return guarded([&] { fillStats(static_cast<SimAllocator*>(handle)->alloc->stats(), stats); });
}
int dipuAmdSimAllocatorRecordHistory(void* handle, int enabled, uint64_t max_entries) {
  return guarded([&] { static_cast<SimAllocator*>(handle)->alloc->recordHistory(enabled != 0, max_entries); });
}
int dipuAmdSimAllocatorTrace(void* handle, dipuAmdTraceEntry* entries, uint64_t capacity, uint64_t* count) {
  return guarded([&] { copyTrace(static_cast<SimAllocator*>(handle)->alloc->trace(), entries, capacity, count); });
}
int dipuAmdSimAllocatorCompleteEvents(void* handle, void* stream) {
  return guarded([&] {
    auto* sim = static_cast<SimAllocator*>(handle);
    for (auto* e : sim->backend.events)
      if (stream == nullptr || e->stream == stream) e->ready = true;
    sim->alloc->processEvents();
  });
}
int dipuAmdSimAllocatorBackendUsage(void* handle, uint64_t* bytes_in_use, uint64_t* live_segments) {
  return guarded([&] {
    auto* sim = static_cast<SimAllocator*>(handle);
    *bytes_in_use = sim->backend.inUse;
    *live_segments = sim->backend.segments;
  });
}
uint64_t dipuAmdRoundSize(uint64_t nbytes, const char* conf) {
  try {
    return DeviceCachingAllocator::roundSize(nbytes, AllocatorConfig::parse(conf ? conf : ""));
  } catch (...) {
    return 0;
  }
}
uint64_t dipuAmdSegmentSize(uint64_t rounded, const char* conf) {
  try {
    return DeviceCachingAllocator::allocationSize(rounded, AllocatorConfig::parse(conf ? conf : ""));
  } catch (...) {
    return 0;
  }
}

int dipuAmdContextCreate(void* stream, void** ctx) { return guarded([&] { *ctx = contextCreate(S(stream)); }); }
int dipuAmdContextDestroy(void* ctx) { return guarded([&] { contextDestroy(ctx); }); }
int dipuAmdContextReset(void* ctx) { return guarded([&] { contextReset(ctx); }); }
int dipuAmdContextWorkspace(void* ctx, uint64_t* tensors, uint64_t* bytes) {
  return guarded([&] { contextWorkspace(ctx, tensors, bytes); });
}

int dipuAmdProfilerEnable(const char* dump_path) {
  return guarded([&] { dipu::devapis::enableProfiler(dump_path ? dump_path : "", false, false, false); });
}
int dipuAmdProfilerDisable() { return guarded([&] { dipu::devapis::disableProfiler(); }); }
int dipuAmdProfilerCounts(uint64_t* started, uint64_t* stopped, int* roctx_bound) {
  return guarded([&] { dipu::profile::counts(started, stopped, roctx_bound); });
}


int dipuAmdMetricsEnable(int update, int* enabled) {
  return guarded([&] {
    const bool v = metricsEnable(update);
    if (enabled) *enabled = v ? 1 : 0;
  });
}
int dipuAmdMetricsText(char* buffer, size_t capacity, size_t* needed) {
  return guarded([&] {
    const std::string text = metricsText();
    if (needed) *needed = text.size() + 1;
    if (buffer && capacity > 0) {
      const size_t n = text.size() < capacity - 1 ? text.size() : capacity - 1;
      std::memcpy(buffer, text.data(), n);
      buffer[n] = 0;
    }
  });
}
int dipuAmdMetricsRecord(const char* type, int device, int deallocate, void* data, size_t size) {
  return guarded([&] {
    AllocatorMetrics& m = allocatorMetrics(type ? type : "", device);
    if (deallocate) m.deallocate(data); else m.allocate(data, size);
  });
}

}  // extern "C"
