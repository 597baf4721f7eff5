#include <sstream>

#include "runtime_core.h"
#include "allocator_metrics.h"
#include "expandable_segment.h"

#include <cstdlib>
#include <cstring>
#include <stdexcept>

namespace dipu {
namespace amdrt {

namespace {
int checkedDevice(int device) {
  if (device < 0) device = devapis::current_device();
  if (device >= kMaxDevices) throw std::out_of_range("device index exceeds the supported maximum of 16");
  return device;
}

struct DeviceSwitch {  // sets the device for the scope and restores the previous one
  int prev;
  bool changed;
  explicit DeviceSwitch(int device) : prev(devapis::current_device()), changed(prev != device) {
    if (changed) devapis::setDevice(static_cast<devapis::deviceId_t>(device));
  }
  ~DeviceSwitch() {
    if (changed) {
      try {
        devapis::setDevice(static_cast<devapis::deviceId_t>(prev));
      } catch (...) {
      }
    }
  }
};
}  // namespace

namespace {
// The caching allocator's view of a HipExpandableSegment.
struct HipExpandableRange final : ExpandableRange {
  HipExpandableSegment seg;
  HipExpandableRange(int device, deviceStream_t stream, size_t segmentSize) : seg(device, stream, segmentSize) {}
  void map(char* ptr, size_t size, char** mappedPtr, size_t* mappedSize) override {
    const SegmentRange r = seg.map({ptr, size});
    *mappedPtr = r.ptr, *mappedSize = r.size;
  }
  void unmap(char* ptr, size_t size, char** unmappedPtr, size_t* unmappedSize) override {
    const SegmentRange r = seg.unmap({ptr, size});
    *unmappedPtr = r.ptr, *unmappedSize = r.size;
  }
  char* ptr() const override { return seg.ptr(); }
  size_t size() const override { return seg.size(); }
};
}  // namespace

// The raw vendor calls with their metrics, as DIPU's device proxy wraps them
// (dipu/torch_dipu/csrc_dipu/runtime/devproxy/deviceproxy.cpp:196-218): type "host" and "device".
namespace devproxy {
void mallocHost(void** p, size_t nbytes) {
  devapis::mallocHost(p, nbytes);
  allocatorMetrics("host", devapis::current_device()).allocate(p ? *p : nullptr, nbytes);
}
void freeHost(void* p) {
  allocatorMetrics("host", devapis::current_device()).deallocate(p);
  devapis::freeHost(p);
}
devapis::OpStatus mallocDevice(void** p, size_t nbytes, bool throwException) {
  const devapis::OpStatus code = devapis::mallocDevice(p, nbytes, throwException);
  allocatorMetrics("device", devapis::current_device()).allocate(p ? *p : nullptr, nbytes);
  return code;
}
void freeDevice(void* p) {
  allocatorMetrics("device", devapis::current_device()).deallocate(p);
  devapis::freeDevice(p);
}
}  // namespace devproxy

RawBackend RawBackend::hip() {
  RawBackend b;
  b.createExpandable = [](StreamHandle s, size_t segmentSize) -> ExpandableRange* {
    return new HipExpandableRange(static_cast<int>(devapis::current_device()), static_cast<deviceStream_t>(s), segmentSize);
  };
  b.mallocDevice = [](void** p, size_t n) { return devproxy::mallocDevice(p, n, false) == devapis::OpStatus::SUCCESS; };
  b.freeDevice = [](void* p) { devproxy::freeDevice(p); };
  b.createEvent = []() {
    deviceEvent_t e;
    devapis::createEvent(&e);
    return static_cast<EventHandle>(e);
  };
  b.destroyEvent = [](EventHandle e) { devapis::destroyEvent(static_cast<deviceEvent_t>(e)); };
  b.recordEvent = [](EventHandle e, StreamHandle s) {
    devapis::recordEvent(static_cast<deviceEvent_t>(e), static_cast<deviceStream_t>(s));
  };
  b.eventReady = [](EventHandle e) {
    return devapis::getEventStatus(static_cast<deviceEvent_t>(e)) == devapis::EventStatus::READY;
  };
  b.syncDevice = []() { devapis::syncDevice(); };
  return b;
}

// ---------------------------------------------------------------- streams ---
deviceStream_t StreamPool::defaultStream(int device) {
  device = checkedDevice(device);
  PerDevice& d = dev_[device];
  std::call_once(d.defaultOnce, [&] {
    DeviceSwitch sw(device);
    devapis::createStream(&d.defaultStream);
    d.defaultMade = true;
  });
  return d.defaultStream;
}

deviceStream_t StreamPool::fromPool(int device) {
  device = checkedDevice(device);
  PerDevice& d = dev_[device];
  std::call_once(d.poolOnce, [&] {
    DeviceSwitch sw(device);
    for (auto& s : d.pool) devapis::createStream(&s);
    d.poolMade = true;
  });
  return d.pool[d.next++ % kStreamsPerPool];
}

namespace {
thread_local deviceStream_t t_current[kMaxDevices] = {};
thread_local bool t_currentSet[kMaxDevices] = {};
}  // namespace

deviceStream_t StreamPool::current(int device) {
  device = checkedDevice(device);
  if (!t_currentSet[device]) return defaultStream(device);
  return t_current[device];
}

void StreamPool::setCurrent(int device, deviceStream_t s) {
  device = checkedDevice(device);
  t_current[device] = s;
  t_currentSet[device] = true;
}

void StreamPool::destroyAll() {
  for (int i = 0; i < kMaxDevices; ++i) {
    PerDevice& d = dev_[i];
    if (d.defaultMade) {
      devapis::destroyStream(d.defaultStream, static_cast<devapis::deviceId_t>(i));
      d.defaultMade = false;
    }
    if (d.poolMade) {
      for (auto s : d.pool) devapis::destroyStream(s, static_cast<devapis::deviceId_t>(i));
      d.poolMade = false;
    }
  }
}

// ----------------------------------------------------------------- events ---
deviceEvent_t EventPool::get(int device) {
  device = checkedDevice(device);
  {
    std::lock_guard<std::mutex> lock(mu_[device]);
    if (!free_[device].empty()) {
      deviceEvent_t e = free_[device].back();
      free_[device].pop_back();
      return e;
    }
  }
  deviceEvent_t e;
  devapis::createEvent(&e);
  return e;
}

void EventPool::put(int device, deviceEvent_t e) {
  device = checkedDevice(device);
  std::lock_guard<std::mutex> lock(mu_[device]);
  free_[device].push_back(e);
}

void EventPool::destroyAll() {
  for (int i = 0; i < kMaxDevices; ++i) {
    std::lock_guard<std::mutex> lock(mu_[i]);
    for (auto e : free_[i]) devapis::destroyEvent(e);
    free_[i].clear();
  }
}

// ------------------------------------------------------------ pinned host ---
static size_t nextPow2(size_t n) {
  size_t p = 512;
  while (p < n) p <<= 1;
  return p;
}

void HostCachingAllocator::processEvents() {
  for (size_t i = 0; i < pending_.size();) {
    HostBlock& b = blocks_[pending_[i]];
    while (!b.events.empty() && devapis::getEventStatus(b.events.back()) == devapis::EventStatus::READY) {
      Runtime::get().events.put(-1, b.events.back());
      b.events.pop_back();
    }
    if (b.events.empty()) {
      freeBySize_[b.size].push_back(pending_[i]);
      pending_[i] = pending_.back();
      pending_.pop_back();
    } else {
      ++i;
    }
  }
}

void* HostCachingAllocator::malloc(size_t nbytes) {
  if (nbytes == 0) return nullptr;
  size_t size = nextPow2(nbytes);
  std::lock_guard<std::mutex> lock(mu_);
  processEvents();
  auto& fl = freeBySize_[size];
  void* p = nullptr;
  if (!fl.empty()) {
    p = fl.back();
    fl.pop_back();
  } else {
    devproxy::mallocHost(&p, size);
    blocks_[p].size = size;
  }
  blocks_[p].allocated = true;
  return p;
}

void HostCachingAllocator::recordStream(void* p, deviceStream_t s) {
  std::lock_guard<std::mutex> lock(mu_);
  auto it = blocks_.find(p);
  if (it == blocks_.end()) throw std::invalid_argument("host allocator: unknown pointer");
  for (auto x : it->second.streams)
    if (x == s) return;
  it->second.streams.push_back(s);
}

void HostCachingAllocator::free(void* p) {
  if (!p) return;
  std::lock_guard<std::mutex> lock(mu_);
  auto it = blocks_.find(p);
  if (it == blocks_.end() || !it->second.allocated) throw std::invalid_argument("host allocator: free of an unknown pointer");
  HostBlock& b = it->second;
  b.allocated = false;
  if (b.streams.empty()) {
    freeBySize_[b.size].push_back(p);
    return;
  }
  for (auto s : b.streams) {
    deviceEvent_t e = Runtime::get().events.get(-1);
    devapis::recordEvent(e, s);
    b.events.push_back(e);
  }
  b.streams.clear();
  pending_.push_back(p);
}

void HostCachingAllocator::emptyCache() {
  std::lock_guard<std::mutex> lock(mu_);
  processEvents();
  for (auto& kv : freeBySize_) {
    for (void* p : kv.second) {
      devproxy::freeHost(p);
      blocks_.erase(p);
    }
    kv.second.clear();
  }
}

bool HostCachingAllocator::owns(const void* p) {
  std::lock_guard<std::mutex> lock(mu_);
  return blocks_.count(const_cast<void*>(p)) != 0;
}

// ---------------------------------------------------------------- runtime ---
Runtime& Runtime::get() {
  static Runtime* rt = new Runtime();  // intentionally leaked: outlives static destructors
  return *rt;
}

bool Runtime::useRaw() {
  if (algorithm_ < 0) {
    const char* env = std::getenv("DIPU_DEVICE_MEMCACHING_ALGORITHM");
    std::string a = env ? env : "TORCH";
    if (a == "TORCH") {
      algorithm_ = 0;
    } else if (a == "BF") {
      algorithm_ = 2;
    } else if (a == "BS") {
      algorithm_ = 3;
    } else if (a == "RAW") {
      algorithm_ = 1;
    } else {
      throw std::invalid_argument("DIPU_DEVICE_MEMCACHING_ALGORITHM: unknown algorithm '" + a + "'");
    }
  }
  return algorithm_ == 1;
}

DeviceAllocator* Runtime::caching(int device) {
  device = checkedDevice(device);
  useRaw();  // reads the algorithm selection once
  std::lock_guard<std::mutex> lock(mu_);
  if (!caching_[device] && algorithm_ == 2) caching_[device] = std::make_unique<BFCachingAllocator>(RawBackend::hip());
  if (!caching_[device] && algorithm_ == 3) caching_[device] = std::make_unique<BSCachingAllocator>(RawBackend::hip());
  if (!caching_[device]) {
    const char* conf = std::getenv("DIPU_TORCH_ALLOCATOR_CONF");
    AllocatorConfig cfg = AllocatorConfig::parse(conf ? conf : "");
    try {
      cfg.deviceCapacity = devapis::getDeviceProperties(device).totalGlobalMem;
    } catch (...) {
      cfg.deviceCapacity = 0;
    }
    caching_[device] = std::make_unique<DeviceCachingAllocator>(RawBackend::hip(), cfg);
  }
  return caching_[device].get();
}

RawAllocator* Runtime::raw(int device) {
  device = checkedDevice(device);
  std::lock_guard<std::mutex> lock(mu_);
  if (!raw_[device]) raw_[device] = std::make_unique<RawAllocator>(RawBackend::hip());
  return raw_[device].get();
}

// hipStreamIsCapturing on the null stream fails while another stream captures in global mode; that failure is not
// this request's and is cleared.
static bool streamIsCapturing(deviceStream_t stream) {
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &status) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return status == hipStreamCaptureStatusActive;
}

void* Runtime::deviceMalloc(size_t nbytes, deviceStream_t stream) {
  int device = devapis::current_device();
  void* p = nullptr;
  if (nbytes > 0 && streamIsCapturing(stream)) {
    // Recording into a graph: hipMalloc, hipFree, event records and device-wide waits are all illegal, so only a
    // block already in the TORCH algorithm's cache can serve the request.
    if (!useRaw() && algorithm_ == 0) p = caching(device)->mallocFromCache(nbytes, stream);
    if (!p) {
      std::ostringstream os;
      os << "request for " << nbytes << " bytes on a stream that is being captured into a graph";
      if (useRaw() || algorithm_ != 0)
        os << ": only DIPU_DEVICE_MEMCACHING_ALGORITHM=TORCH serves requests during capture";
      else
        os << " found no cached block: run the same calls on this stream once before capturing, holding their workspace";
      throw std::runtime_error(os.str());
    }
  } else {
    p = useRaw() ? raw(device)->malloc(nbytes) : caching(device)->malloc(nbytes, stream);
  }
  if (p) {
    std::lock_guard<std::mutex> lock(mu_);
    ownerDevice_[p] = device;
  }
  // type "caching" (DIPUCachingDeviceAllocator.cpp:1845-1875), with the size that was asked for
  allocatorMetrics("caching", device).allocate(p, nbytes);
  return p;
}

void Runtime::deviceFree(void* p) {
  if (!p) return;
  int device;
  {
    std::lock_guard<std::mutex> lock(mu_);
    auto it = ownerDevice_.find(p);
    if (it == ownerDevice_.end()) throw std::invalid_argument("caching free of a pointer this allocator did not hand out");
    device = it->second;
    ownerDevice_.erase(it);
  }
  allocatorMetrics("caching", device).deallocate(p);
  if (useRaw()) raw(device)->free(p); else caching(device)->free(p);
}

void Runtime::shutdown() {
  for (auto& a : caching_)
    if (a) a->emptyCache();
  host.emptyCache();
  events.destroyAll();
  streams.destroyAll();
}

}  // namespace amdrt
}  // namespace dipu
