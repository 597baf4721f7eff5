// Process-wide runtime state above devapis: stream pool, event pool, device and pinned-host
// caching allocators. Mirrors the responsibilities of DIPU's runtime/core layer
// (dipu/torch_dipu/csrc_dipu/runtime/core/DIPUStream.cpp, DIPUEventPool.cpp,
// allocator/DIPUCachingAllocator.cpp:76-163,336-343) for a host that is not DIPU.
#pragma once

#include <array>
#include <atomic>
#include <deque>
#include <memory>
#include <mutex>
#include <vector>

#include "caching_allocator.h"
#include "devapis_contract.h"

namespace dipu {
namespace amdrt {

constexpr int kMaxDevices = 16;       // same hard cap as DIPU's event pool
constexpr int kStreamsPerPool = 8;    // 1 default + 8 pooled streams per device

class StreamPool {
 public:
  deviceStream_t defaultStream(int device);
  deviceStream_t fromPool(int device);
  deviceStream_t current(int device);
  void setCurrent(int device, deviceStream_t s);
  void destroyAll();

 private:
  struct PerDevice {
    std::once_flag defaultOnce, poolOnce;
    deviceStream_t defaultStream = nullptr;
    std::array<deviceStream_t, kStreamsPerPool> pool{};
    std::atomic<uint32_t> next{0};
    bool defaultMade = false, poolMade = false;
  };
  std::array<PerDevice, kMaxDevices> dev_;
};

class EventPool {
 public:
  deviceEvent_t get(int device);
  void put(int device, deviceEvent_t e);
  void destroyAll();

 private:
  std::array<std::mutex, kMaxDevices> mu_;
  std::array<std::deque<deviceEvent_t>, kMaxDevices> free_;
};

// Pinned host blocks, sizes rounded to powers of two; a freed block that was used on
// streams is reusable only after an event on each of those streams has completed.
class HostCachingAllocator {
 public:
  void* malloc(size_t nbytes);
  void free(void* p);
  void recordStream(void* p, deviceStream_t s);
  void emptyCache();
  bool owns(const void* p);

 private:
  struct HostBlock {
    size_t size = 0;
    bool allocated = false;
    std::vector<deviceStream_t> streams;
    std::vector<deviceEvent_t> events;
  };
  void processEvents();
  std::mutex mu_;
  std::unordered_map<void*, HostBlock> blocks_;
  std::unordered_map<size_t, std::vector<void*>> freeBySize_;
  std::vector<void*> pending_;
};

// devapis::malloc* / free* with the "host" and "device" allocator metrics recorded around them.
namespace devproxy {
void mallocHost(void** p, size_t nbytes);
void freeHost(void* p);
devapis::OpStatus mallocDevice(void** p, size_t nbytes, bool throwException);
void freeDevice(void* p);
}  // namespace devproxy

struct Runtime {
  StreamPool streams;
  EventPool events;
  HostCachingAllocator host;
  // device allocators are created lazily per device according to the environment
  DeviceAllocator* caching(int device);  // TORCH or BF, whichever the environment selects
  RawAllocator* raw(int device);
  bool useRaw();
  void* deviceMalloc(size_t nbytes, deviceStream_t stream);
  void deviceFree(void* p);
  void shutdown();
  static Runtime& get();

 private:
  std::mutex mu_;
  std::array<std::unique_ptr<DeviceAllocator>, kMaxDevices> caching_;
  std::array<std::unique_ptr<RawAllocator>, kMaxDevices> raw_;
  std::unordered_map<void*, int> ownerDevice_;
  int algorithm_ = -1;  // 0 TORCH, 1 RAW, 2 BF, 3 BS
};

}  // namespace amdrt
}  // namespace dipu
