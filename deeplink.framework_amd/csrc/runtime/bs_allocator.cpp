// The BS ("by size") device caching algorithm, selected with DIPU_DEVICE_MEMCACHING_ALGORITHM=BS. Behaviour follows
// dipu/torch_dipu/csrc_dipu/runtime/core/allocator/DIPUBSCachingAllocator.cpp (size rule :36-70, allocate :72-128,
// restore :130-138, empty cache :152-173, event-deferred free :200-222).
#include <algorithm>
#include <cstdlib>
#include <stdexcept>
#include <string>
#include <thread>

#include "caching_allocator.h"

namespace dipu {
namespace amdrt {

BSCachingAllocator::BSCachingAllocator(RawBackend backend, size_t minAllocate, int powerOfTwo)
    : backend_(std::move(backend)) {
  if (minAllocate == 0) {
    const char* e = std::getenv("DIPU_BS_ALLOCATOR_MIN_ALLOCATE_SIZE");
    const long v = e ? std::atol(e) : 512;
    minAllocate = static_cast<size_t>(v > 0 ? v : 512);
  }
  // the multiple-of rule needs a power of two to round with a mask, as the reference does
  size_t p2 = 1;
  while (p2 < minAllocate) p2 <<= 1;
  minAllocate_ = p2;
  powerOfTwo_ = powerOfTwo < 0 ? std::getenv("DIPU_BS_MORE_ADAPTABLE") != nullptr : powerOfTwo != 0;
}

BSCachingAllocator::~BSCachingAllocator() {
  try {
    std::lock_guard<std::mutex> lock(mutex_);
    backend_.syncDevice();
    drainPending(true);
    releaseIdle();
    for (EventHandle e : eventPool_) backend_.destroyEvent(e);
  } catch (...) {
  }
}

size_t BSCachingAllocator::allocateSize(size_t nbytes) const {
  if (!powerOfTwo_) return ((nbytes - 1) | (minAllocate_ - 1)) + 1;
  size_t s = minAllocate_;
  while (s <= nbytes) s <<= 1;  // the reference takes 1 << bit_length(n): a power of two itself doubles
  return s;
}

EventHandle BSCachingAllocator::newEvent() {
  if (!eventPool_.empty()) {
    EventHandle e = eventPool_.back();
    eventPool_.pop_back();
    return e;
  }
  return backend_.createEvent();
}

bool BSCachingAllocator::drainPending(bool wait) {
  size_t kept = 0;
  for (size_t i = 0; i < pending_.size(); ++i) {
    Pending& p = pending_[i];
    bool ready = true;
    for (EventHandle e : p.events) {
      if (wait) {
        while (!backend_.eventReady(e)) std::this_thread::yield();
      } else if (!backend_.eventReady(e)) {
        ready = false;
        break;
      }
    }
    if (ready) {
      for (EventHandle e : p.events) eventPool_.push_back(e);
      idle_[p.size].push_back(p.ptr);
    } else {
      if (kept != i) pending_[kept] = std::move(p);
      ++kept;
    }
  }
  pending_.resize(kept);
  return kept == 0;
}

void BSCachingAllocator::releaseIdle() {
  for (auto& kv : idle_) {
    for (void* p : kv.second) {
      backend_.freeDevice(p);
      stats_.reservedBytes.add(-static_cast<int64_t>(kv.first));
      stats_.segment.add(-1);
      ++stats_.numDeviceFree;
    }
    kv.second.clear();
  }
}

void* BSCachingAllocator::malloc(size_t size, StreamHandle stream) {
  if (size == 0) return nullptr;
  const size_t nbytes = allocateSize(size);
  std::lock_guard<std::mutex> lock(mutex_);
  drainPending(false);
  auto& idle = idle_[nbytes];
  if (idle.empty() && !pending_.empty()) {  // the reference waits for everything on its way back first (:82-85)
    backend_.syncDevice();
    drainPending(true);
  }
  void* p = nullptr;
  if (!idle.empty()) {
    p = idle.front();
    idle.erase(idle.begin());
  } else {
    for (int attempt = 0; attempt < 2 && !p; ++attempt) {
      if (backend_.mallocDevice(&p, nbytes)) {
        ++stats_.numDeviceMalloc;
        stats_.reservedBytes.add(static_cast<int64_t>(nbytes));
        stats_.segment.add(1);
      } else {
        p = nullptr;
        if (attempt == 0) {
          ++stats_.numAllocRetries;
          releaseIdle();
        }
      }
    }
    if (!p) {
      ++stats_.numOoms;
      throw OutOfMemory("BS allocator: no memory available for " + std::to_string(nbytes) + " bytes");
    }
  }
  Live& l = live_[p];
  l.size = nbytes;
  l.stream = stream;
  l.extraStreams.clear();
  stats_.allocation.add(1);
  stats_.activeBlocks.add(1);
  stats_.allocatedBytes.add(static_cast<int64_t>(nbytes));
  stats_.activeBytes.add(static_cast<int64_t>(nbytes));
  stats_.requestedBytes.add(static_cast<int64_t>(size));
  return p;
}

void BSCachingAllocator::free(void* ptr) {
  if (!ptr) return;
  std::lock_guard<std::mutex> lock(mutex_);
  auto it = live_.find(ptr);
  if (it == live_.end()) throw std::invalid_argument("BS allocator: free of a pointer it did not hand out");
  Pending p;
  p.ptr = ptr;
  p.size = it->second.size;
  EventHandle e = newEvent();
  backend_.recordEvent(e, it->second.stream);
  p.events.push_back(e);
  for (StreamHandle s : it->second.extraStreams) {
    EventHandle x = newEvent();
    backend_.recordEvent(x, s);
    p.events.push_back(x);
  }
  stats_.allocation.add(-1);
  stats_.activeBlocks.add(-1);
  stats_.allocatedBytes.add(-static_cast<int64_t>(p.size));
  stats_.activeBytes.add(-static_cast<int64_t>(p.size));
  live_.erase(it);
  pending_.push_back(std::move(p));
  drainPending(false);
}

void BSCachingAllocator::recordStream(void* ptr, StreamHandle stream) {
  std::lock_guard<std::mutex> lock(mutex_);
  auto it = live_.find(ptr);
  if (it == live_.end()) throw std::invalid_argument("BS allocator: recordStream on a pointer it did not hand out");
  Live& l = it->second;
  if (stream != l.stream && std::find(l.extraStreams.begin(), l.extraStreams.end(), stream) == l.extraStreams.end())
    l.extraStreams.push_back(stream);
}

void BSCachingAllocator::emptyCache() {
  std::lock_guard<std::mutex> lock(mutex_);
  backend_.syncDevice();
  drainPending(true);
  releaseIdle();
}

void BSCachingAllocator::processEvents() {
  std::lock_guard<std::mutex> lock(mutex_);
  drainPending(false);
}

DeviceStats BSCachingAllocator::stats() const {
  std::lock_guard<std::mutex> lock(mutex_);
  return stats_;
}

void BSCachingAllocator::resetPeakStats() {
  std::lock_guard<std::mutex> lock(mutex_);
  for (Stat* st : {&stats_.allocation, &stats_.segment, &stats_.activeBlocks, &stats_.allocatedBytes, &stats_.reservedBytes,
                   &stats_.activeBytes, &stats_.requestedBytes})
    st->peak = st->current;
}

}  // namespace amdrt
}  // namespace dipu
