// The BF ("best fit" by size class) device caching algorithm, selected with DIPU_DEVICE_MEMCACHING_ALGORITHM=BF.
// Behaviour follows dipu/torch_dipu/csrc_dipu/runtime/core/allocator/DIPUBFCachingAllocator.cpp:21-405 (size classes
// :171-187, lookup :233-252, split rule :375-378, merge :284-301, extend :303-331, shrink :254-267) and its
// event-deferred release (:414-548); the data structures are this backend's own (pointer-linked chunks, one mutex).
#include <algorithm>
#include <cstdlib>
#include <stdexcept>
#include <string>
#include <thread>

#include "caching_allocator.h"

namespace dipu {
namespace amdrt {

namespace {
size_t round512(size_t n) { return ((n - 1) | (kMinBlockSize - 1)) + 1; }

size_t maxExtendFromEnv() {
  const char* e = std::getenv("DIPU_MAX_EXTEND_SIZE");  // MiB
  const long v = e ? std::atol(e) : 1024;
  return static_cast<size_t>(v > 0 ? v : 1024) << 20;
}
}  // namespace

BFCachingAllocator::BFCachingAllocator(RawBackend backend, size_t maxExtendBytes)
    : backend_(std::move(backend)), maxExtend_(maxExtendBytes ? maxExtendBytes : maxExtendFromEnv()) {}

BFCachingAllocator::~BFCachingAllocator() {
  try {
    std::lock_guard<std::mutex> lock(mutex_);
    backend_.syncDevice();
    drainPending(true);
    releaseWholeChunks();
    for (EventHandle e : eventPool_) backend_.destroyEvent(e);
  } catch (...) {
  }
}

// Class of a size: 4 * floor(log2(units)) + the two bits below the leading one, units = size / 512.
int BFCachingAllocator::binOf(size_t nbytes) {
  const unsigned long long units = nbytes / kMinBlockSize;
  const int top = 63 - __builtin_clzll(units ? units : 1);
  if (top >= kBigBins) return kBins - 1;
  const unsigned long long below = units ^ (1ull << top);
  const int sub = static_cast<int>(top >= 2 ? below >> (top - 2) : below);
  return top * kSubBins + sub;
}

void BFCachingAllocator::pushFree(Chunk* c) {
  c->bin = binOf(c->size);
  c->binPrev = nullptr;
  c->binNext = heads_[c->bin];
  if (c->binNext) c->binNext->binPrev = c;
  heads_[c->bin] = c;
  occupied_ |= static_cast<unsigned __int128>(1) << c->bin;
}

void BFCachingAllocator::popFree(Chunk* c) {
  if (c->binPrev) c->binPrev->binNext = c->binNext; else heads_[c->bin] = c->binNext;
  if (c->binNext) c->binNext->binPrev = c->binPrev;
  if (!heads_[c->bin]) occupied_ &= ~(static_cast<unsigned __int128>(1) << c->bin);
  c->binPrev = c->binNext = nullptr;
  c->bin = -1;
}

// First chunk of the request's own class if it is large enough, else the first chunk of the next occupied class.
BFCachingAllocator::Chunk* BFCachingAllocator::take(size_t nbytes) {
  const int least = binOf(nbytes);
  Chunk* c = heads_[least];
  if (c && c->size < nbytes) c = nullptr;
  if (!c && least + 1 < kBins) {
    const unsigned __int128 above = occupied_ >> (least + 1);
    if (above) {
      const unsigned long long lo = static_cast<unsigned long long>(above), hi = static_cast<unsigned long long>(above >> 64);
      const int first = lo ? __builtin_ctzll(lo) : 64 + __builtin_ctzll(hi);
      c = heads_[least + 1 + first];
    }
  }
  if (c) popFree(c);
  return c;
}

void BFCachingAllocator::releaseWholeChunks() {
  for (int b = 0; b < kBins; ++b) {
    Chunk* c = heads_[b];
    while (c) {
      Chunk* next = c->binNext;
      if (c->whole()) {
        popFree(c);
        backend_.freeDevice(c->ptr);
        stats_.reservedBytes.add(-static_cast<int64_t>(c->size));
        stats_.segment.add(-1);
        ++stats_.numDeviceFree;
        delete c;
      }
      c = next;
    }
  }
}

BFCachingAllocator::Chunk* BFCachingAllocator::extend(size_t nbytes) {
  releaseWholeChunks();
  bool grew = false;
  while (extendSize_ < nbytes && extendSize_ < maxExtend_) extendSize_ *= 2, grew = true;
  size_t bytes = std::max(nbytes, extendSize_);
  void* p = nullptr;
  if (backend_.mallocDevice(&p, bytes)) {
    if (!grew && extendSize_ < maxExtend_) extendSize_ *= 2;
  } else if (bytes > nbytes) {
    bytes = nbytes;
    if (!backend_.mallocDevice(&p, bytes)) p = nullptr;
  } else {
    p = nullptr;
  }
  if (!p) return nullptr;
  ++stats_.numDeviceMalloc;
  stats_.reservedBytes.add(static_cast<int64_t>(bytes));
  stats_.segment.add(1);
  auto* c = new Chunk();
  c->ptr = static_cast<char*>(p);
  c->size = bytes;
  return c;
}

EventHandle BFCachingAllocator::newEvent() {
  if (!eventPool_.empty()) {
    EventHandle e = eventPool_.back();
    eventPool_.pop_back();
    return e;
  }
  return backend_.createEvent();
}

// A chunk whose events have all completed goes back to the free lists, merged with its free neighbours.
void BFCachingAllocator::giveBack(Chunk* c) {
  c->allocated = false;
  c->extraStreams.clear();
  if (Chunk* n = c->after; n && !n->allocated && n->bin >= 0) {
    popFree(n);
    c->size += n->size;
    c->after = n->after;
    if (c->after) c->after->before = c;
    delete n;
  }
  if (Chunk* b = c->before; b && !b->allocated && b->bin >= 0) {
    popFree(b);
    b->size += c->size;
    b->after = c->after;
    if (b->after) b->after->before = b;
    delete c;
    c = b;
  }
  pushFree(c);
}

bool BFCachingAllocator::drainPending(bool wait) {
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
      giveBack(p.chunk);
    } else {
      if (kept != i) pending_[kept] = std::move(p);
      ++kept;
    }
  }
  const bool all = kept == 0;
  pending_.resize(kept);
  return all;
}

void* BFCachingAllocator::malloc(size_t size, StreamHandle stream) {
  if (size == 0) return nullptr;
  const size_t nbytes = round512(size);
  std::lock_guard<std::mutex> lock(mutex_);
  drainPending(false);
  Chunk* c = take(nbytes);
  if (!c) c = extend(nbytes);
  if (!c && !pending_.empty()) {  // wait for what is on its way back, then look again
    ++stats_.numAllocRetries;
    backend_.syncDevice();
    drainPending(true);
    c = take(nbytes);
    if (!c) c = extend(nbytes);
  }
  if (!c) {
    ++stats_.numOoms;
    throw OutOfMemory("BF allocator: no memory available for " + std::to_string(nbytes) + " bytes (" +
                      std::to_string(stats_.reservedBytes.current) + " reserved, " +
                      std::to_string(stats_.allocatedBytes.current) + " allocated)");
  }
  if (c->size >= nbytes * 2 || c->size >= nbytes + kMaxInternalFragmentation) {
    auto* rest = new Chunk();
    rest->ptr = c->ptr + nbytes;
    rest->size = c->size - nbytes;
    rest->before = c;
    rest->after = c->after;
    if (rest->after) rest->after->before = rest;
    c->after = rest;
    c->size = nbytes;
    pushFree(rest);
  }
  c->allocated = true;
  c->requested = nbytes;
  c->stream = stream;
  live_[c->ptr] = c;
  stats_.allocation.add(1);
  stats_.activeBlocks.add(1);
  stats_.allocatedBytes.add(static_cast<int64_t>(nbytes));
  stats_.activeBytes.add(static_cast<int64_t>(c->size));
  stats_.requestedBytes.add(static_cast<int64_t>(size));
  return c->ptr;
}

void BFCachingAllocator::free(void* ptr) {
  if (!ptr) return;
  std::lock_guard<std::mutex> lock(mutex_);
  auto it = live_.find(ptr);
  if (it == live_.end()) throw std::invalid_argument("BF allocator: free of a pointer it did not hand out");
  Chunk* c = it->second;
  live_.erase(it);
  stats_.allocation.add(-1);
  stats_.activeBlocks.add(-1);
  stats_.allocatedBytes.add(-static_cast<int64_t>(c->requested));
  stats_.activeBytes.add(-static_cast<int64_t>(c->size));
  Pending p;
  p.chunk = c;
  EventHandle e = newEvent();
  backend_.recordEvent(e, c->stream);
  p.events.push_back(e);
  for (StreamHandle s : c->extraStreams) {
    EventHandle x = newEvent();
    backend_.recordEvent(x, s);
    p.events.push_back(x);
  }
  pending_.push_back(std::move(p));
  drainPending(false);
}

void BFCachingAllocator::recordStream(void* ptr, StreamHandle stream) {
  std::lock_guard<std::mutex> lock(mutex_);
  auto it = live_.find(ptr);
  if (it == live_.end()) throw std::invalid_argument("BF allocator: recordStream on a pointer it did not hand out");
  Chunk* c = it->second;
  if (stream == c->stream) return;
  if (std::find(c->extraStreams.begin(), c->extraStreams.end(), stream) == c->extraStreams.end()) c->extraStreams.push_back(stream);
}

void BFCachingAllocator::emptyCache() {
  std::lock_guard<std::mutex> lock(mutex_);
  backend_.syncDevice();
  drainPending(true);
  releaseWholeChunks();
}

void BFCachingAllocator::processEvents() {
  std::lock_guard<std::mutex> lock(mutex_);
  drainPending(false);
}

DeviceStats BFCachingAllocator::stats() const {
  std::lock_guard<std::mutex> lock(mutex_);
  return stats_;
}

void BFCachingAllocator::resetPeakStats() {
  std::lock_guard<std::mutex> lock(mutex_);
  for (Stat* st : {&stats_.allocation, &stats_.segment, &stats_.activeBlocks, &stats_.allocatedBytes, &stats_.reservedBytes,
                   &stats_.activeBytes, &stats_.requestedBytes})
    st->peak = st->current;
}

}  // namespace amdrt
}  // namespace dipu
