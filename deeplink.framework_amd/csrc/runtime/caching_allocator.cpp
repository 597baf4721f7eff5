#include "caching_allocator.h"

#include <algorithm>
#include <cstdlib>
#include <sstream>
#include <stdexcept>

namespace dipu {
namespace amdrt {

bool BlockLess::operator()(const Block* a, const Block* b) const {
  if (a->stream != b->stream) return reinterpret_cast<uintptr_t>(a->stream) < reinterpret_cast<uintptr_t>(b->stream);
  if (a->size != b->size) return a->size < b->size;
  return reinterpret_cast<uintptr_t>(a->ptr) < reinterpret_cast<uintptr_t>(b->ptr);
}

// ---------------------------------------------------------------- config ----
bool BlockAddressLess::operator()(const Block* a, const Block* b) const {
  if (a->stream != b->stream) return reinterpret_cast<uintptr_t>(a->stream) < reinterpret_cast<uintptr_t>(b->stream);
  return reinterpret_cast<uintptr_t>(a->ptr) < reinterpret_cast<uintptr_t>(b->ptr);
}

AllocatorConfig AllocatorConfig::parse(const std::string& conf) {
  AllocatorConfig cfg;
  std::stringstream ss(conf);
  std::string item;
  while (std::getline(ss, item, ',')) {
    if (item.empty()) continue;
    auto colon = item.find(':');
    if (colon == std::string::npos) throw std::invalid_argument("allocator conf: missing ':' in '" + item + "'");
    std::string key = item.substr(0, colon), val = item.substr(colon + 1);
    auto trim = [](std::string& s) {
      s.erase(0, s.find_first_not_of(" \t"));
      s.erase(s.find_last_not_of(" \t") + 1);
    };
    trim(key);
    trim(val);
    if (key == "max_split_size_mb") {
      long mb = std::stol(val);
      if (mb <= static_cast<long>(kLargeBuffer / (1024 * 1024)))
        throw std::invalid_argument("allocator conf: max_split_size_mb must exceed 20");
      cfg.maxSplitSize = static_cast<size_t>(mb) * 1024 * 1024;
    } else if (key == "garbage_collection_threshold") {
      double f = std::stod(val);
      if (!(f > 0.0 && f < 1.0)) throw std::invalid_argument("allocator conf: garbage_collection_threshold not in (0,1)");
      cfg.gcThreshold = f;
    } else if (key == "roundup_power2_divisions") {
      long d = std::stol(val);
      if (d < 0 || (d & (d - 1)) != 0) throw std::invalid_argument("allocator conf: roundup_power2_divisions not a power of 2");
      cfg.roundupPower2Divisions = static_cast<size_t>(d);
    } else if (key == "huge_segments") {
      cfg.hugeSegments = (val == "1" || val == "true" || val == "True");
    } else if (key == "expandable_segments") {
      if (val != "True" && val != "False") throw std::invalid_argument("allocator conf: expandable_segments expects True or False");
      cfg.expandableSegments = val == "True";
    } else {
      throw std::invalid_argument("allocator conf: unknown option '" + key + "'");
    }
  }
  return cfg;
}

// ---------------------------------------------------------------- sizing ----
size_t DeviceCachingAllocator::roundSize(size_t size, const AllocatorConfig& cfg) {
  if (size < kMinBlockSize) return kMinBlockSize;
  size_t div = cfg.roundupPower2Divisions;
  if (div > 0 && size > kMinBlockSize * div) {
    // next multiple of (largest power of two <= size) / div
    size_t pow2 = size_t(1) << (63 - __builtin_clzll(static_cast<unsigned long long>(size)));
    size_t step = pow2 / div;
    if (step < kMinBlockSize) step = kMinBlockSize;
    size_t floor = size & ~(step - 1);
    return floor == size ? size : floor + step;
  }
  return kMinBlockSize * ((size + kMinBlockSize - 1) / kMinBlockSize);
}

size_t DeviceCachingAllocator::allocationSize(size_t size, const AllocatorConfig& cfg) {
  if (size <= kSmallSize) return kSmallBuffer;
  if (size < kMinLargeAlloc) return kLargeBuffer;
  if (cfg.hugeSegments && size >= kHugeAlloc) return kRoundHuge * ((size + kRoundHuge - 1) / kRoundHuge);
  return kRoundLarge * ((size + kRoundLarge - 1) / kRoundLarge);
}

DeviceCachingAllocator::DeviceCachingAllocator(RawBackend backend, AllocatorConfig config)
    : backend_(std::move(backend)), config_(config) {}

DeviceCachingAllocator::~DeviceCachingAllocator() {
  // Teardown may run after the device runtime is gone; never throw from here.
  try {
    synchronizeAndFreeEvents();
    releaseBlocks(large_);
    releaseBlocks(small_);
    for (auto e : eventPool_) backend_.destroyEvent(e);
    for (ExpandableRange* es : expandables_) delete es;  // ranges that still hold live blocks at teardown
  } catch (...) {
  }
  for (auto& kv : active_) delete kv.second;
}

// ---------------------------------------------------------------- malloc ----
void DeviceCachingAllocator::recordHistory(bool enabled, size_t maxEntries) {
  std::lock_guard<std::recursive_mutex> lock(mutex_);
  recordHistory_ = enabled;
  traceMax_ = std::max<size_t>(1, maxEntries);
  traceNext_ = 0;
  trace_.clear();
}

void DeviceCachingAllocator::recordTrace(int action, int64_t addr, size_t size, StreamHandle stream) const {
  if (!recordHistory_) return;
  const TraceEntry e{action, addr, size, stream};
  if (trace_.size() < traceMax_) {
    trace_.push_back(e);
  } else {  // full: the oldest entry is overwritten
    trace_[traceNext_] = e;
    traceNext_ = (traceNext_ + 1) % traceMax_;
  }
}

std::vector<TraceEntry> DeviceCachingAllocator::trace() const {
  std::lock_guard<std::recursive_mutex> lock(mutex_);
  std::vector<TraceEntry> out;
  out.reserve(trace_.size());
  out.insert(out.end(), trace_.begin() + static_cast<std::ptrdiff_t>(traceNext_), trace_.end());
  out.insert(out.end(), trace_.begin(), trace_.begin() + static_cast<std::ptrdiff_t>(traceNext_));
  return out;
}

bool DeviceCachingAllocator::shouldSplit(const Block* block, size_t size) const {
  size_t remaining = block->size - size;
  if (block->pool->isSmall) return remaining >= kMinBlockSize;
  return size < config_.maxSplitSize && remaining > kSmallSize;
}

Block* DeviceCachingAllocator::getFreeBlock(BlockPool& pool, size_t size, StreamHandle stream) {
  Block key;
  key.stream = stream;
  key.size = size;
  key.ptr = nullptr;
  auto it = pool.blocks.lower_bound(&key);
  if (it == pool.blocks.end() || (*it)->stream != stream) return nullptr;
  Block* b = *it;
  // Oversize blocks (>= maxSplitSize) serve only requests close to their own size, so a
  // small request does not pin a huge unsplittable block.
  if (size < config_.maxSplitSize && b->size >= config_.maxSplitSize) return nullptr;
  if (size >= config_.maxSplitSize && b->size >= size + kLargeBuffer) return nullptr;
  b->gcCount = 0;
  pool.blocks.erase(it);
  return b;
}

// ---- expandable segments (DIPUCachingDeviceAllocator.cpp:1086-1215, 1633-1705) ----
// One address range per (stream, pool) grows at its end instead of new fixed-size segments being requested: a
// request is served by free mapped blocks followed by enough freshly mapped segments, so a large block can always
// be assembled from what smaller ones left behind.
Block* DeviceCachingAllocator::findExpandableBlock(BlockPool& pool, size_t size, StreamHandle stream) {
  auto allocatable = [](const Block* b) { return b && !b->allocated && b->eventCount == 0 && b->streamUses.empty(); };
  auto roomFrom = [&](const Block* b) {
    size_t bytes = 0;
    while (bytes < size && allocatable(b)) bytes += b->size, b = b->next;
    return bytes >= size;
  };
  Block key;
  key.stream = stream;
  key.ptr = nullptr;
  for (auto it = pool.unmapped.lower_bound(&key); it != pool.unmapped.end() && (*it)->stream == stream; ++it) {
    Block* c = *it;
    if (allocatable(c->prev)) c = c->prev;  // a free mapped block right before the unmapped range is used first
    if (roomFrom(c)) return c;
  }
  ExpandableRange* es = backend_.createExpandable(stream, pool.isSmall ? kSmallBuffer : kLargeBuffer);
  expandables_.push_back(es);
  stats_.segment.add(1);
  Block* candidate = new Block();
  candidate->stream = stream;
  candidate->size = es->size();
  candidate->pool = &pool;
  candidate->ptr = es->ptr();
  candidate->mapped = false;
  candidate->expandable = es;
  pool.unmapped.insert(candidate);
  return candidate;
}

bool DeviceCachingAllocator::mapBlock(Block* toMap, size_t size) {
  char* mp = nullptr;
  size_t ms = 0;
  toMap->expandable->map(static_cast<char*>(toMap->ptr), size, &mp, &ms);
  if (ms == 0) return false;
  BlockPool& pool = *toMap->pool;
  pool.unmapped.erase(toMap);
  toMap->mapped = true;
  if (ms < toMap->size) {  // the rest of the range stays unmapped behind it
    Block* rest = new Block();
    rest->stream = toMap->stream;
    rest->pool = &pool;
    rest->ptr = static_cast<char*>(toMap->ptr) + ms;
    rest->size = toMap->size - ms;
    rest->mapped = false;
    rest->expandable = toMap->expandable;
    rest->prev = toMap;
    rest->next = toMap->next;
    if (rest->next) rest->next->prev = rest;
    toMap->next = rest;
    toMap->size = ms;
    pool.unmapped.insert(rest);
  }
  tryMerge(toMap, toMap->prev, pool);
  tryMerge(toMap, toMap->next, pool);
  pool.blocks.insert(toMap);
  totalReserved_ += ms;
  stats_.reservedBytes.add(static_cast<int64_t>(ms));
  recordTrace(TraceEntry::SEGMENT_MAP, reinterpret_cast<int64_t>(mp), ms, toMap->stream);
  return true;
}

Block* DeviceCachingAllocator::tryAllocateExpandableBlock(BlockPool& pool, size_t size, StreamHandle stream) {
  Block* candidate = findExpandableBlock(pool, size, stream);
  // candidate heads a run of free / unmapped blocks with room for `size`: unmapped, unmapped -> free, free -> unmapped
  if (!candidate->mapped && !mapBlock(candidate, std::min(candidate->size, size))) return nullptr;
  while (candidate->size < size) {  // free -> unmapped: map some of the unmapped part, it merges into the free one
    Block* next = candidate->next;
    if (!mapBlock(next, std::min(size - candidate->size, next->size))) return nullptr;
    candidate = next;  // the free block in front was merged into the newly mapped one
  }
  pool.blocks.erase(candidate);
  return candidate;
}

// Gives the whole segments inside a free block of an expandable range back to the device.
void DeviceCachingAllocator::unmapBlock(Block* block) {
  char* up = nullptr;
  size_t us = 0;
  block->expandable->unmap(static_cast<char*>(block->ptr), block->size, &up, &us);
  if (us == 0) return;
  BlockPool& pool = *block->pool;
  pool.blocks.erase(block);
  const size_t before = static_cast<size_t>(up - static_cast<char*>(block->ptr));
  const size_t after = block->size - before - us;
  auto piece = [&](char* p, size_t n) {
    Block* b = new Block();
    b->stream = block->stream;
    b->pool = &pool;
    b->ptr = p;
    b->size = n;
    b->expandable = block->expandable;
    return b;
  };
  if (before > 0) {  // prev? -> beforeFree -> block
    Block* b = piece(static_cast<char*>(block->ptr), before);
    b->prev = block->prev;
    if (b->prev) b->prev->next = b;
    b->next = block;
    block->prev = b;
    pool.blocks.insert(b);
  }
  if (after > 0) {  // block -> afterFree -> next?
    Block* b = piece(up + us, after);
    b->next = block->next;
    if (b->next) b->next->prev = b;
    b->prev = block;
    block->next = b;
    pool.blocks.insert(b);
  }
  block->ptr = up;
  block->size = us;
  block->mapped = false;
  tryMerge(block, block->prev, pool);
  tryMerge(block, block->next, pool);
  pool.unmapped.insert(block);
  totalReserved_ -= us;
  stats_.reservedBytes.add(-static_cast<int64_t>(us));
  recordTrace(TraceEntry::SEGMENT_UNMAP, reinterpret_cast<int64_t>(up), us, block->stream);
}

void DeviceCachingAllocator::releaseExpandable(Block* block) {
  // the block is the range's only one and nothing of it is mapped
  auto it = std::find(expandables_.begin(), expandables_.end(), block->expandable);
  if (it != expandables_.end()) expandables_.erase(it);
  block->pool->unmapped.erase(block);
  delete block->expandable;
  stats_.segment.add(-1);
  delete block;
}

bool DeviceCachingAllocator::allocBlock(BlockPool& pool, size_t size, size_t allocSize, StreamHandle stream, Block** out) {
  if (config_.expandableSegments && backend_.createExpandable) {
    *out = tryAllocateExpandableBlock(pool, size, stream);
    return *out != nullptr;
  }
  void* p = nullptr;
  ++stats_.numDeviceMalloc;
  if (!backend_.mallocDevice(&p, allocSize) || p == nullptr) return false;
  Block* b = new Block();
  b->stream = stream;
  b->size = allocSize;
  b->pool = &pool;
  b->ptr = p;
  totalReserved_ += allocSize;
  stats_.segment.add(1);
  stats_.reservedBytes.add(static_cast<int64_t>(allocSize));
  recordTrace(TraceEntry::SEGMENT_ALLOC, reinterpret_cast<int64_t>(p), allocSize, stream);
  *out = b;
  return true;
}

void* DeviceCachingAllocator::mallocFromCache(size_t size, StreamHandle stream) {
  std::lock_guard<std::recursive_mutex> lock(mutex_);
  cacheOnly_ = true;
  void* p = nullptr;
  try {
    p = malloc(size, stream);
  } catch (...) {
    cacheOnly_ = false;
    throw;
  }
  cacheOnly_ = false;
  return p;
}

void* DeviceCachingAllocator::malloc(size_t origSize, StreamHandle stream) {
  if (origSize == 0) return nullptr;
  std::lock_guard<std::recursive_mutex> lock(mutex_);
  // A cache-only request comes from inside a stream capture, where an event query may be refused:
  // blocks whose events are still pending stay parked until the next ordinary malloc.
  if (!cacheOnly_) processEvents();
  size_t size = roundSize(origSize, config_);
  BlockPool& pool = size <= kSmallSize ? small_ : large_;
  size_t allocSize = allocationSize(size, config_);

  Block* block = getFreeBlock(pool, size, stream);
  if (!block && cacheOnly_) return nullptr;
  if (!block) {
    if (config_.gcThreshold > 0.0) garbageCollect();
    bool ok = allocBlock(pool, size, allocSize, stream, &block);
    if (!ok) {
      ++stats_.numAllocRetries;
      ok = releaseAvailableCachedBlocks(pool, allocSize, stream) && allocBlock(pool, size, allocSize, stream, &block);
    }
    if (!ok) {
      ++stats_.numAllocRetries;
      ok = releaseCachedBlocks() && allocBlock(pool, size, allocSize, stream, &block);
    }
    if (!ok) {
      ++stats_.numOoms;
      recordTrace(TraceEntry::OOM, static_cast<int64_t>(allocSize), origSize, stream);
      std::ostringstream os;
      os << "HIP out of memory. Tried to allocate " << allocSize << " bytes (request " << origSize << "). "
         << stats_.allocatedBytes.current << " bytes allocated, " << stats_.reservedBytes.current
         << " bytes reserved by the caching allocator.";
      throw OutOfMemory(os.str());
    }
  }

  const bool alreadySplit = block->isSplit();
  if (!shouldSplit(block, size)) {
    if (alreadySplit) {  // an inactive split block becomes active as a whole
      stats_.inactiveSplit.add(-1);
      stats_.inactiveSplitBytes.add(-static_cast<int64_t>(block->size));
    }
  } else if (alreadySplit) {  // an inactive split block shrinks by `size` bytes
    stats_.inactiveSplitBytes.add(-static_cast<int64_t>(block->size));
    stats_.inactiveSplit.add(-1);
  }
  if (shouldSplit(block, size)) {
    Block* rem = new Block();
    rem->stream = block->stream;
    rem->pool = block->pool;
    rem->ptr = static_cast<char*>(block->ptr) + size;
    rem->size = block->size - size;
    rem->expandable = block->expandable;
    rem->prev = block;
    rem->next = block->next;
    if (rem->next) rem->next->prev = rem;
    block->next = rem;
    block->size = size;
    pool.blocks.insert(rem);
    stats_.inactiveSplit.add(1);
    stats_.inactiveSplitBytes.add(static_cast<int64_t>(rem->size));
  }
  block->allocated = true;
  block->requested = origSize;
  active_[block->ptr] = block;
  stats_.allocation.add(1);
  stats_.allocatedBytes.add(static_cast<int64_t>(block->size));
  stats_.activeBlocks.add(1);
  stats_.activeBytes.add(static_cast<int64_t>(block->size));
  stats_.requestedBytes.add(static_cast<int64_t>(origSize));
  recordTrace(TraceEntry::ALLOC, reinterpret_cast<int64_t>(block->ptr), origSize, block->stream);
  return block->ptr;
}

// ------------------------------------------------------------------ free ----
void DeviceCachingAllocator::free(void* ptr) {
  if (ptr == nullptr) return;
  std::lock_guard<std::recursive_mutex> lock(mutex_);
  auto it = active_.find(ptr);
  if (it == active_.end()) throw std::invalid_argument("caching allocator: free of an unknown pointer");
  Block* block = it->second;
  active_.erase(it);
  block->allocated = false;
  stats_.allocation.add(-1);
  stats_.allocatedBytes.add(-static_cast<int64_t>(block->size));
  stats_.requestedBytes.add(-static_cast<int64_t>(block->requested));
  recordTrace(TraceEntry::FREE_REQUESTED, reinterpret_cast<int64_t>(block->ptr), block->requested, block->stream);
  if (!block->streamUses.empty()) {
    insertEvents(block);  // reuse waits until every recorded stream has passed this point
  } else {
    freeBlock(block);
  }
}

size_t DeviceCachingAllocator::tryMerge(Block* dst, Block* src, BlockPool& pool) {
  if (!src || src->allocated || src->eventCount > 0 || !src->streamUses.empty() || dst->mapped != src->mapped) return 0;
  if (dst->prev == src) {
    dst->ptr = src->ptr;
    dst->prev = src->prev;
    if (dst->prev) dst->prev->next = dst;
  } else {
    dst->next = src->next;
    if (dst->next) dst->next->prev = dst;
  }
  size_t subsumed = src->size;
  dst->size += subsumed;
  if (src->mapped) pool.blocks.erase(src); else pool.unmapped.erase(src);
  delete src;
  return subsumed;
}

void DeviceCachingAllocator::freeBlock(Block* block) {
  size_t origSize = block->size;
  recordTrace(TraceEntry::FREE_COMPLETED, reinterpret_cast<int64_t>(block->ptr), block->requested, block->stream);
  BlockPool& pool = *block->pool;
  int64_t netInactiveBlocks = 0, netInactiveBytes = 0;
  Block* neighbours[2] = {block->prev, block->next};
  for (Block* n : neighbours) {
    size_t subsumed = tryMerge(block, n, pool);
    if (subsumed > 0) {
      netInactiveBlocks -= 1;
      netInactiveBytes -= static_cast<int64_t>(subsumed);
    }
  }
  pool.blocks.insert(block);
  if (block->isSplit()) {
    netInactiveBlocks += 1;
    netInactiveBytes += static_cast<int64_t>(block->size);
  }
  stats_.inactiveSplit.add(netInactiveBlocks);
  stats_.inactiveSplitBytes.add(netInactiveBytes);
  stats_.activeBlocks.add(-1);
  stats_.activeBytes.add(-static_cast<int64_t>(origSize));
}

void DeviceCachingAllocator::recordStream(void* ptr, StreamHandle stream) {
  std::lock_guard<std::recursive_mutex> lock(mutex_);
  auto it = active_.find(ptr);
  if (it == active_.end()) return;
  if (stream == it->second->stream) return;  // the allocating stream orders reuse by itself
  it->second->streamUses.insert(stream);
}

void DeviceCachingAllocator::insertEvents(Block* block) {
  std::unordered_set<StreamHandle> streams;
  streams.swap(block->streamUses);
  for (StreamHandle s : streams) {
    EventHandle e;
    if (!eventPool_.empty()) {
      e = eventPool_.back();
      eventPool_.pop_back();
    } else {
      e = backend_.createEvent();
    }
    backend_.recordEvent(e, s);
    ++block->eventCount;
    events_[s].emplace_back(e, block);
  }
}

void DeviceCachingAllocator::processEvents() {
  std::lock_guard<std::recursive_mutex> lock(mutex_);
  for (auto it = events_.begin(); it != events_.end();) {
    auto& q = it->second;
    size_t done = 0;
    // events of one stream complete in order: stop at the first pending one
    while (done < q.size() && backend_.eventReady(q[done].first)) {
      eventPool_.push_back(q[done].first);
      Block* b = q[done].second;
      if (--b->eventCount == 0) freeBlock(b);
      ++done;
    }
    q.erase(q.begin(), q.begin() + static_cast<long>(done));
    it = q.empty() ? events_.erase(it) : std::next(it);
  }
}

void DeviceCachingAllocator::synchronizeAndFreeEvents() {
  if (events_.empty()) return;
  backend_.syncDevice();
  for (auto& kv : events_) {
    for (auto& eb : kv.second) {
      eventPool_.push_back(eb.first);
      if (--eb.second->eventCount == 0) freeBlock(eb.second);
    }
  }
  events_.clear();
}

// --------------------------------------------------------------- release ----
void DeviceCachingAllocator::releaseBlock(Block* block) {
  recordTrace(TraceEntry::SEGMENT_FREE, reinterpret_cast<int64_t>(block->ptr), block->size, block->stream);
  backend_.freeDevice(block->ptr);
  ++stats_.numDeviceFree;
  totalReserved_ -= block->size;
  stats_.segment.add(-1);
  stats_.reservedBytes.add(-static_cast<int64_t>(block->size));
  block->pool->blocks.erase(block);
  delete block;
}

void DeviceCachingAllocator::releaseBlocks(BlockPool& pool) {
  std::vector<Block*> toUnmap;  // unmapping changes the pool: collect first
  for (auto it = pool.blocks.begin(); it != pool.blocks.end();) {
    Block* b = *it;
    ++it;
    if (b->expandable) toUnmap.push_back(b);
    else if (!b->prev && !b->next) releaseBlock(b);  // only whole segments go back to the device
  }
  for (Block* b : toUnmap) {
    unmapBlock(b);
    if (!b->mapped && !b->prev && !b->next) releaseExpandable(b);  // nothing of the range is in use any more
  }
}

bool DeviceCachingAllocator::releaseAvailableCachedBlocks(BlockPool& pool, size_t size, StreamHandle stream) {
  if (config_.maxSplitSize == SIZE_MAX) return false;
  Block key;
  key.stream = stream;
  key.size = size < config_.maxSplitSize ? config_.maxSplitSize : size;
  key.ptr = nullptr;
  auto it = pool.blocks.lower_bound(&key);
  if (it == pool.blocks.end() || (*it)->stream != stream) {
    // no single block is large enough: free oversize blocks, largest first, until enough
    if (it == pool.blocks.begin()) return false;
    size_t freed = 0;
    --it;
    while (freed < size && (*it)->size >= config_.maxSplitSize && (*it)->stream == stream) {
      Block* cur = *it;
      bool atBegin = it == pool.blocks.begin();
      if (!atBegin) --it;
      if (!cur->prev && !cur->next && !cur->expandable) {
        freed += cur->size;
        releaseBlock(cur);
      }
      if (atBegin) break;
    }
    return freed >= size;
  }
  if ((*it)->prev || (*it)->next || (*it)->expandable) return false;
  releaseBlock(*it);
  return true;
}

bool DeviceCachingAllocator::releaseCachedBlocks() {
  synchronizeAndFreeEvents();
  releaseBlocks(large_);
  releaseBlocks(small_);
  return true;
}

void DeviceCachingAllocator::emptyCache() {
  std::lock_guard<std::recursive_mutex> lock(mutex_);
  releaseCachedBlocks();
}

// Frees cached large segments, oldest first, until reserved memory is back under the
// configured fraction of the device.
void DeviceCachingAllocator::garbageCollect() {
  if (config_.deviceCapacity == 0) return;
  size_t limit = static_cast<size_t>(config_.gcThreshold * static_cast<double>(config_.deviceCapacity));
  if (totalReserved_ <= limit) return;
  size_t target = totalReserved_ - limit, freed = 0;
  int64_t totalAge = 0, count = 0;
  for (Block* b : large_.blocks)
    if (!b->isSplit() && !b->expandable) totalAge += ++b->gcCount, ++count;  // parts of expandable ranges stay
  if (count == 0) return;
  bool progressed = true;
  while (freed < target && progressed && count > 0) {
    double avg = static_cast<double>(totalAge) / static_cast<double>(count);
    progressed = false;
    for (auto it = large_.blocks.begin(); it != large_.blocks.end() && freed < target;) {
      Block* b = *it;
      ++it;
      if (!b->isSplit() && !b->expandable && static_cast<double>(b->gcCount) >= avg) {
        freed += b->size;
        totalAge -= b->gcCount;
        --count;
        releaseBlock(b);
        progressed = true;
      }
    }
  }
}

// ----------------------------------------------------------------- stats ----
DeviceStats DeviceCachingAllocator::stats() const {
  std::lock_guard<std::recursive_mutex> lock(mutex_);
  return stats_;
}

void DeviceCachingAllocator::resetPeakStats() {
  std::lock_guard<std::recursive_mutex> lock(mutex_);
  Stat* all[] = {&stats_.allocation,     &stats_.segment,     &stats_.activeBlocks,       &stats_.inactiveSplit,
                 &stats_.allocatedBytes, &stats_.reservedBytes, &stats_.activeBytes,      &stats_.inactiveSplitBytes,
                 &stats_.requestedBytes};
  for (Stat* s : all) s->peak = s->current;
}

size_t DeviceCachingAllocator::blockSize(void* ptr) const {
  std::lock_guard<std::recursive_mutex> lock(mutex_);
  auto it = active_.find(ptr);
  return it == active_.end() ? 0 : it->second->size;
}

std::vector<SegmentInfo> DeviceCachingAllocator::snapshot() const {
  std::lock_guard<std::recursive_mutex> lock(mutex_);
  std::vector<const Block*> heads;
  auto visit = [&](const Block* b) {
    if (b->prev == nullptr) heads.push_back(b);
  };
  for (const Block* b : small_.blocks) visit(b);
  for (const Block* b : large_.blocks) visit(b);
  for (const auto& kv : active_) visit(kv.second);
  for (const auto& kv : events_)
    for (const auto& eb : kv.second) visit(eb.second);
  std::sort(heads.begin(), heads.end(), [](const Block* a, const Block* b) { return a->ptr < b->ptr; });
  heads.erase(std::unique(heads.begin(), heads.end()), heads.end());
  std::vector<SegmentInfo> out;
  for (const Block* h : heads) {
    SegmentInfo s{h->ptr, 0, 0, 0, !h->pool->isSmall, 0};
    for (const Block* b = h; b; b = b->next) {
      if (!b->mapped) continue;  // address space only
      s.totalSize += b->size;
      if (b->allocated) s.allocatedSize += b->size;
      if (b->allocated || b->eventCount > 0) s.activeSize += b->size;
      ++s.numBlocks;
    }
    out.push_back(s);
  }
  size_t active = 0;
  for (const SegmentInfo& si : out) active += si.activeSize;
  recordTrace(TraceEntry::SNAPSHOT, 0, active, nullptr);
  return out;
}

// ------------------------------------------------------------------- RAW ----
void* RawAllocator::malloc(size_t size) {
  if (size == 0) return nullptr;
  size_t rounded = kMinBlockSize * ((size + kMinBlockSize - 1) / kMinBlockSize);
  void* p = nullptr;
  std::lock_guard<std::mutex> lock(mutex_);
  ++stats_.numDeviceMalloc;
  if (!backend_.mallocDevice(&p, rounded) || !p) {
    ++stats_.numOoms;
    throw OutOfMemory("HIP out of memory (raw allocator), tried to allocate " + std::to_string(rounded) + " bytes");
  }
  live_[p] = rounded;
  stats_.allocation.add(1);
  stats_.allocatedBytes.add(static_cast<int64_t>(rounded));
  stats_.reservedBytes.add(static_cast<int64_t>(rounded));
  return p;
}

void RawAllocator::free(void* ptr) {
  if (!ptr) return;
  std::lock_guard<std::mutex> lock(mutex_);
  auto it = live_.find(ptr);
  if (it == live_.end()) throw std::invalid_argument("raw allocator: free of an unknown pointer");
  backend_.syncDevice();  // pending kernels may still read the buffer
  backend_.freeDevice(ptr);
  ++stats_.numDeviceFree;
  stats_.allocation.add(-1);
  stats_.allocatedBytes.add(-static_cast<int64_t>(it->second));
  stats_.reservedBytes.add(-static_cast<int64_t>(it->second));
  live_.erase(it);
}

DeviceStats RawAllocator::stats() const {
  std::lock_guard<std::mutex> lock(mutex_);
  return stats_;
}

}  // namespace amdrt
}  // namespace dipu
