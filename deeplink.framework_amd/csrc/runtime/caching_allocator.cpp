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
      // accepted for configuration compatibility; this backend sizes segments instead
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
  } catch (...) {
  }
  for (auto& kv : active_) delete kv.second;
}

// ---------------------------------------------------------------- malloc ----
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

bool DeviceCachingAllocator::allocBlock(BlockPool& pool, size_t allocSize, StreamHandle stream, Block** out) {
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
  *out = b;
  return true;
}

void* DeviceCachingAllocator::malloc(size_t origSize, StreamHandle stream) {
  if (origSize == 0) return nullptr;
  std::lock_guard<std::recursive_mutex> lock(mutex_);
  processEvents();
  size_t size = roundSize(origSize, config_);
  BlockPool& pool = size <= kSmallSize ? small_ : large_;
  size_t allocSize = allocationSize(size, config_);

  Block* block = getFreeBlock(pool, size, stream);
  if (!block) {
    if (config_.gcThreshold > 0.0) garbageCollect();
    bool ok = allocBlock(pool, allocSize, stream, &block);
    if (!ok) {
      ++stats_.numAllocRetries;
      ok = releaseAvailableCachedBlocks(pool, allocSize, stream) && allocBlock(pool, allocSize, stream, &block);
    }
    if (!ok) {
      ++stats_.numAllocRetries;
      ok = releaseCachedBlocks() && allocBlock(pool, allocSize, stream, &block);
    }
    if (!ok) {
      ++stats_.numOoms;
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
  if (!block->streamUses.empty()) {
    insertEvents(block);  // reuse waits until every recorded stream has passed this point
  } else {
    freeBlock(block);
  }
}

size_t DeviceCachingAllocator::tryMerge(Block* dst, Block* src, BlockPool& pool) {
  if (!src || src->allocated || src->eventCount > 0 || !src->streamUses.empty()) return 0;
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
  pool.blocks.erase(src);
  delete src;
  return subsumed;
}

void DeviceCachingAllocator::freeBlock(Block* block) {
  size_t origSize = block->size;
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
  backend_.freeDevice(block->ptr);
  ++stats_.numDeviceFree;
  totalReserved_ -= block->size;
  stats_.segment.add(-1);
  stats_.reservedBytes.add(-static_cast<int64_t>(block->size));
  block->pool->blocks.erase(block);
  delete block;
}

void DeviceCachingAllocator::releaseBlocks(BlockPool& pool) {
  for (auto it = pool.blocks.begin(); it != pool.blocks.end();) {
    Block* b = *it;
    ++it;
    if (!b->prev && !b->next) releaseBlock(b);  // only whole segments go back to the device
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
      if (!cur->prev && !cur->next) {
        freed += cur->size;
        releaseBlock(cur);
      }
      if (atBegin) break;
    }
    return freed >= size;
  }
  if ((*it)->prev || (*it)->next) return false;
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
    if (!b->isSplit()) totalAge += ++b->gcCount, ++count;
  if (count == 0) return;
  bool progressed = true;
  while (freed < target && progressed && count > 0) {
    double avg = static_cast<double>(totalAge) / static_cast<double>(count);
    progressed = false;
    for (auto it = large_.blocks.begin(); it != large_.blocks.end() && freed < target;) {
      Block* b = *it;
      ++it;
      if (!b->isSplit() && static_cast<double>(b->gcCount) >= avg) {
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
      s.totalSize += b->size;
      if (b->allocated) s.allocatedSize += b->size;
      if (b->allocated || b->eventCount > 0) s.activeSize += b->size;
      ++s.numBlocks;
    }
    out.push_back(s);
  }
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
