// Device caching allocator for the AMD backend (288 GB HBM3E per MI355X).
//
// Behavioural model: DIPU's default "TORCH" device algorithm
// (dipu/torch_dipu/csrc_dipu/runtime/core/allocator/DIPUCachingDeviceAllocator.cpp:84-95
// constants, :584-714 malloc ladder, :833-837 event-deferred free, :1055-1065 rounding,
// :1306-1343 pools/splitting) plus the RAW pass-through used for debugging
// (DIPURawCachingAllocator.cpp). The selection variable and spelling are DIPU's
// (dipu/torch_dipu/csrc_dipu/base/environ.hpp:88-92).
//
// The allocator talks to the device only through RawBackend, so the whole state
// machine (rounding, pools, split/merge, stream-ordered reuse, deferred free,
// out-of-memory ladder, statistics) is exercised on a CPU-only machine with a
// host-memory backend.
#pragma once

#include <cstddef>
#include <cstdint>
#include <functional>
#include <memory>
#include <mutex>
#include <set>
#include <string>
#include <unordered_map>
#include <unordered_set>
#include <vector>

namespace dipu {
namespace amdrt {

using StreamHandle = void*;
using EventHandle = void*;

// A reserved address range whose segments are backed and released on demand (DIPU's ExpandableSegment,
// runtime/core/allocator/ExpandableSegment.h:114-136). map() backs every segment the range touches and reports what
// is mapped now (size 0: out of memory, nothing changed); unmap() releases the segments entirely inside the range.
struct ExpandableRange {
  virtual ~ExpandableRange() = default;
  virtual void map(char* ptr, size_t size, char** mappedPtr, size_t* mappedSize) = 0;
  virtual void unmap(char* ptr, size_t size, char** unmappedPtr, size_t* unmappedSize) = 0;
  virtual char* ptr() const = 0;
  virtual size_t size() const = 0;
};

struct RawBackend {
  // returns false on out-of-memory (never throws for OOM)
  std::function<bool(void** p, size_t nbytes)> mallocDevice;
  // null when the device has no virtual memory management: expandable_segments:True is then ignored, as the
  // reference ignores it without vendorCreateExpandableSegment (DIPUCachingDeviceAllocator.cpp:481-487)
  std::function<ExpandableRange*(StreamHandle stream, size_t segmentSize)> createExpandable;
  std::function<void(void* p)> freeDevice;
  std::function<EventHandle()> createEvent;
  std::function<void(EventHandle)> destroyEvent;
  std::function<void(EventHandle, StreamHandle)> recordEvent;
  std::function<bool(EventHandle)> eventReady;
  std::function<void()> syncDevice;
  static RawBackend hip();  // devapis-backed
};

constexpr size_t kMinBlockSize = 512;          // every size is a multiple of 512 B
constexpr size_t kSmallSize = 1048576;         // requests up to 1 MiB use the small pool
constexpr size_t kSmallBuffer = 2097152;       // small pool segments are 2 MiB
constexpr size_t kLargeBuffer = 20971520;      // 1..10 MiB requests share 20 MiB segments
constexpr size_t kMinLargeAlloc = 10485760;
constexpr size_t kRoundLarge = 2097152;        // larger requests round up to 2 MiB
// Requests of 1 GiB and more get segments rounded to 64 MiB: with 288 GB per device the
// slack is negligible and a later request of a similar size can reuse the segment.
constexpr size_t kHugeAlloc = size_t(1) << 30;
constexpr size_t kRoundHuge = size_t(64) << 20;

struct AllocatorConfig {
  size_t maxSplitSize = SIZE_MAX;        // blocks of at least this size are never split
  double gcThreshold = 0.0;              // fraction of device capacity; 0 = off
  size_t roundupPower2Divisions = 0;     // 0 = plain 512 B rounding
  bool hugeSegments = true;
  bool expandableSegments = false;       // expandable_segments:True
  size_t deviceCapacity = 0;             // for gcThreshold; 0 = unknown
  // Parses DIPU's "max_split_size_mb:N,garbage_collection_threshold:F,roundup_power2_divisions:N"
  // (dipu/.../DIPUCachingDeviceAllocator.cpp:454-496). Unknown keys raise std::invalid_argument.
  static AllocatorConfig parse(const std::string& conf);
};

struct Stat {
  int64_t current = 0, peak = 0, allocated = 0, freed = 0;
  void add(int64_t v) {
    current += v;
    if (v > 0) allocated += v; else freed += -v;
    if (current > peak) peak = current;
  }
};

struct DeviceStats {
  Stat allocation, segment, activeBlocks, inactiveSplit;
  Stat allocatedBytes, reservedBytes, activeBytes, inactiveSplitBytes, requestedBytes;
  int64_t numAllocRetries = 0, numOoms = 0, numDeviceMalloc = 0, numDeviceFree = 0;
};

struct Block;
struct BlockLess {
  bool operator()(const Block* a, const Block* b) const;
};
struct BlockAddressLess {
  bool operator()(const Block* a, const Block* b) const;
};
struct BlockPool {
  std::set<Block*, BlockLess> blocks;
  std::set<Block*, BlockAddressLess> unmapped;  // address ranges of expandable segments with nothing behind them
  bool isSmall;
  explicit BlockPool(bool small) : isSmall(small) {}
};

struct Block {
  StreamHandle stream = nullptr;
  std::unordered_set<StreamHandle> streamUses;
  size_t size = 0;
  size_t requested = 0;
  BlockPool* pool = nullptr;
  void* ptr = nullptr;
  bool allocated = false;
  Block* prev = nullptr;
  Block* next = nullptr;
  int eventCount = 0;
  int gcCount = 0;
  bool mapped = true;                  // false: part of an expandable segment's range with no memory behind it
  ExpandableRange* expandable = nullptr;
  bool isSplit() const { return prev != nullptr || next != nullptr; }
};

// One step of the allocator's history (DIPUCachingDeviceAllocator.h:134-164, without the Python stack context).
struct TraceEntry {
  enum Action {
    ALLOC = 0,           // a request served (addr, requested size)
    FREE_REQUESTED = 1,  // free() called
    FREE_COMPLETED = 2,  // the block actually went back to the pool (after the events of recordStream, if any)
    SEGMENT_ALLOC = 3,   // memory taken from the device
    SEGMENT_FREE = 4,    // memory given back to the device
    SEGMENT_MAP = 5,     // expandable segments: part of a range mapped
    SEGMENT_UNMAP = 6,   // expandable segments: part of a range unmapped
    SNAPSHOT = 7,        // snapshot() called (size = active bytes)
    OOM = 8              // OutOfMemory thrown (addr = bytes the request would have taken from the device)
  };
  int action;
  int64_t addr;
  size_t size;
  StreamHandle stream;
};

struct SegmentInfo {
  void* address;
  size_t totalSize, allocatedSize, activeSize;
  bool isLarge;
  int numBlocks;
};

// What the runtime needs from a device allocator, whichever algorithm DIPU_DEVICE_MEMCACHING_ALGORITHM selects.
class DeviceAllocator {
 public:
  virtual ~DeviceAllocator() = default;
  // Never returns nullptr for size > 0; throws OutOfMemory once every way of finding the bytes has failed.
  virtual void* malloc(size_t size, StreamHandle stream) = 0;
  // A block out of the cache or nullptr: never calls the device allocator, never synchronises, records no event.
  // For requests made while `stream` is being captured into a graph. nullptr also means "not supported".
  virtual void* mallocFromCache(size_t size, StreamHandle stream) {
    (void)size, (void)stream;
    return nullptr;
  }
  virtual void free(void* ptr) = 0;
  // `ptr` is also being used on `stream`; its reuse waits for an event on that stream.
  virtual void recordStream(void* ptr, StreamHandle stream) = 0;
  virtual void emptyCache() = 0;
  virtual void processEvents() = 0;
  virtual DeviceStats stats() const = 0;
  virtual void resetPeakStats() = 0;
  // History of the allocator's steps; only the TORCH algorithm keeps one (the others ignore the switch).
  virtual void recordHistory(bool /*enabled*/, size_t /*maxEntries*/) {}
  virtual bool isHistoryEnabled() const { return false; }
  virtual std::vector<TraceEntry> trace() const { return {}; }
};

class DeviceCachingAllocator : public DeviceAllocator {
 public:
  explicit DeviceCachingAllocator(RawBackend backend, AllocatorConfig config = AllocatorConfig());
  ~DeviceCachingAllocator() override;

  // Never returns nullptr for size > 0; throws std::bad_alloc-derived OutOfMemory after the
  // full retry ladder (reuse -> device malloc -> release enough cached -> release all cached).
  void* malloc(size_t size, StreamHandle stream) override;
  void* mallocFromCache(size_t size, StreamHandle stream) override;
  void free(void* ptr) override;
  // `ptr` is also being used on `stream`; its reuse waits for an event on that stream.
  void recordStream(void* ptr, StreamHandle stream) override;
  void emptyCache() override;
  void processEvents() override;

  static size_t roundSize(size_t size, const AllocatorConfig& cfg);
  static size_t allocationSize(size_t size, const AllocatorConfig& cfg);

  DeviceStats stats() const override;
  void resetPeakStats() override;
  std::vector<SegmentInfo> snapshot() const;
  size_t blockSize(void* ptr) const;  // rounded size of a live allocation (0 if unknown)
  // History of the allocator's steps (DIPUCachingDeviceAllocator.cpp:555-566, 1017-1027): a ring of the last maxEntries
  // entries, cleared whenever it is switched; trace() returns them oldest first.
  void recordHistory(bool enabled, size_t maxEntries) override;
  bool isHistoryEnabled() const override { return recordHistory_; }
  std::vector<TraceEntry> trace() const override;

 private:
  bool cacheOnly_ = false;  // set for the duration of mallocFromCache (under mutex_)
  bool recordHistory_ = false;
  size_t traceMax_ = 1;
  mutable size_t traceNext_ = 0;           // the ring is also written by const members (snapshot records itself)
  mutable std::vector<TraceEntry> trace_;
  void recordTrace(int action, int64_t addr, size_t size, StreamHandle stream) const;
  Block* getFreeBlock(BlockPool& pool, size_t size, StreamHandle stream);
  bool allocBlock(BlockPool& pool, size_t size, size_t allocSize, StreamHandle stream, Block** out);
  Block* findExpandableBlock(BlockPool& pool, size_t size, StreamHandle stream);
  bool mapBlock(Block* toMap, size_t size);
  Block* tryAllocateExpandableBlock(BlockPool& pool, size_t size, StreamHandle stream);
  void unmapBlock(Block* block);
  void releaseExpandable(Block* block);
  bool releaseAvailableCachedBlocks(BlockPool& pool, size_t size, StreamHandle stream);
  bool releaseCachedBlocks();
  void releaseBlocks(BlockPool& pool);
  void releaseBlock(Block* block);
  void garbageCollect();
  bool shouldSplit(const Block* block, size_t size) const;
  void freeBlock(Block* block);
  size_t tryMerge(Block* dst, Block* src, BlockPool& pool);
  void insertEvents(Block* block);
  void synchronizeAndFreeEvents();

  mutable std::recursive_mutex mutex_;
  RawBackend backend_;
  AllocatorConfig config_;
  DeviceStats stats_;
  BlockPool large_{false};
  BlockPool small_{true};
  std::unordered_map<void*, Block*> active_;
  std::unordered_map<StreamHandle, std::vector<std::pair<EventHandle, Block*>>> events_;
  std::vector<EventHandle> eventPool_;
  std::vector<ExpandableRange*> expandables_;
  size_t totalReserved_ = 0;
};

struct OutOfMemory : std::bad_alloc {
  std::string msg;
  explicit OutOfMemory(std::string m) : msg(std::move(m)) {}
  const char* what() const noexcept override { return msg.c_str(); }
};

// BF algorithm (dipu/torch_dipu/csrc_dipu/runtime/core/allocator/DIPUBFCachingAllocator.cpp:21-405): free chunks
// sit in 32 x 4 size classes (powers of two of 512-byte units, each split four ways) with one occupancy bit per
// class; a request takes the first chunk of its own class if that is large enough, else the first chunk of the
// next occupied class; a chunk at least twice the request, or 8 MiB larger, is split; freed chunks merge with
// free neighbours; when nothing fits the cache is emptied and the device is asked for max(request, extend size),
// the extend size doubling from 8 MiB up to DIPU_MAX_EXTEND_SIZE MiB (1024). All streams share one set of
// chunks, as in the reference (:357 uses stream set 0): a freed chunk becomes reusable once events recorded at
// free() on its allocation stream and on every stream given to recordStream() have completed (:525-548).
class BFCachingAllocator : public DeviceAllocator {
 public:
  explicit BFCachingAllocator(RawBackend backend, size_t maxExtendBytes = 0);  // 0: read DIPU_MAX_EXTEND_SIZE
  ~BFCachingAllocator() override;
  void* malloc(size_t size, StreamHandle stream) override;
  void free(void* ptr) override;
  void recordStream(void* ptr, StreamHandle stream) override;
  void emptyCache() override;
  void processEvents() override;
  DeviceStats stats() const override;
  void resetPeakStats() override;

  static constexpr int kBigBins = 32, kSubBins = 4, kBins = kBigBins * kSubBins;
  static constexpr size_t kMaxInternalFragmentation = size_t(8) << 20, kMinExtend = size_t(8) << 20;
  static int binOf(size_t nbytes);  // size class of a 512-byte-rounded size

 private:
  struct Chunk {
    char* ptr = nullptr;
    size_t size = 0, requested = 0;
    bool allocated = false;
    Chunk* before = nullptr;  // neighbours inside the device allocation this chunk was cut from
    Chunk* after = nullptr;
    Chunk* binPrev = nullptr;  // neighbours in the free list of its size class
    Chunk* binNext = nullptr;
    int bin = -1;
    StreamHandle stream = nullptr;
    std::vector<StreamHandle> extraStreams;
    bool whole() const { return before == nullptr && after == nullptr; }
  };
  struct Pending {
    Chunk* chunk;
    std::vector<EventHandle> events;
  };
  Chunk* take(size_t nbytes);
  Chunk* extend(size_t nbytes);
  void pushFree(Chunk* c);
  void popFree(Chunk* c);
  void giveBack(Chunk* c);
  void releaseWholeChunks();
  bool drainPending(bool wait);
  EventHandle newEvent();

  mutable std::mutex mutex_;
  RawBackend backend_;
  size_t maxExtend_, extendSize_ = kMinExtend;
  Chunk* heads_[kBins] = {};
  unsigned __int128 occupied_ = 0;
  std::unordered_map<void*, Chunk*> live_;
  std::vector<Pending> pending_;
  std::vector<EventHandle> eventPool_;
  DeviceStats stats_;
};

// BS algorithm (dipu/torch_dipu/csrc_dipu/runtime/core/allocator/DIPUBSCachingAllocator.cpp:18-242): one device
// allocation per distinct size, kept in a free list of exactly that size. Sizes round up to a multiple of
// DIPU_BS_ALLOCATOR_MIN_ALLOCATE_SIZE (512), or with DIPU_BS_MORE_ADAPTABLE set to the next power of two (:36-70).
// Nothing is split or merged; when the device refuses, every idle block is returned to it and the request is tried
// once more (:84-113). Reuse of a freed block waits for events on its streams (:205-222).
class BSCachingAllocator : public DeviceAllocator {
 public:
  // minAllocate = 0 / powerOfTwo < 0: read the two environment variables
  explicit BSCachingAllocator(RawBackend backend, size_t minAllocate = 0, int powerOfTwo = -1);
  ~BSCachingAllocator() override;
  void* malloc(size_t size, StreamHandle stream) override;
  void free(void* ptr) override;
  void recordStream(void* ptr, StreamHandle stream) override;
  void emptyCache() override;
  void processEvents() override;
  DeviceStats stats() const override;
  void resetPeakStats() override;
  size_t allocateSize(size_t nbytes) const;

 private:
  struct Live {
    size_t size = 0;
    StreamHandle stream = nullptr;
    std::vector<StreamHandle> extraStreams;
  };
  struct Pending {
    void* ptr;
    size_t size;
    std::vector<EventHandle> events;
  };
  bool drainPending(bool wait);
  void releaseIdle();
  EventHandle newEvent();

  mutable std::mutex mutex_;
  RawBackend backend_;
  size_t minAllocate_;
  bool powerOfTwo_;
  std::unordered_map<size_t, std::vector<void*>> idle_;
  std::unordered_map<void*, Live> live_;
  std::vector<Pending> pending_;
  std::vector<EventHandle> eventPool_;
  DeviceStats stats_;
};

// RAW algorithm: one device allocation per request, freed when its stream work is known
// to be finished (synchronous free after a device sync is the conservative choice made here).
class RawAllocator {
 public:
  explicit RawAllocator(RawBackend backend) : backend_(std::move(backend)) {}
  void* malloc(size_t size);
  void free(void* ptr);
  DeviceStats stats() const;

 private:
  mutable std::mutex mutex_;
  RawBackend backend_;
  std::unordered_map<void*, size_t> live_;
  DeviceStats stats_;
};

}  // namespace amdrt
}  // namespace dipu
