#include "expandable_segment.h"

#include <stdexcept>
#include <string>

namespace dipu {
namespace amdrt {

HipExpandableSegment::HipExpandableSegment(int device, deviceStream_t stream, size_t segmentSize, std::vector<int> peers)
    : device_(device), stream_(stream), segmentSize_(segmentSize), peers_(std::move(peers)) {
  hipMemAllocationProp prop = {};
  prop.type = hipMemAllocationTypePinned;
  prop.location.type = hipMemLocationTypeDevice;
  prop.location.id = device_;
  size_t granularity = 0;
  DIPU_CALLHIP(hipMemGetAllocationGranularity(&granularity, &prop, hipMemAllocationGranularityMinimum));
  if (segmentSize_ == 0 || (granularity && segmentSize_ % granularity != 0))
    throw std::invalid_argument("expandable segment: segment size " + std::to_string(segmentSize_) +
                                " is not a multiple of the allocation granularity " + std::to_string(granularity));
  hipDeviceProp_t dp;
  DIPU_CALLHIP(hipGetDeviceProperties(&dp, device_));
  // room for all of the device's memory and an eighth more, as the reference reserves
  const size_t span = dp.totalGlobalMem + dp.totalGlobalMem / 8;
  maxSegments_ = (span + segmentSize_ - 1) / segmentSize_;
  void* p = nullptr;
  DIPU_CALLHIP(hipMemAddressReserve(&p, maxSegments_ * segmentSize_, 0, nullptr, 0));
  base_ = static_cast<char*>(p);
}

HipExpandableSegment::~HipExpandableSegment() {
  try {
    size_t i = 0;
    while (i < slots_.size()) {
      if (!slots_[i].mapped) {
        ++i;
        continue;
      }
      size_t j = i;
      while (j < slots_.size() && slots_[j].mapped) ++j;
      release(i, j);
      i = j;
    }
    if (base_) (void)hipMemAddressFree(base_, maxSegments_ * segmentSize_);
  } catch (...) {
  }
}

void HipExpandableSegment::setAccess(int device, size_t begin, size_t end) {
  hipMemAccessDesc desc = {};
  desc.location.type = hipMemLocationTypeDevice;
  desc.location.id = device;
  desc.flags = hipMemAccessFlagsProtReadWrite;
  DIPU_CALLHIP(hipMemSetAccess(base_ + begin * segmentSize_, (end - begin) * segmentSize_, &desc, 1));
}

void HipExpandableSegment::trim() {
  while (!slots_.empty() && !slots_.back().mapped) slots_.pop_back();
}

void HipExpandableSegment::release(size_t begin, size_t end) {
  // the mapping goes away for good: everything queued on the stream that may touch it has to be done first
  DIPU_CALLHIP(hipStreamSynchronize(stream_));
  for (size_t i = begin; i < end; ++i) {
    DIPU_CALLHIP(hipMemUnmap(base_ + i * segmentSize_, segmentSize_));
    DIPU_CALLHIP(hipMemRelease(slots_[i].handle));
    slots_[i].mapped = false;
  }
  trim();
}

SegmentRange HipExpandableSegment::map(SegmentRange range) {
  const size_t off = static_cast<size_t>(range.ptr - base_);
  if (range.ptr < base_ || off % segmentSize_ != 0) throw std::invalid_argument("expandable segment: map() must start at a segment boundary");
  const size_t begin = off / segmentSize_;
  const size_t end = (off + range.size + segmentSize_ - 1) / segmentSize_;
  if (end > maxSegments_) throw std::invalid_argument("expandable segment: map() past the reserved range");
  if (begin == end) return rangeOf(begin, end);
  if (slots_.size() < end) slots_.resize(end);
  for (size_t i = begin; i < end; ++i)
    if (slots_[i].mapped) throw std::invalid_argument("expandable segment: map() over a segment that is already mapped");
  hipMemAllocationProp prop = {};
  prop.type = hipMemAllocationTypePinned;
  prop.location.type = hipMemLocationTypeDevice;
  prop.location.id = device_;
  size_t made = begin;
  for (; made < end; ++made) {
    const hipError_t st = hipMemCreate(&slots_[made].handle, segmentSize_, &prop, 0);
    if (st == hipErrorOutOfMemory) {
      (void)hipGetLastError();
      for (size_t j = begin; j < made; ++j) DIPU_CALLHIP(hipMemRelease(slots_[j].handle));
      trim();
      return rangeOf(begin, begin);
    }
    DIPU_CALLHIP(st);
  }
  for (size_t i = begin; i < end; ++i) {
    DIPU_CALLHIP(hipMemMap(base_ + i * segmentSize_, segmentSize_, 0, slots_[i].handle, 0));
    slots_[i].mapped = true;
  }
  setAccess(device_, begin, end);
  for (int p : peers_) setAccess(p, begin, end);
  return rangeOf(begin, end);
}

SegmentRange HipExpandableSegment::unmap(SegmentRange range) {
  const size_t lo = static_cast<size_t>(range.ptr - base_), hi = lo + range.size;
  const size_t begin = (lo + segmentSize_ - 1) / segmentSize_;  // first segment that starts inside the range
  const size_t end = hi / segmentSize_;                          // one past the last segment that ends inside it
  if (begin >= end) return SegmentRange{range.ptr, 0};
  if (end > slots_.size()) throw std::invalid_argument("expandable segment: unmap() of segments that are not mapped");
  for (size_t i = begin; i < end; ++i)
    if (!slots_[i].mapped) throw std::invalid_argument("expandable segment: unmap() of a segment that is not mapped");
  release(begin, end);
  return rangeOf(begin, end);
}

void HipExpandableSegment::addPeer(int device) {
  peers_.push_back(device);
  size_t i = 0;
  while (i < slots_.size()) {
    if (!slots_[i].mapped) {
      ++i;
      continue;
    }
    size_t j = i;
    while (j < slots_.size() && slots_[j].mapped) ++j;
    setAccess(device, i, j);
    i = j;
  }
}

size_t HipExpandableSegment::mappedBytes() const {
  size_t n = 0;
  for (const Slot& s : slots_) n += s.mapped ? segmentSize_ : 0;
  return n;
}

}  // namespace amdrt
}  // namespace dipu
