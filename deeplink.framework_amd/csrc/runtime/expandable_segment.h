// A range of device virtual addresses that grows and shrinks in whole segments: the vendor half of DIPU's
// expandable segments (contract dipu/torch_dipu/csrc_dipu/runtime/core/allocator/ExpandableSegment.h:114-136;
// the CUDA vendor's form is vendor/cuda/CUDAExpandableSegment.cpp:15-176), on HIP's virtual memory management:
// one hipMemAddressReserve for 9/8 of the device's memory, one physical allocation (hipMemCreate) per mapped
// segment, hipMemMap + hipMemSetAccess to make it addressable, hipMemUnmap + hipMemRelease to give it back.
#pragma once

#include <cstddef>
#include <vector>

#include "vendorapi.h"

namespace dipu {
namespace amdrt {

struct SegmentRange {
  char* ptr = nullptr;
  size_t size = 0;
};

class HipExpandableSegment {
 public:
  // segmentSize must be a multiple of the device's allocation granularity (2 MiB and 20 MiB, the two sizes the
  // caching allocator uses, are)
  HipExpandableSegment(int device, deviceStream_t stream, size_t segmentSize, std::vector<int> peers = {});
  ~HipExpandableSegment();
  HipExpandableSegment(const HipExpandableSegment&) = delete;
  HipExpandableSegment& operator=(const HipExpandableSegment&) = delete;

  // Backs every segment touched by [range.ptr, range.ptr + range.size) with memory; range.ptr must be the start of
  // a segment none of which is mapped yet. Returns what is now mapped (whole segments), or an empty range at
  // range.ptr if the device is out of memory (nothing stays mapped then).
  SegmentRange map(SegmentRange range);
  // Gives back the segments that lie entirely inside the range, after the stream's work is done. Returns them.
  SegmentRange unmap(SegmentRange range);
  void addPeer(int device);
  char* ptr() const { return base_; }
  size_t size() const { return maxSegments_ * segmentSize_; }
  size_t segmentSize() const { return segmentSize_; }
  size_t mappedBytes() const;

 private:
  void setAccess(int device, size_t begin, size_t end);
  void release(size_t begin, size_t end);
  void trim();
  SegmentRange rangeOf(size_t begin, size_t end) const { return {base_ + begin * segmentSize_, (end - begin) * segmentSize_}; }

  int device_;
  deviceStream_t stream_;
  size_t segmentSize_, maxSegments_ = 0;
  char* base_ = nullptr;
  struct Slot {
    hipMemGenericAllocationHandle_t handle;
    bool mapped = false;
  };
  std::vector<Slot> slots_;
  std::vector<int> peers_;
};

}  // namespace amdrt
}  // namespace dipu
