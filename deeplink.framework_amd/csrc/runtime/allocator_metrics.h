// Allocator metrics with the label sets of dipu/torch_dipu/csrc_dipu/runtime/core/allocator/allocator_metrics.h:17-160:
//   allocator_event_count{type, device, method = allocate | deallocate, event = nullptr | duplicated | unexpected}
//   allocator_size{type, device, method}      histogram, upper bounds 2^4 .. 2^31 bytes, plus the sum of the sizes
// type is "caching" for the caching device allocators, "device" and "host" for the raw vendor calls underneath
// (runtime/devproxy/deviceproxy.cpp:196-218). Recording is on by default and can be switched off
// (metrics/metrics.cpp:5-11); while off nothing is counted and the live-pointer table is not maintained.
#pragma once

#include <array>
#include <atomic>
#include <cstddef>
#include <cstdint>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <tuple>
#include <unordered_map>

namespace dipu {
namespace amdrt {

// Returns the current setting; update = 0 / 1 changes it first, any other value only reads.
bool metricsEnable(int update = -1);

class AllocatorMetrics {
 public:
  static constexpr int kFirstBit = 4, kBuckets = 32 - kFirstBit;  // bounds 2^4 .. 2^31, then +Inf
  AllocatorMetrics(std::string type, int device) : type_(std::move(type)), device_(device) {}
  // A block handed out: size 0 is ignored, a null pointer and a pointer already live are events.
  void allocate(void* data, size_t size);
  // A block taken back: a null pointer and a pointer that is not live are events.
  void deallocate(void* data);
  void appendText(std::string* out) const;

 private:
  struct Histogram {
    std::array<uint64_t, kBuckets + 1> buckets{};  // the last one is +Inf
    uint64_t sum = 0;
    void put(size_t v);
  };
  const std::string type_;
  const int device_;
  mutable std::mutex mutex_;
  std::unordered_map<void*, size_t> live_;
  uint64_t allocNull_ = 0, allocDuplicated_ = 0, freeNull_ = 0, freeUnexpected_ = 0;
  Histogram allocSize_, freeSize_;
};

// One AllocatorMetrics per (type, device), created on first use and kept until the process ends.
AllocatorMetrics& allocatorMetrics(const std::string& type, int device);
// Every value in the text exposition format, one line each, sorted by (type, device).
std::string metricsText();

}  // namespace amdrt
}  // namespace dipu
