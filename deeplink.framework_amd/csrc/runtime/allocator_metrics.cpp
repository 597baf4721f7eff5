#include "allocator_metrics.h"

#include <cstdio>

namespace dipu {
namespace amdrt {

bool metricsEnable(int update) {
  static std::atomic<bool> value{true};
  if (update == 0 || update == 1) value.store(update == 1, std::memory_order_release);
  return value.load(std::memory_order_acquire);
}

void AllocatorMetrics::Histogram::put(size_t v) {
  int b = 0;
  while (b < kBuckets && v > (size_t{1} << (kFirstBit + b))) ++b;  // bucket b holds values <= 2^(4 + b)
  buckets[b] += 1;
  sum += v;
}

void AllocatorMetrics::allocate(void* data, size_t size) {
  if (size == 0 || !metricsEnable()) return;
  std::lock_guard<std::mutex> lock(mutex_);
  if (data == nullptr) {
    allocNull_ += 1;
  } else if (live_.emplace(data, size).second) {
    allocSize_.put(size);
  } else {
    allocDuplicated_ += 1;
  }
}

void AllocatorMetrics::deallocate(void* data) {
  if (!metricsEnable()) return;
  std::lock_guard<std::mutex> lock(mutex_);
  if (data == nullptr) {
    freeNull_ += 1;
    return;
  }
  auto it = live_.find(data);
  if (it == live_.end()) {
    freeUnexpected_ += 1;
    return;
  }
  freeSize_.put(it->second);
  live_.erase(it);
}

void AllocatorMetrics::appendText(std::string* out) const {
  std::lock_guard<std::mutex> lock(mutex_);
  char line[256];
  const std::string base = "device=\"" + std::to_string(device_) + "\",";
  auto counter = [&](const char* method, const char* event, uint64_t v) {
    std::snprintf(line, sizeof(line), "allocator_event_count{%sevent=\"%s\",method=\"%s\",type=\"%s\"} %llu\n", base.c_str(), event,
                  method, type_.c_str(), (unsigned long long)v);
    *out += line;
  };
  counter("allocate", "nullptr", allocNull_);
  counter("allocate", "duplicated", allocDuplicated_);
  counter("deallocate", "nullptr", freeNull_);
  counter("deallocate", "unexpected", freeUnexpected_);
  auto histogram = [&](const char* method, const Histogram& h) {
    uint64_t cumulative = 0;
    for (int b = 0; b <= kBuckets; ++b) {
      cumulative += h.buckets[b];
      if (b < kBuckets)
        std::snprintf(line, sizeof(line), "allocator_size_bucket{%sle=\"%llu\",method=\"%s\",type=\"%s\"} %llu\n", base.c_str(),
                      1ull << (kFirstBit + b), method, type_.c_str(), (unsigned long long)cumulative);
      else
        std::snprintf(line, sizeof(line), "allocator_size_bucket{%sle=\"+Inf\",method=\"%s\",type=\"%s\"} %llu\n", base.c_str(), method,
                      type_.c_str(), (unsigned long long)cumulative);
      *out += line;
    }
    std::snprintf(line, sizeof(line), "allocator_size_sum{%smethod=\"%s\",type=\"%s\"} %llu\n", base.c_str(), method, type_.c_str(),
                  (unsigned long long)h.sum);
    *out += line;
    std::snprintf(line, sizeof(line), "allocator_size_count{%smethod=\"%s\",type=\"%s\"} %llu\n", base.c_str(), method, type_.c_str(),
                  (unsigned long long)cumulative);
    *out += line;
  };
  histogram("allocate", allocSize_);
  histogram("deallocate", freeSize_);
}

namespace {
std::mutex g_registryMutex;
// never destroyed: allocators may report while static destructors run
auto* g_registry = new std::map<std::pair<std::string, int>, std::unique_ptr<AllocatorMetrics>>();
}  // namespace

AllocatorMetrics& allocatorMetrics(const std::string& type, int device) {
  std::lock_guard<std::mutex> lock(g_registryMutex);
  auto& slot = (*g_registry)[{type, device}];
  if (!slot) slot = std::make_unique<AllocatorMetrics>(type, device);
  return *slot;
}

std::string metricsText() {
  std::string out;
  std::lock_guard<std::mutex> lock(g_registryMutex);
  for (auto& kv : *g_registry) kv.second->appendText(&out);
  return out;
}

}  // namespace amdrt
}  // namespace dipu
