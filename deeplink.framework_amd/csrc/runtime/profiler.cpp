// Profiler hooks of the vendor layer: devapis::enableProfiler / disableProfiler
// (dipu/torch_dipu/csrc_dipu/runtime/device/profilerapis.h:12-14, weak in DIPU, so a vendor may
// supply them) and the range pair behind diopiRecordStart / diopiRecordEnd
// (dipu/torch_dipu/csrc_dipu/diopirt/diopirt_impl.cpp:224-237).
//
// On this vendor a profile is taken from outside the process with rocprofv3, which already sees
// every kernel; what the process can add are named host ranges. They are emitted as ROCTX ranges
// (rocprofv3 --marker-trace shows them on the timeline next to the kernels). The ROCTX library is
// looked up at enable time with dlopen, so nothing links against it and a machine without it
// simply records range counts. While the profiler is disabled a range costs one relaxed load.
#include <dlfcn.h>

#include <atomic>
#include <mutex>
#include <string>

#include "devapis_contract.h"
#include "runtime_core.h"

namespace dipu {
namespace profile {

namespace {
using RangeStartFn = uint64_t (*)(const char*);
using RangeStopFn = void (*)(uint64_t);

std::atomic<bool> g_enabled{false};
std::atomic<uint64_t> g_started{0}, g_stopped{0};
std::mutex g_mutex;
void* g_lib = nullptr;
RangeStartFn g_start = nullptr;
RangeStopFn g_stop = nullptr;
std::string g_dumpPath;

void bindRoctx() {
  if (g_lib) return;
  const char* names[] = {"librocprofiler-sdk-roctx.so.1", "librocprofiler-sdk-roctx.so", "libroctx64.so.4",
                         "libroctx64.so"};
  for (const char* n : names) {
    void* lib = dlopen(n, RTLD_NOW | RTLD_LOCAL);
    if (!lib) continue;
    auto s = reinterpret_cast<RangeStartFn>(dlsym(lib, "roctxRangeStartA"));
    auto e = reinterpret_cast<RangeStopFn>(dlsym(lib, "roctxRangeStop"));
    if (s && e) {
      g_lib = lib, g_start = s, g_stop = e;
      return;
    }
    dlclose(lib);
  }
}
}  // namespace

bool enabled() { return g_enabled.load(std::memory_order_relaxed); }

// Returns a heap cell holding the ROCTX id (or 0 when no ROCTX library is bound), or nullptr
// when the profiler is off.
void* rangeStart(const char* name) {
  if (!enabled()) return nullptr;
  g_started.fetch_add(1, std::memory_order_relaxed);
  uint64_t id = g_start ? g_start(name ? name : "") : 0;
  return new uint64_t(id);
}

void rangeStop(void* record) {
  if (!record) return;
  auto* cell = static_cast<uint64_t*>(record);
  if (g_stop && g_start) g_stop(*cell);
  delete cell;
  g_stopped.fetch_add(1, std::memory_order_relaxed);
}

void counts(uint64_t* started, uint64_t* stopped, int* roctxBound) {
  if (started) *started = g_started.load();
  if (stopped) *stopped = g_stopped.load();
  if (roctxBound) *roctxBound = g_start != nullptr;
}

}  // namespace profile

namespace devapis {

// call_stack / record_shapes / profile_memory select kineto features DIPU's own profiler layer
// implements above the vendor; a vendor hook only has to switch its device-side collection.
void enableProfiler(const std::string& dump_path, bool /*call_stack*/, bool /*record_shapes*/,
                    bool /*profile_memory*/) {
  std::lock_guard<std::mutex> lock(profile::g_mutex);
  profile::g_dumpPath = dump_path;
  profile::bindRoctx();
  profile::g_enabled.store(true);
}

void disableProfiler() {
  std::lock_guard<std::mutex> lock(profile::g_mutex);
  profile::g_enabled.store(false);
}

}  // namespace devapis
}  // namespace dipu
