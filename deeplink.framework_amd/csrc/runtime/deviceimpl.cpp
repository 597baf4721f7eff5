// dipu::devapis over HIP for MI355X. This is the file a DIPU tree would hold as
// vendor/amd/deviceimpl.cpp; behaviour notes cite the contract each function
// has to honour (dipu/torch_dipu/csrc_dipu/runtime/device/deviceapis.h:23-124) and the
// behaviours DIPU's callers rely on.
#include <cstdlib>

// A DIPU tree declares the contract itself (csrc_dipu/runtime/device/deviceapis.h) before it compiles these bodies
// as vendor/amd/deviceimpl.cpp; on its own the runtime library uses the restated declarations.
#ifndef DIPU_AMD_DEVAPIS_DECLARED
#include "devapis_contract.h"
#endif

namespace dipu {
namespace devapis {

void initializeVendor() {}
void finalizeVendor() {}

deviceId_t current_device() {
  int dev = 0;
  DIPU_CALLHIP(hipGetDevice(&dev))
  return static_cast<deviceId_t>(dev);
}

// Must work for any index without a prior setDevice
// (dipu/tests/python/individual_scripts/test_get_device_properties.py:5-13).
DIPUDeviceProperties getDeviceProperties(int32_t device_index) {
  hipDeviceProp_t p;
  DIPU_CALLHIP(hipGetDeviceProperties(&p, device_index))
  DIPUDeviceProperties out;
  out.name = p.name;
  out.totalGlobalMem = p.totalGlobalMem;
  out.major = p.major;
  out.minor = p.minor;
  out.multiProcessorCount = p.multiProcessorCount;
  return out;
}

DIPUDeviceStatus getDeviceStatus(int32_t device_index) {
  int prev = 0;
  DIPU_CALLHIP(hipGetDevice(&prev))
  if (prev != device_index) DIPU_CALLHIP(hipSetDevice(device_index))
  DIPUDeviceStatus st;
  hipError_t r = hipMemGetInfo(&st.freeGlobalMem, &st.totalGlobalMem);
  if (prev != device_index) (void)hipSetDevice(prev);
  DIPU_CALLHIP(r)
  return st;
}

void setDevice(deviceId_t devId) { DIPU_CALLHIP(hipSetDevice(static_cast<int>(devId))) }

void resetDevice(deviceId_t devId) {
  (void)devId;
  DIPU_CALLHIP(hipDeviceReset())
}

void syncDevice() { DIPU_CALLHIP(hipDeviceSynchronize()) }

void checkLastError() { DIPU_CALLHIP(hipGetLastError()) }

// Runs while the library is being loaded in DIPU (allocator static initialiser), so a
// box without a usable GPU has to yield 0 rather than throw.
int getDeviceCount() {
  int n = 0;
  hipError_t r = hipGetDeviceCount(&n);
  if (r != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  return n;
}

void getDriverVersion(int* version) { DIPU_CALLHIP(hipDriverGetVersion(version)) }
void getRuntimeVersion(int* version) { DIPU_CALLHIP(hipRuntimeGetVersion(version)) }

// Every stream is created at the default priority: mixed-priority queues are not
// used on this platform, so `prior` is accepted and ignored.
void createStream(deviceStream_t* stream, bool prior) {
  (void)prior;
  DIPU_CALLHIP(hipStreamCreate(stream))
}

void destroyStream(deviceStream_t stream) { DIPU_CALLHIP(hipStreamDestroy(stream)) }

void destroyStream(deviceStream_t stream, deviceId_t devId) {
  setDevice(devId);
  destroyStream(stream);
}

void releaseStream() {}

void syncStream(deviceStream_t stream) { DIPU_CALLHIP(hipStreamSynchronize(stream)) }

bool streamNotNull(deviceStream_t stream) { return stream != nullptr && stream != hipStreamPerThread; }

void streamWaitEvent(deviceStream_t stream, deviceEvent_t event) { DIPU_CALLHIP(hipStreamWaitEvent(stream, event, 0)) }

bool isStreamEmpty(deviceStream_t stream) {
  hipError_t r = hipStreamQuery(stream);
  if (r == hipErrorNotReady) (void)hipGetLastError();
  return r == hipSuccess;
}

void createEvent(deviceEvent_t* event) {
  static const bool timing = [] {
    const char* env = std::getenv("DIPU_HIP_EVENT_TIMING");
    return env ? std::atoi(env) > 0 : true;
  }();
  DIPU_CALLHIP(hipEventCreateWithFlags(event, timing ? hipEventDefault : hipEventDisableTiming))
}

void destroyEvent(deviceEvent_t event) { DIPU_CALLHIP(hipEventDestroy(event)) }
void waitEvent(deviceEvent_t event) { DIPU_CALLHIP(hipEventSynchronize(event)) }
void recordEvent(deviceEvent_t event, deviceStream_t stream) { DIPU_CALLHIP(hipEventRecord(event, stream)) }
void eventElapsedTime(float* time, deviceEvent_t start, deviceEvent_t end) {
  DIPU_CALLHIP(hipEventElapsedTime(time, start, end))
}

// Not-ready maps to PENDING and the sticky error is cleared, as the allocator's async
// pools poll this in a loop (dipu/torch_dipu/csrc_dipu/vendor/cuda/deviceimpl.cpp:148-159).
EventStatus getEventStatus(deviceEvent_t event) {
  hipError_t r = hipEventQuery(event);
  if (r == hipSuccess) return EventStatus::READY;
  if (r == hipErrorNotReady) {
    (void)hipGetLastError();
    return EventStatus::PENDING;
  }
  DIPU_CALLHIP(r)
  return EventStatus::PENDING;
}

void mallocHost(void** p, size_t nbytes) { DIPU_CALLHIP(hipHostMalloc(p, nbytes, hipHostMallocDefault)) }
void freeHost(void* p) { DIPU_CALLHIP(hipHostFree(p)) }

OpStatus mallocDevice(void** p, size_t nbytes, bool throwExcepion) {
  hipError_t r = hipMalloc(p, nbytes);
  if (r == hipSuccess) return OpStatus::SUCCESS;
  if (r == hipErrorOutOfMemory && !throwExcepion) {
    (void)hipGetLastError();
    *p = nullptr;
    return OpStatus::ERR_NOMEM;
  }
  (void)hipGetLastError();
  throw std::runtime_error("hipMalloc failed, ret = " + std::to_string(static_cast<int>(r)) +
                           " size = " + std::to_string(nbytes));
}

void freeDevice(void* p) { DIPU_CALLHIP(hipFree(p)) }

// Exact for arbitrary host pointers: pageable memory is unknown to HIP and reports
// hipErrorInvalidValue, which is an answer ("not pinned"), not a failure
// (dipu/tests/python/unittests/test_pin_memory.py:9-32).
bool isPinnedPtr(const void* p) {
  hipPointerAttribute_t attr;
  hipError_t r = hipPointerGetAttributes(&attr, p);
  if (r != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return attr.type == hipMemoryTypeHost;
}

void memSetAsync(deviceStream_t stream, void* ptr, int val, size_t size) {
  DIPU_CALLHIP(hipMemsetAsync(ptr, val, size, stream))
}

void memCopyD2D(size_t nbytes, deviceId_t dstDevId, void* dst, deviceId_t srcDevId, const void* src) {
  if (dstDevId == srcDevId) {
    DIPU_CALLHIP(hipMemcpy(dst, src, nbytes, hipMemcpyDeviceToDevice))
  } else {
    DIPU_CALLHIP(hipMemcpyPeer(dst, dstDevId, src, srcDevId, nbytes))
  }
}
void memCopyH2D(size_t nbytes, void* dst, const void* src) {
  DIPU_CALLHIP(hipMemcpy(dst, src, nbytes, hipMemcpyHostToDevice))
}
void memCopyD2H(size_t nbytes, void* dst, const void* src) {
  DIPU_CALLHIP(hipMemcpy(dst, src, nbytes, hipMemcpyDeviceToHost))
}
void memCopyD2DAsync(deviceStream_t stream, size_t nbytes, deviceId_t dstDevId, void* dst, deviceId_t srcDevId,
                     const void* src) {
  if (dstDevId == srcDevId) {
    DIPU_CALLHIP(hipMemcpyAsync(dst, src, nbytes, hipMemcpyDeviceToDevice, stream))
  } else {
    DIPU_CALLHIP(hipMemcpyPeerAsync(dst, dstDevId, src, srcDevId, nbytes, stream))
  }
}
void memCopyH2DAsync(deviceStream_t stream, size_t nbytes, void* dst, const void* src) {
  DIPU_CALLHIP(hipMemcpyAsync(dst, src, nbytes, hipMemcpyHostToDevice, stream))
}
void memCopyD2HAsync(deviceStream_t stream, size_t nbytes, void* dst, const void* src) {
  DIPU_CALLHIP(hipMemcpyAsync(dst, src, nbytes, hipMemcpyDeviceToHost, stream))
}

}  // namespace devapis
}  // namespace dipu
