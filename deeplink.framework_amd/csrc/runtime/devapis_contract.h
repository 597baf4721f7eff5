// The device-API contract a DIPU vendor directory implements, restated without the
// c10 dependency so this runtime builds and is testable on its own.
//
// In a DIPU tree these declarations come from
//   dipu/torch_dipu/csrc_dipu/runtime/device/deviceapis.h:23-124   (functions)
//   dipu/torch_dipu/csrc_dipu/runtime/device/basedef.h:35-83        (enums, property structs)
// and the vendor supplies only vendorapi.h + deviceimpl.cpp. Names, argument order and
// return conventions here are those of that contract; deviceimpl.cpp is the part a DIPU
// build would compile unchanged as vendor/amd/deviceimpl.cpp.
#pragma once

#include <cstddef>
#include <cstdint>
#include <string>

#include "vendorapi.h"

namespace dipu {
namespace devapis {

using enum_t = int32_t;
using deviceId_t = int8_t;  // c10::DeviceIndex

enum class VendorDeviceType : enum_t { CUDA, MLU, NPU, MUXI, GCU, DROPLET, SUPA, KLX, AMD };
enum class EventStatus : enum_t { PENDING, RUNNING, DEFERRED, READY };
enum class OpStatus : enum_t { SUCCESS, ERR_UNKNOWN, ERR_NOMEM };

struct DIPUDeviceStatus {
  size_t freeGlobalMem = 0;
  size_t totalGlobalMem = 0;
};

struct DIPUDeviceProperties {
  std::string name;
  size_t totalGlobalMem = 0;
  int32_t major = 0;
  int32_t minor = 0;
  int32_t multiProcessorCount = 0;
};

// --- device ---
void initializeVendor();
void finalizeVendor();
deviceId_t current_device();
DIPUDeviceProperties getDeviceProperties(int32_t device_index);
DIPUDeviceStatus getDeviceStatus(int32_t device_index);
void setDevice(deviceId_t devId);
void resetDevice(deviceId_t devId = 0);
void syncDevice();
void checkLastError();
int getDeviceCount();
void getDriverVersion(int* version);
void getRuntimeVersion(int* version);

// --- stream ---
void createStream(deviceStream_t* stream, bool prior = false);
void destroyStream(deviceStream_t stream);
void destroyStream(deviceStream_t stream, deviceId_t devId);
void releaseStream();
void syncStream(deviceStream_t stream);
bool streamNotNull(deviceStream_t stream);
void streamWaitEvent(deviceStream_t stream, deviceEvent_t event);
bool isStreamEmpty(deviceStream_t stream);

// --- event ---
void createEvent(deviceEvent_t* event);
void destroyEvent(deviceEvent_t event);
void waitEvent(deviceEvent_t event);
void recordEvent(deviceEvent_t event, deviceStream_t stream);
void eventElapsedTime(float* time, deviceEvent_t start, deviceEvent_t end);
EventStatus getEventStatus(deviceEvent_t event);

// --- memory ---
void mallocHost(void** p, size_t nbytes);
void freeHost(void* p);
OpStatus mallocDevice(void** p, size_t nbytes, bool throwExcepion = true);
void freeDevice(void* p);
bool isPinnedPtr(const void* p);
void memSetAsync(deviceStream_t stream, void* ptr, int val, size_t size);
void memCopyD2D(size_t nbytes, deviceId_t dstDevId, void* dst, deviceId_t srcDevId, const void* src);
void memCopyH2D(size_t nbytes, void* dst, const void* src);
void memCopyD2H(size_t nbytes, void* dst, const void* src);
void memCopyD2DAsync(deviceStream_t stream, size_t nbytes, deviceId_t dstDevId, void* dst, deviceId_t srcDevId,
                     const void* src);
void memCopyH2DAsync(deviceStream_t stream, size_t nbytes, void* dst, const void* src);
void memCopyD2HAsync(deviceStream_t stream, size_t nbytes, void* dst, const void* src);


// ---- profiler hooks (runtime/device/profilerapis.h:12-14) ----
void enableProfiler(const std::string& dump_path, bool call_stack, bool record_shapes, bool profile_memory);
void disableProfiler();

}  // namespace devapis

namespace profile {
bool enabled();
void* rangeStart(const char* name);  // nullptr while the profiler is disabled
void rangeStop(void* record);
void counts(uint64_t* started, uint64_t* stopped, int* roctxBound);
}  // namespace profile
}  // namespace dipu
