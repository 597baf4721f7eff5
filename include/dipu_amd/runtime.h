/*
 * C facade of the MI355X host runtime (libdipu_amd_rt.so): device / stream / event /
 * memory functions, the caching allocator, and the diopirt tensor + context objects
 * that libdiopi_impl.so's callbacks resolve against when DIPU itself is not the host.
 *
 * Every function returns 0 on success and non-zero on failure; the text of the last
 * failure on the calling thread is dipuAmdGetLastError(). No exception crosses this ABI.
 * Each group cites the reference interface it stands in for (paths relative to the
 * reference tree, dipu/torch_dipu/csrc_dipu/...).
 */
#ifndef DIPU_AMD_RUNTIME_H_
#define DIPU_AMD_RUNTIME_H_

#include <stddef.h>
#include <stdint.h>

#if defined(__cplusplus)
extern "C" {
#endif

#define DIPU_AMD_API __attribute__((visibility("default")))

DIPU_AMD_API const char* dipuAmdGetLastError(void);

/* ---- device: runtime/device/deviceapis.h:23-46 ---- */
DIPU_AMD_API int dipuAmdInitializeVendor(void);
DIPU_AMD_API int dipuAmdFinalizeVendor(void);
DIPU_AMD_API int dipuAmdGetDeviceCount(int* count);
DIPU_AMD_API int dipuAmdCurrentDevice(int* device);
DIPU_AMD_API int dipuAmdSetDevice(int device);
DIPU_AMD_API int dipuAmdSyncDevice(void);
DIPU_AMD_API int dipuAmdCheckLastError(void);
DIPU_AMD_API int dipuAmdGetDriverVersion(int* version);
DIPU_AMD_API int dipuAmdGetRuntimeVersion(int* version);
typedef struct dipuAmdDeviceProperties {
  char name[256];
  uint64_t totalGlobalMem;
  int32_t major, minor, multiProcessorCount;
} dipuAmdDeviceProperties; /* runtime/device/basedef.h:74-80 */
DIPU_AMD_API int dipuAmdGetDeviceProperties(int device, dipuAmdDeviceProperties* props);
/* runtime/device/basedef.h:69-72 */
DIPU_AMD_API int dipuAmdGetDeviceStatus(int device, uint64_t* free_bytes, uint64_t* total_bytes);

/* ---- streams: deviceapis.h:48-62; pool of 1 default + 8 streams per device and a
 * per-thread current stream, runtime/core/DIPUStream.cpp:38-39,75-87,149-154 ---- */
DIPU_AMD_API int dipuAmdCreateStream(void** stream);
DIPU_AMD_API int dipuAmdDestroyStream(void* stream);
DIPU_AMD_API int dipuAmdSyncStream(void* stream);
DIPU_AMD_API int dipuAmdIsStreamEmpty(void* stream, int* empty);
DIPU_AMD_API int dipuAmdStreamWaitEvent(void* stream, void* event);
DIPU_AMD_API int dipuAmdGetDefaultStream(int device, void** stream);
DIPU_AMD_API int dipuAmdGetStreamFromPool(int device, void** stream);
DIPU_AMD_API int dipuAmdGetCurrentStream(int device, void** stream);
DIPU_AMD_API int dipuAmdSetCurrentStream(int device, void* stream);

/* ---- events: deviceapis.h:68-79; pooled per device, runtime/core/DIPUEventPool.cpp:11-101 ---- */
DIPU_AMD_API int dipuAmdCreateEvent(void** event);   /* taken from the pool */
DIPU_AMD_API int dipuAmdDestroyEvent(void* event);   /* returned to the pool */
DIPU_AMD_API int dipuAmdRecordEvent(void* event, void* stream);
DIPU_AMD_API int dipuAmdWaitEvent(void* event);
DIPU_AMD_API int dipuAmdEventElapsedTime(float* ms, void* start, void* end);
/* status: 0 PENDING, 1 RUNNING, 2 DEFERRED, 3 READY (runtime/device/basedef.h:46) */
DIPU_AMD_API int dipuAmdGetEventStatus(void* event, int* status);

/* ---- raw memory: deviceapis.h:84-124 ---- */
DIPU_AMD_API int dipuAmdMallocHost(void** p, size_t nbytes);
DIPU_AMD_API int dipuAmdFreeHost(void* p);
/* status: 0 SUCCESS, 2 ERR_NOMEM when throw_on_oom == 0 (runtime/device/basedef.h:48-52) */
DIPU_AMD_API int dipuAmdMallocDevice(void** p, size_t nbytes, int throw_on_oom, int* status);
DIPU_AMD_API int dipuAmdFreeDevice(void* p);
DIPU_AMD_API int dipuAmdIsPinnedPtr(const void* p, int* pinned);
DIPU_AMD_API int dipuAmdMemSetAsync(void* stream, void* ptr, int val, size_t size);
DIPU_AMD_API int dipuAmdMemCopyD2D(size_t nbytes, int dst_dev, void* dst, int src_dev, const void* src);
DIPU_AMD_API int dipuAmdMemCopyH2D(size_t nbytes, void* dst, const void* src);
DIPU_AMD_API int dipuAmdMemCopyD2H(size_t nbytes, void* dst, const void* src);
DIPU_AMD_API int dipuAmdMemCopyD2DAsync(void* stream, size_t nbytes, int dst_dev, void* dst, int src_dev,
                                        const void* src);
DIPU_AMD_API int dipuAmdMemCopyH2DAsync(void* stream, size_t nbytes, void* dst, const void* src);
DIPU_AMD_API int dipuAmdMemCopyD2HAsync(void* stream, size_t nbytes, void* dst, const void* src);

/* ---- caching allocator: runtime/core/allocator/DIPUCachingDeviceAllocator.cpp:500-2037,
 * selection by DIPU_DEVICE_MEMCACHING_ALGORITHM in {TORCH, RAW} (base/environ.hpp:88-92),
 * options from DIPU_TORCH_ALLOCATOR_CONF (DIPUCachingDeviceAllocator.cpp:454-496) ---- */
typedef struct dipuAmdMemoryStats {
  int64_t allocated_bytes, allocated_bytes_peak;
  int64_t reserved_bytes, reserved_bytes_peak;
  int64_t active_bytes, inactive_split_bytes, requested_bytes;
  int64_t allocations, segments;
  int64_t num_alloc_retries, num_ooms, num_device_malloc, num_device_free;
} dipuAmdMemoryStats;
DIPU_AMD_API int dipuAmdCachingMalloc(void** p, size_t nbytes, void* stream);
DIPU_AMD_API int dipuAmdCachingFree(void* p);
DIPU_AMD_API int dipuAmdCachingRecordStream(void* p, void* stream);
DIPU_AMD_API int dipuAmdCachingEmptyCache(void);
DIPU_AMD_API int dipuAmdCachingStats(int device, dipuAmdMemoryStats* stats);
DIPU_AMD_API int dipuAmdCachingResetPeakStats(int device);
/* History of the TORCH allocator's steps: recordHistory / trace of DIPUCachingDeviceAllocator.cpp:555-566, 1017-1027,
 * entries of DIPUCachingDeviceAllocator.h:134-164 without the Python stack context. A ring of the last max_entries
 * steps, cleared whenever it is switched. action: 0 ALLOC, 1 FREE_REQUESTED, 2 FREE_COMPLETED, 3 SEGMENT_ALLOC,
 * 4 SEGMENT_FREE, 5 SEGMENT_MAP, 6 SEGMENT_UNMAP, 7 SNAPSHOT (size = active bytes), 8 OOM (addr = bytes the request
 * would have taken from the device). Trace copies at most `capacity` entries, oldest first, and reports how many the
 * ring holds in *count. The RAW, BF and BS algorithms keep no history: the switch is ignored and *count is 0. */
typedef struct dipuAmdTraceEntry {
  int32_t action;
  int32_t reserved;
  int64_t addr;
  uint64_t size;
  void* stream;
} dipuAmdTraceEntry;
DIPU_AMD_API int dipuAmdCachingRecordHistory(int device, int enabled, uint64_t max_entries);
DIPU_AMD_API int dipuAmdCachingTrace(int device, dipuAmdTraceEntry* entries, uint64_t capacity, uint64_t* count);
/* pinned host cache: power-of-two sized, runtime/core/allocator/DIPUCachingHostAllocator.cpp:99-123,238 */
DIPU_AMD_API int dipuAmdCachingHostMalloc(void** p, size_t nbytes);
DIPU_AMD_API int dipuAmdCachingHostFree(void* p);
DIPU_AMD_API int dipuAmdCachingHostRecordStream(void* p, void* stream);
DIPU_AMD_API int dipuAmdCachingHostEmptyCache(void);

/* Expandable segment over HIP virtual memory management: the vendor half of DIPU's expandable segments
 * (runtime/core/allocator/ExpandableSegment.h:114-136; CUDA form vendor/cuda/CUDAExpandableSegment.cpp:15-176).
 * A reserved address range of 9/8 of the device's memory whose segments of segment_bytes are backed on map and given
 * back on unmap; offsets are relative to the range's base. map starts at a segment boundary and maps every segment
 * the range touches (mapped_bytes == 0: out of memory); unmap releases the segments entirely inside the range after
 * synchronising the stream. */
DIPU_AMD_API int dipuAmdExpandableSegmentCreate(void** handle, int device, void* stream, uint64_t segment_bytes);
DIPU_AMD_API int dipuAmdExpandableSegmentDestroy(void* handle);
DIPU_AMD_API int dipuAmdExpandableSegmentInfo(void* handle, void** base, uint64_t* reserved_bytes, uint64_t* mapped_bytes);
DIPU_AMD_API int dipuAmdExpandableSegmentMap(void* handle, uint64_t offset, uint64_t nbytes, uint64_t* mapped_offset,
                                             uint64_t* mapped_bytes);
DIPU_AMD_API int dipuAmdExpandableSegmentUnmap(void* handle, uint64_t offset, uint64_t nbytes, uint64_t* unmapped_offset,
                                               uint64_t* unmapped_bytes);

/* A generator object for the diopiGenerator* callbacks of diopirt.h: what vendorMakeGenerator returns in DIPU
 * (runtime/core/DIPUGeneratorImpl.h:62; state layout of vendor/cuda/CudaGeneratorImpl.cpp:17-76), without libtorch. */
struct diopiGenerator;
DIPU_AMD_API int dipuAmdGeneratorCreate(struct diopiGenerator** gen, int device_index);
DIPU_AMD_API int dipuAmdGeneratorDestroy(struct diopiGenerator* gen);

/* The same allocator state machine over a host-memory backend with a capacity limit and
 * manually completed events: lets the allocator be driven on a machine without a GPU. */
DIPU_AMD_API int dipuAmdSimAllocatorCreate(void** handle, uint64_t capacity_bytes, const char* conf);
/* The same stand-in driving the BF algorithm (DIPU_DEVICE_MEMCACHING_ALGORITHM=BF,
 * dipu/torch_dipu/csrc_dipu/runtime/core/allocator/DIPUBFCachingAllocator.cpp:21-405); max_extend_bytes = 0 reads
 * DIPU_MAX_EXTEND_SIZE (MiB, default 1024). The other dipuAmdSimAllocator* calls work on either kind. */
DIPU_AMD_API int dipuAmdSimAllocatorCreateBF(void** handle, uint64_t capacity_bytes, uint64_t max_extend_bytes);
/* ... and the BS algorithm (DIPUBSCachingAllocator.cpp:18-242): one free list per exact size; sizes are multiples of
 * min_allocate_bytes (0 = 512) or, with power_of_two != 0, the next power of two (DIPU_BS_MORE_ADAPTABLE). */
DIPU_AMD_API int dipuAmdSimAllocatorCreateBS(void** handle, uint64_t capacity_bytes, uint64_t min_allocate_bytes,
                                             int power_of_two);
DIPU_AMD_API int dipuAmdSimAllocatorDestroy(void* handle);
DIPU_AMD_API int dipuAmdSimAllocatorMalloc(void* handle, void** p, size_t nbytes, void* stream);
/* The request a workspace allocation makes while its stream is being captured: served from cached blocks only
 * (NULL when none fits), without querying any event. */
DIPU_AMD_API int dipuAmdSimAllocatorMallocFromCache(void* handle, void** p, size_t nbytes, void* stream);
/* How many times the allocator has asked the simulated device whether an event has completed. */
DIPU_AMD_API int dipuAmdSimAllocatorEventQueries(void* handle, uint64_t* queries);
DIPU_AMD_API int dipuAmdSimAllocatorFree(void* handle, void* p);
DIPU_AMD_API int dipuAmdSimAllocatorRecordStream(void* handle, void* p, void* stream);
DIPU_AMD_API int dipuAmdSimAllocatorEmptyCache(void* handle);
DIPU_AMD_API int dipuAmdSimAllocatorStats(void* handle, dipuAmdMemoryStats* stats);
DIPU_AMD_API int dipuAmdSimAllocatorRecordHistory(void* handle, int enabled, uint64_t max_entries);
DIPU_AMD_API int dipuAmdSimAllocatorTrace(void* handle, dipuAmdTraceEntry* entries, uint64_t capacity, uint64_t* count);
/* events recorded so far on `stream` (all streams when null) become ready */
DIPU_AMD_API int dipuAmdSimAllocatorCompleteEvents(void* handle, void* stream);
DIPU_AMD_API int dipuAmdSimAllocatorBackendUsage(void* handle, uint64_t* bytes_in_use, uint64_t* live_segments);
DIPU_AMD_API uint64_t dipuAmdRoundSize(uint64_t nbytes, const char* conf);
DIPU_AMD_API uint64_t dipuAmdSegmentSize(uint64_t rounded_nbytes, const char* conf);

/* ---- diopirt objects: diopirt/diopirt_impl.h:19-26 (context), diopirt_impl.cpp:24-173 ---- */
#define DIPU_AMD_MAX_DIMS 8
/* What a diopiTensorHandle_t points at when this runtime (not DIPU) hosts libdiopi_impl.so. */
typedef struct dipuAmdTensor {
  void* data;
  int64_t ndim;
  int64_t shape[DIPU_AMD_MAX_DIMS];
  int64_t stride[DIPU_AMD_MAX_DIMS];
  int32_t dtype;        /* diopiDtype_t */
  int32_t device;       /* diopiDevice_t */
  int32_t device_index;
  int32_t reserved;
  int64_t storage_offset;
  void* storage_ptr;
  uint64_t storage_nbytes;
} dipuAmdTensor;
/* A diopiContext bound to `stream`; workspace tensors it hands out are returned to the
 * caching allocator (stream-ordered reuse) when the context is destroyed. */
DIPU_AMD_API int dipuAmdContextCreate(void* stream, void** ctx);
DIPU_AMD_API int dipuAmdContextDestroy(void* ctx);
DIPU_AMD_API int dipuAmdContextReset(void* ctx);  /* release workspace, keep the context */
DIPU_AMD_API int dipuAmdContextWorkspace(void* ctx, uint64_t* tensors, uint64_t* bytes);

/* ---- profiler hooks: dipu/torch_dipu/csrc_dipu/runtime/device/profilerapis.h:12-14 (enableProfiler /
 * disableProfiler) and the diopiRecordStart / diopiRecordEnd pair, diopirt/diopirt_impl.cpp:224-237.
 * While enabled, every diopiRecordStart/End pair becomes a ROCTX range (when a ROCTX library can be loaded)
 * and is counted; dipuAmdProfilerCounts reports ranges started, ranges ended, and whether ROCTX is bound. */
DIPU_AMD_API int dipuAmdProfilerEnable(const char* dump_path);
DIPU_AMD_API int dipuAmdProfilerDisable(void);
DIPU_AMD_API int dipuAmdProfilerCounts(uint64_t* started, uint64_t* stopped, int* roctx_bound);

/* ---- allocator metrics: dipu/torch_dipu/csrc_dipu/runtime/core/allocator/allocator_metrics.h:17-160 (label sets
 * type / device / method / event) and metrics/metrics.cpp:5-11 (the switch, on by default). dipuAmdMetricsEnable:
 * update 0 / 1 sets the switch, anything else only reads it. dipuAmdMetricsText writes the Prometheus text
 * exposition of every value (allocator_event_count, allocator_size_bucket / _sum / _count), NUL-terminated and cut to
 * capacity; *needed is the size of the whole text. dipuAmdMetricsRecord feeds one allocate (deallocate = 0) or
 * deallocate event to the metrics of (type, device) directly, the call the allocators make. */
DIPU_AMD_API int dipuAmdMetricsEnable(int update, int* enabled);
DIPU_AMD_API int dipuAmdMetricsText(char* buffer, size_t capacity, size_t* needed);
DIPU_AMD_API int dipuAmdMetricsRecord(const char* type, int device, int deallocate, void* data, size_t size);

#if defined(__cplusplus)
}
#endif

#endif /* DIPU_AMD_RUNTIME_H_ */
