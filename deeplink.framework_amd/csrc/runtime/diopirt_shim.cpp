// diopirt callbacks for a host that is not DIPU: tensors are plain descriptors
// (dipuAmdTensor) and workspace comes from this runtime's caching allocator.
// Same symbol set and behaviour as DIPU's provider,
// dipu/torch_dipu/csrc_dipu/diopirt/diopirt_impl.cpp:15-239 (an at::Tensor* there,
// a dipuAmdTensor* here; the impl library cannot tell the difference).
#include <cstring>
#include <list>
#include <mutex>
#include <string>

#include <diopi/diopirt.h>
#include <dipu_amd/runtime.h>

#include "runtime_core.h"

namespace dipu {
namespace amdrt {
void noteError(const char* what);  // c_api.cpp: text for dipuAmdGetLastError
}  // namespace amdrt
}  // namespace dipu

using dipu::amdrt::Runtime;

struct diopiTensor : dipuAmdTensor {};

struct diopiGenerator {
  mutable std::mutex mutex;
  uint64_t seed = 67280421310721ull;
  uint64_t offset = 0;
  int device_index = 0;
};

struct WorkspaceTensor {
  diopiTensor desc;
  void* allocation = nullptr;  // device pointer from the caching allocator, or host malloc
  bool onDevice = true;
};

// diopirt/diopirt_impl.h:19-26: stream + a list (stable addresses) that keeps workspace
// alive until the context dies.
struct diopiContext {
  dipu::deviceStream_t stream;
  std::list<WorkspaceTensor> arrays;
  explicit diopiContext(dipu::deviceStream_t s) : stream(s) {}
  void release() {
    for (auto& w : arrays) {
      if (!w.allocation) continue;
      if (w.onDevice) {
        Runtime::get().deviceFree(w.allocation);  // same-stream reuse keeps this safe while kernels are queued
      } else {
        ::free(w.allocation);
      }
    }
    arrays.clear();
  }
  ~diopiContext() {
    try {
      release();
    } catch (...) {
    }
  }
};

namespace {
int64_t elemSize(diopiDtype_t dt) {
  switch (dt) {
    case diopi_dtype_int8: case diopi_dtype_uint8: case diopi_dtype_bool: return 1;
    case diopi_dtype_int16: case diopi_dtype_uint16: case diopi_dtype_float16: case diopi_dtype_bfloat16: return 2;
    case diopi_dtype_int32: case diopi_dtype_uint32: case diopi_dtype_float32: case diopi_dtype_tfloat32:
    case diopi_dtype_complex32: return 4;
    case diopi_dtype_int64: case diopi_dtype_uint64: case diopi_dtype_float64: case diopi_dtype_complex64: return 8;
    case diopi_dtype_complex128: return 16;
    default: return 0;
  }
}
}  // namespace

extern "C" {

DIOPI_RT_API const char* diopiGetVersion() {
  static const std::string version = std::string("DIOPI Version: ") + std::to_string(DIOPI_VER_MAJOR) + "." +
                                     std::to_string(DIOPI_VER_MINOR) + "." + std::to_string(DIOPI_VER_PATCH);
  return version.c_str();
}

DIOPI_RT_API diopiError_t diopiGetTensorData(diopiTensorHandle_t th, void** pptr) {
  *pptr = th->data;
  return diopiSuccess;
}
DIOPI_RT_API diopiError_t diopiGetTensorDataConst(diopiConstTensorHandle_t th, const void** pptr) {
  *pptr = th->data;
  return diopiSuccess;
}
DIOPI_RT_API diopiError_t diopiGetTensorShape(diopiConstTensorHandle_t th, diopiSize_t* size) {
  *size = diopiSize_t{th->shape, th->ndim};
  return diopiSuccess;
}
DIOPI_RT_API diopiError_t diopiGetTensorStride(diopiConstTensorHandle_t th, diopiSize_t* stride) {
  *stride = diopiSize_t{th->stride, th->ndim};
  return diopiSuccess;
}
DIOPI_RT_API diopiError_t diopiGetTensorDtype(diopiConstTensorHandle_t th, diopiDtype_t* dtype) {
  *dtype = static_cast<diopiDtype_t>(th->dtype);
  return diopiSuccess;
}
DIOPI_RT_API diopiError_t diopiGetTensorDevice(diopiConstTensorHandle_t th, diopiDevice_t* device) {
  *device = static_cast<diopiDevice_t>(th->device);
  return diopiSuccess;
}
DIOPI_RT_API diopiError_t diopiGetTensorNumel(diopiConstTensorHandle_t th, int64_t* numel) {
  if (th == nullptr) {
    *numel = 0;
    return diopiSuccess;
  }
  int64_t n = 1;
  for (int64_t i = 0; i < th->ndim; ++i) n *= th->shape[i];
  *numel = n;
  return diopiSuccess;
}
DIOPI_RT_API diopiError_t diopiGetTensorElemSize(diopiConstTensorHandle_t th, int64_t* itemsize) {
  *itemsize = elemSize(static_cast<diopiDtype_t>(th->dtype));
  return diopiSuccess;
}
DIOPI_RT_API diopiError_t diopiGetTensorStoragePtr(diopiConstTensorHandle_t th, void** pStoragePtr) {
  *pStoragePtr = th->storage_ptr;
  return diopiSuccess;
}
DIOPI_RT_API diopiError_t diopiGetTensorStorageOffset(diopiConstTensorHandle_t th, int64_t* pOffset) {
  *pOffset = th->storage_offset;
  return diopiSuccess;
}
DIOPI_RT_API diopiError_t diopiGetTensorStorageNbytes(diopiConstTensorHandle_t th, size_t* pNbytes) {
  *pNbytes = th->storage_nbytes;
  return diopiSuccess;
}
DIOPI_RT_API diopiError_t diopiGetTensorDeviceIndex(diopiConstTensorHandle_t th, diopiDeviceIndex_t* pDevIndex) {
  *pDevIndex = th->device_index;
  return diopiSuccess;
}
DIOPI_RT_API diopiError_t diopiGetCurrentDeviceIndex(diopiDeviceIndex_t* pDevIndex) {
  try {
    *pDevIndex = dipu::devapis::current_device();
  } catch (...) {
    return diopiErrorOccurred;
  }
  return diopiSuccess;
}
DIOPI_RT_API diopiError_t diopiGetStream(diopiContextHandle_t ctx, diopiStreamHandle_t* stream) {
  *stream = ctx->stream;
  return diopiSuccess;
}

DIOPI_RT_API diopiError_t diopiRequireTensor(diopiContextHandle_t ctx, diopiTensorHandle_t* tensor,
                                             const diopiSize_t* size, const diopiSize_t* stride,
                                             const diopiDtype_t dtype, const diopiDevice_t device) {
  if (size->len > DIPU_AMD_MAX_DIMS || (stride && stride->len != size->len)) return diopiErrorOccurred;
  int64_t item = elemSize(dtype);
  if (item == 0) return diopiDtypeNotSupported;
  WorkspaceTensor w;
  w.desc = diopiTensor{};
  w.desc.ndim = size->len;
  int64_t numel = 1, span = 1;  // span: elements covered when strides are given
  int64_t expect = 1;
  for (int64_t i = size->len - 1; i >= 0; --i) {
    w.desc.shape[i] = size->data[i];
    w.desc.stride[i] = stride ? stride->data[i] : expect;
    expect *= size->data[i];
    numel *= size->data[i];
    if (size->data[i] > 0) span += (size->data[i] - 1) * w.desc.stride[i];
  }
  if (numel == 0) span = 0;
  w.desc.dtype = dtype;
  w.desc.device = device;
  w.desc.storage_offset = 0;
  w.desc.storage_nbytes = static_cast<uint64_t>(span * item);
  w.onDevice = device == diopi_device;
  try {
    if (w.onDevice) {
      w.desc.device_index = dipu::devapis::current_device();
      w.allocation = span > 0 ? Runtime::get().deviceMalloc(static_cast<size_t>(span * item), ctx->stream) : nullptr;
    } else {
      w.desc.device_index = -1;
      w.allocation = span > 0 ? ::malloc(static_cast<size_t>(span * item)) : nullptr;
    }
  } catch (const std::exception& e) {
    dipu::amdrt::noteError(e.what());
    return diopiErrorOccurred;
  } catch (...) {
    dipu::amdrt::noteError("diopiRequireTensor: unknown C++ exception");
    return diopiErrorOccurred;
  }
  w.desc.data = w.allocation;
  w.desc.storage_ptr = w.allocation;
  ctx->arrays.emplace_back(std::move(w));
  *tensor = &ctx->arrays.back().desc;
  return diopiSuccess;
}

DIOPI_RT_API diopiError_t diopiRequireBuffer(diopiContextHandle_t ctx, diopiTensorHandle_t* tensor, int64_t num_bytes,
                                             diopiDevice_t device) {
  diopiSize_t size{&num_bytes, 1};
  return diopiRequireTensor(ctx, tensor, &size, nullptr, diopi_dtype_int8, device);
}

// Generator state as the reference's CUDA vendor keeps it (dipu/torch_dipu/csrc_dipu/vendor/cuda/CudaGeneratorImpl.cpp:
// 17-76): a Philox seed and offset, serialised as 16 bytes on the host (seed, then offset; an 8-byte state is a seed
// with offset 0), the offset a multiple of 4. The inference path draws no random numbers; the callbacks are here so
// that an operator library that does can keep its counter (diopirt_impl.cpp:175-226).
DIOPI_RT_API diopiError_t diopiGeneratorGetState(diopiContextHandle_t ctx, diopiConstGeneratorHandle_t gen,
                                                 diopiTensorHandle_t* data) {
  if (!ctx || !gen || !data) return diopiErrorOccurred;
  const int64_t n = 16;
  diopiSize_t size{&n, 1};
  diopiError_t err = diopiRequireTensor(ctx, data, &size, nullptr, diopi_dtype_uint8, diopi_host);
  if (err != diopiSuccess) return err;
  uint64_t words[2];
  {
    std::lock_guard<std::mutex> lock(gen->mutex);
    words[0] = gen->seed, words[1] = gen->offset;
  }
  std::memcpy((*data)->data, words, sizeof(words));
  return diopiSuccess;
}
DIOPI_RT_API diopiError_t diopiGeneratorSetState(diopiGeneratorHandle_t gen, diopiConstTensorHandle_t state) {
  if (!gen || !state || state->device != diopi_host || state->dtype != diopi_dtype_uint8 || state->ndim != 1 ||
      state->stride[0] != 1 || (state->shape[0] != 16 && state->shape[0] != 8))
    return diopiErrorOccurred;  // "RNG state is wrong size" / not a byte tensor on the host
  uint64_t words[2] = {0, 0};
  std::memcpy(words, state->data, static_cast<size_t>(state->shape[0]));
  if (words[1] % 4 != 0) return diopiErrorOccurred;  // offset must be a multiple of 4
  std::lock_guard<std::mutex> lock(gen->mutex);
  gen->seed = words[0], gen->offset = words[1];
  return diopiSuccess;
}
DIOPI_RT_API diopiError_t diopiGeneratorGetSeedAndOffset(diopiGeneratorHandle_t gen, uint64_t* seed, uint64_t* offset) {
  if (!gen || !seed || !offset) return diopiErrorOccurred;
  std::lock_guard<std::mutex> lock(gen->mutex);
  *seed = gen->seed, *offset = gen->offset;
  return diopiSuccess;
}
DIOPI_RT_API diopiError_t diopiGeneratorSetSeedAndOffset(diopiGeneratorHandle_t gen, uint64_t seed, uint64_t offset) {
  if (!gen || offset % 4 != 0) return diopiErrorOccurred;
  std::lock_guard<std::mutex> lock(gen->mutex);
  gen->seed = seed, gen->offset = offset;
  return diopiSuccess;
}

// The object vendorMakeGenerator hands out (runtime/core/DIPUGeneratorImpl.h:62), without libtorch: seed 67280421310721
// is torch's default_rng_seed_val.
int dipuAmdGeneratorCreate(diopiGeneratorHandle_t* gen, int device_index) {
  if (!gen) return 1;
  auto* g = new diopiGenerator();
  g->device_index = device_index;
  *gen = g;
  return 0;
}
int dipuAmdGeneratorDestroy(diopiGeneratorHandle_t gen) {
  delete gen;
  return 0;
}

// Named host ranges: ROCTX ranges while devapis::enableProfiler is in effect, nothing otherwise
// (diopirt_impl.cpp:224-237 wraps the same pair around a RecordBlockCreator).
DIOPI_RT_API diopiError_t diopiRecordStart(const char* record_name, void** record) {
  if (!record) return diopiErrorOccurred;
  *record = dipu::profile::rangeStart(record_name);
  return diopiSuccess;
}
DIOPI_RT_API diopiError_t diopiRecordEnd(void** record) {
  if (!record) return diopiErrorOccurred;
  dipu::profile::rangeStop(*record);
  *record = nullptr;
  return diopiSuccess;
}

}  // extern "C"

// Context lifetime for the C facade (c_api.cpp).
namespace dipu {
namespace amdrt {
void* contextCreate(deviceStream_t s) { return new diopiContext(s); }
void contextDestroy(void* c) { delete static_cast<diopiContext*>(c); }
void contextReset(void* c) { static_cast<diopiContext*>(c)->release(); }
void contextWorkspace(void* c, uint64_t* tensors, uint64_t* bytes) {
  auto* ctx = static_cast<diopiContext*>(c);
  *tensors = ctx->arrays.size();
  uint64_t b = 0;
  for (auto& w : ctx->arrays) b += w.desc.storage_nbytes;
  *bytes = b;
}
}  // namespace amdrt
}  // namespace dipu
