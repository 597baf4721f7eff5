/*
 * DIOPI runtime interface (types + callbacks), reconstructed for the MI355X backend.
 *
 * The upstream DIOPI headers are an un-vendored submodule of the reference
 * (/root/reference/.gitmodules:1-6, dipu/third_party/DIOPI is empty), so every
 * declaration below is pinned to the reference call site that uses it:
 *
 *   handle/scalar/size/dtype/device conversions ... dipu/torch_dipu/csrc_dipu/diopirt/diopi_helper.cpp:9-261
 *   runtime callbacks (the symbols an impl library imports) ... dipu/torch_dipu/csrc_dipu/diopirt/diopirt_impl.cpp:15-239
 *   struct diopiContext is owned by the runtime side ... dipu/torch_dipu/csrc_dipu/diopirt/diopirt_impl.h:19-26
 *
 * Enumerator NAMES are the reference's; their numeric VALUES are not recoverable
 * from the reference (it only uses the names) and follow upstream DIOPI as
 * recalled. They are isolated in this one header so a maintainer can correct
 * them against the real diopirt.h without touching any kernel.
 */
#ifndef DIOPI_DIOPIRT_H_
#define DIOPI_DIOPIRT_H_

#include <stddef.h>
#include <stdint.h>

#ifndef DIOPI_ATTR_WEAK
#define DIOPI_ATTR_WEAK
#endif

#if defined(__cplusplus)
#define DIOPI_API extern "C" __attribute__((visibility("default"))) DIOPI_ATTR_WEAK
#define DIOPI_RT_API extern "C" __attribute__((visibility("default")))
#else
#define DIOPI_API __attribute__((visibility("default"))) DIOPI_ATTR_WEAK
#define DIOPI_RT_API __attribute__((visibility("default")))
#endif

#define DIOPI_VER_MAJOR 1
#define DIOPI_VER_MINOR 0
#define DIOPI_VER_PATCH 0

#if defined(__cplusplus)
extern "C" {
#endif

/* dipu/torch_dipu/csrc_dipu/diopirt/diopi_helper.cpp:229-243 and diopirt_impl.cpp:39:
 * a borrowed (pointer, length) pair, passed by value. */
typedef struct diopiSize_t_ {
  const int64_t* data;
  int64_t len;
} diopiSize_t;

/* names: diopi_helper.cpp:121-215. Order below follows upstream DIOPI. */
typedef enum {
  diopi_dtype_int8 = 0,
  diopi_dtype_uint8 = 1,
  diopi_dtype_int16 = 2,
  diopi_dtype_uint16 = 3,
  diopi_dtype_int32 = 4,
  diopi_dtype_uint32 = 5,
  diopi_dtype_int64 = 6,
  diopi_dtype_uint64 = 7,
  diopi_dtype_float16 = 8,
  diopi_dtype_float32 = 9,
  diopi_dtype_float64 = 10,
  diopi_dtype_bool = 11,
  diopi_dtype_bfloat16 = 12,
  diopi_dtype_tfloat32 = 13,
  diopi_dtype_complex32 = 14,
  diopi_dtype_complex64 = 15,
  diopi_dtype_complex128 = 16,
  diopi_dtype_unsupported = 255
} diopiDtype_t;

/* diopi_helper.cpp:218-227 */
typedef enum { diopi_host = 0, diopi_device = 1 } diopiDevice_t;

/* diopirt_impl.cpp:111-121 */
typedef int32_t diopiDeviceIndex_t;

/* diopiSuccess / diopiForceFallbackToCPU are named by the generated wrappers
 * (dipu/scripts/autogen_diopi_wrapper/autogen_diopi_wrapper.py:404-439,1001). */
typedef enum {
  diopiSuccess = 0,
  diopiErrorOccurred = 1,
  diopiNotInited = 2,
  diopiNoRegisteredStreamCreateFunction = 3,
  diopiNoRegisteredStreamDestoryFunction = 4,
  diopiNoRegisteredStreamSyncFunction = 5,
  diopiNoRegisteredDeviceMemoryMallocFunction = 6,
  diopiNoRegisteredDeviceMemoryFreeFunction = 7,
  diopiNoRegisteredDevice2DdeviceMemoryCopyFunction = 8,
  diopiNoRegisteredDevice2HostMemoryCopyFunction = 9,
  diopiNoRegisteredHost2DeviceMemoryCopyFunction = 10,
  diopiNoRegisteredGetLastErrorFunction = 11,
  diopi5DNotSupported = 12,
  diopiNoImplement = 13,
  diopiForceFallbackToCPU = 14,
  diopiDtypeNotSupported = 1000
} diopiError_t;

/* diopi_helper.cpp:245-259 */
typedef enum { RoundModeNone = 0, RoundModeFloor = 1, RoundModeTrunc = 2, RoundModeEND = 3 } diopiRoundMode_t;

/* dipu/scripts/autogen_diopi_wrapper/diopi_functions.yaml:602-617 casts ATen's int */
typedef enum { ReductionNone = 0, ReductionMean = 1, ReductionSum = 2, ReductionEND = 3 } diopiReduction_t;

/* diopi_helper.cpp:74-97: only int64 and float64 payloads are ever produced */
typedef struct diopiScalar_t_ {
  diopiDtype_t stype;
  union {
    double fval;
    int64_t ival;
  };
} diopiScalar_t;

/* Opaque to an impl library. The runtime side defines the structs:
 * DIPU uses {deviceStream_t stream; std::list<at::Tensor> arrays;} and at::Tensor*. */
struct diopiContext;
typedef struct diopiContext* diopiContextHandle_t;
struct diopiTensor;
typedef struct diopiTensor* diopiTensorHandle_t;
typedef const struct diopiTensor* diopiConstTensorHandle_t;
struct diopiGenerator;
typedef struct diopiGenerator* diopiGeneratorHandle_t;
typedef const struct diopiGenerator* diopiConstGeneratorHandle_t;
/* diopirt_impl.cpp:122-126: the raw vendor stream (hipStream_t on this backend) */
typedef void* diopiStreamHandle_t;

/* ---- callbacks the impl library IMPORTS (diopirt_impl.cpp:17-237) ---- */
DIOPI_RT_API const char* diopiGetVersion(void);
DIOPI_RT_API diopiError_t diopiGetTensorData(diopiTensorHandle_t th, void** pptr);
DIOPI_RT_API diopiError_t diopiGetTensorDataConst(diopiConstTensorHandle_t th, const void** pptr);
DIOPI_RT_API diopiError_t diopiGetTensorShape(diopiConstTensorHandle_t th, diopiSize_t* size);
DIOPI_RT_API diopiError_t diopiGetTensorStride(diopiConstTensorHandle_t th, diopiSize_t* stride);
DIOPI_RT_API diopiError_t diopiGetTensorDtype(diopiConstTensorHandle_t th, diopiDtype_t* dtype);
DIOPI_RT_API diopiError_t diopiGetTensorDevice(diopiConstTensorHandle_t th, diopiDevice_t* device);
DIOPI_RT_API diopiError_t diopiGetTensorNumel(diopiConstTensorHandle_t th, int64_t* numel);
DIOPI_RT_API diopiError_t diopiGetTensorElemSize(diopiConstTensorHandle_t th, int64_t* itemsize);
DIOPI_RT_API diopiError_t diopiGetTensorStoragePtr(diopiConstTensorHandle_t th, void** pStoragePtr);
DIOPI_RT_API diopiError_t diopiGetTensorStorageOffset(diopiConstTensorHandle_t th, int64_t* pOffset);
DIOPI_RT_API diopiError_t diopiGetTensorStorageNbytes(diopiConstTensorHandle_t th, size_t* pNbytes);
DIOPI_RT_API diopiError_t diopiGetTensorDeviceIndex(diopiConstTensorHandle_t th, diopiDeviceIndex_t* pDevIndex);
DIOPI_RT_API diopiError_t diopiGetCurrentDeviceIndex(diopiDeviceIndex_t* pDevIndex);
DIOPI_RT_API diopiError_t diopiGetStream(diopiContextHandle_t ctx, diopiStreamHandle_t* stream);
DIOPI_RT_API diopiError_t diopiRequireTensor(diopiContextHandle_t ctx, diopiTensorHandle_t* tensor,
                                             const diopiSize_t* size, const diopiSize_t* stride,
                                             const diopiDtype_t dtype, const diopiDevice_t device);
DIOPI_RT_API diopiError_t diopiRequireBuffer(diopiContextHandle_t ctx, diopiTensorHandle_t* tensor,
                                             int64_t num_bytes, diopiDevice_t device);
DIOPI_RT_API diopiError_t diopiGeneratorGetState(diopiContextHandle_t ctx, diopiConstGeneratorHandle_t th,
                                                 diopiTensorHandle_t* data);
DIOPI_RT_API diopiError_t diopiGeneratorSetState(diopiGeneratorHandle_t th, diopiConstTensorHandle_t state);
DIOPI_RT_API diopiError_t diopiGeneratorGetSeedAndOffset(diopiGeneratorHandle_t th, uint64_t* seed,
                                                         uint64_t* offset);
DIOPI_RT_API diopiError_t diopiGeneratorSetSeedAndOffset(diopiGeneratorHandle_t th, uint64_t seed,
                                                         uint64_t offset);
DIOPI_RT_API diopiError_t diopiRecordStart(const char* record_name, void** record);
DIOPI_RT_API diopiError_t diopiRecordEnd(void** record);

#if defined(__cplusplus)
}
#endif

#endif /* DIOPI_DIOPIRT_H_ */
