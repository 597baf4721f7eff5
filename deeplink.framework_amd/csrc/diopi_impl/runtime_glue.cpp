// Host-side glue between the DIOPI entry points and the diopirt callbacks.
// The impl library only ever learns about a tensor through these callbacks
// (dipu/torch_dipu/csrc_dipu/diopirt/diopirt_impl.cpp:24-173 is the provider in DIPU).
#include <cstring>
#include <mutex>
#include <set>
#include <utility>

#include "common.hpp"

namespace amd {

namespace {
thread_local char g_last_error[2048] = "";
}

void setLastError(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
}

const char* lastError() { return g_last_error; }

int computeUnits() {
  static const int cus = [] {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    return n;
  }();
  return cus;
}

hipError_t allowDynamicLds(const void* kernel, int bytes) {
  static std::mutex mu;
  static std::set<std::pair<const void*, int>> done;  // (kernel, device)
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return e;
  std::lock_guard<std::mutex> lock(mu);
  if (done.count({kernel, device})) return hipSuccess;
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e == hipSuccess) done.insert({kernel, device});
  return e;
}

int64_t dtypeSize(diopiDtype_t dt) {
  switch (dt) {
    case diopi_dtype_int8:
    case diopi_dtype_uint8:
    case diopi_dtype_bool: return 1;
    case diopi_dtype_int16:
    case diopi_dtype_uint16:
    case diopi_dtype_float16:
    case diopi_dtype_bfloat16: return 2;
    case diopi_dtype_int32:
    case diopi_dtype_uint32:
    case diopi_dtype_float32:
    case diopi_dtype_tfloat32:
    case diopi_dtype_complex32: return 4;
    case diopi_dtype_int64:
    case diopi_dtype_uint64:
    case diopi_dtype_float64:
    case diopi_dtype_complex64: return 8;
    case diopi_dtype_complex128: return 16;
    default: return 0;
  }
}

const char* dtypeName(diopiDtype_t dt) {
  switch (dt) {
    case diopi_dtype_int8: return "int8";
    case diopi_dtype_uint8: return "uint8";
    case diopi_dtype_int16: return "int16";
    case diopi_dtype_uint16: return "uint16";
    case diopi_dtype_int32: return "int32";
    case diopi_dtype_uint32: return "uint32";
    case diopi_dtype_int64: return "int64";
    case diopi_dtype_uint64: return "uint64";
    case diopi_dtype_float16: return "float16";
    case diopi_dtype_float32: return "float32";
    case diopi_dtype_float64: return "float64";
    case diopi_dtype_bool: return "bool";
    case diopi_dtype_bfloat16: return "bfloat16";
    case diopi_dtype_tfloat32: return "tfloat32";
    case diopi_dtype_complex32: return "complex32";
    case diopi_dtype_complex64: return "complex64";
    case diopi_dtype_complex128: return "complex128";
    default: return "unsupported";
  }
}

diopiError_t getView(diopiConstTensorHandle_t th, TensorView* v, const char* what) {
  *v = TensorView();
  if (th == nullptr) return diopiSuccess;
  diopiSize_t shape, stride;
  AMD_TRY(diopiGetTensorShape(th, &shape));
  AMD_TRY(diopiGetTensorStride(th, &stride));
  AMD_CHECK(shape.len <= kMaxDims, "%s: %ld dims exceed the supported maximum of %d", what, (long)shape.len, kMaxDims);
  AMD_CHECK(shape.len == stride.len, "%s: shape/stride rank mismatch", what);
  v->ndim = static_cast<int>(shape.len);
  int64_t numel = 1;
  for (int i = 0; i < v->ndim; ++i) {
    v->shape[i] = shape.data[i];
    v->stride[i] = stride.data[i];
    numel *= shape.data[i];
  }
  v->numel = numel;
  AMD_TRY(diopiGetTensorDtype(th, &v->dtype));
  v->itemsize = dtypeSize(v->dtype);
  AMD_CHECK(v->itemsize > 0, "%s: unsupported dtype %d", what, (int)v->dtype);
  const void* p = nullptr;
  AMD_TRY(diopiGetTensorDataConst(th, &p));
  v->data = const_cast<void*>(p);
  diopiDevice_t dev;
  AMD_TRY(diopiGetTensorDevice(th, &dev));
  AMD_CHECK(dev == diopi_device, "%s: tensor lives on the host; device tensor required", what);
  AMD_CHECK(numel == 0 || v->data != nullptr, "%s: null data pointer for a non-empty tensor", what);
  return diopiSuccess;
}

diopiError_t getStream(diopiContextHandle_t ctx, hipStream_t* stream) {
  AMD_CHECK(ctx != nullptr, "null diopiContext");
  diopiStreamHandle_t s = nullptr;
  AMD_TRY(diopiGetStream(ctx, &s));
  *stream = reinterpret_cast<hipStream_t>(s);
  return diopiSuccess;
}

diopiError_t requireWorkspace(diopiContextHandle_t ctx, int64_t nbytes, void** ptr) {
  diopiTensorHandle_t th = nullptr;
  if (nbytes < 1) nbytes = 1;
  AMD_CHECK(diopiRequireBuffer(ctx, &th, nbytes, diopi_device) == diopiSuccess,
            "diopiRequireBuffer failed for %ld bytes of workspace (the runtime holds the cause)", (long)nbytes);
  AMD_CHECK(th != nullptr, "diopiRequireBuffer returned a null handle for %ld bytes", (long)nbytes);
  AMD_TRY(diopiGetTensorData(th, ptr));
  AMD_CHECK(*ptr != nullptr, "diopiRequireBuffer returned null data for %ld bytes", (long)nbytes);
  return diopiSuccess;
}

diopiError_t requireTensor(diopiContextHandle_t ctx, const int64_t* shape, int ndim, diopiDtype_t dtype,
                           diopiTensorHandle_t* th, TensorView* view) {
  diopiSize_t size{shape, ndim};
  *th = nullptr;
  AMD_CHECK(diopiRequireTensor(ctx, th, &size, nullptr, dtype, diopi_device) == diopiSuccess,
            "diopiRequireTensor failed for a workspace tensor (the runtime holds the cause)");
  AMD_CHECK(*th != nullptr, "diopiRequireTensor returned a null handle");
  return getView(*th, view, "workspace tensor");
}

diopiError_t makeContiguous(diopiContextHandle_t ctx, hipStream_t stream, const TensorView& v, TensorView* out) {
  if (v.isContiguous()) {
    *out = v;
    // normalise strides so callers can index by shape alone
    int64_t expect = 1;
    for (int i = v.ndim - 1; i >= 0; --i) {
      out->stride[i] = expect;
      expect *= v.shape[i];
    }
    return diopiSuccess;
  }
  diopiTensorHandle_t th = nullptr;
  AMD_TRY(requireTensor(ctx, v.shape, v.ndim, v.dtype, &th, out));
  return stridedCopy(stream, v, *out);
}

double scalarToDouble(const diopiScalar_t* s, double dflt) {
  if (s == nullptr) return dflt;
  return s->stype == diopi_dtype_float64 ? s->fval : static_cast<double>(s->ival);
}
bool scalarIsFloat(const diopiScalar_t* s) { return s != nullptr && s->stype == diopi_dtype_float64; }
int64_t scalarToInt(const diopiScalar_t* s, int64_t dflt) {
  if (s == nullptr) return dflt;
  return s->stype == diopi_dtype_float64 ? static_cast<int64_t>(s->fval) : s->ival;
}

}  // namespace amd

namespace amd {
const char* lastError();
}

extern "C" __attribute__((visibility("default"))) const char* diopiGetLastErrorString(void) { return amd::lastError(); }
