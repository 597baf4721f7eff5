// Shared host/device helpers for the MI355X DIOPI implementation library.
//
// Host side: a TensorView snapshot of what the diopirt callbacks report
// (the impl library never looks inside a handle; it only calls the runtime,
// as the reference's runtime contract requires:
// dipu/torch_dipu/csrc_dipu/diopirt/diopirt_impl.cpp:24-126), error plumbing
// for diopiGetLastErrorString, and launch helpers.
// Device side: wave64 reductions, 16-byte vector types, dtype conversion.
#pragma once

#include <hip/hip_runtime.h>

#include <utility>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include <diopi/diopirt.h>
#include <diopi/functions.h>
#include <diopi/functions_ext.h>

namespace amd {

constexpr int kMaxDims = 8;
constexpr int kWave = 64;

// ---------------------------------------------------------------- errors ----
void setLastError(const char* fmt, ...) __attribute__((format(printf, 1, 2)));

#define AMD_CHECK(cond, ...)                    \
  do {                                          \
    if (!(cond)) {                              \
      ::amd::setLastError(__VA_ARGS__);         \
      return diopiErrorOccurred;                \
    }                                           \
  } while (0)

#define AMD_TRY(expr)                           \
  do {                                          \
    diopiError_t _e = (expr);                   \
    if (_e != diopiSuccess) return _e;          \
  } while (0)

#define AMD_HIP(expr)                                                                         \
  do {                                                                                        \
    hipError_t _h = (expr);                                                                   \
    if (_h != hipSuccess) {                                                                   \
      ::amd::setLastError("%s failed: %s (%s:%d)", #expr, hipGetErrorString(_h), __FILE__, __LINE__); \
      return diopiErrorOccurred;                                                              \
    }                                                                                         \
  } while (0)

// Checked after every launch; clears nothing on success.
#define AMD_LAUNCH_CHECK() AMD_HIP(hipGetLastError())

// Raises a kernel's dynamic-LDS limit (kernels here use up to 128 KiB of the CU's 160 KiB; the
// default limit is 64 KiB). Done once per (kernel, device); callable from any thread before
// every launch.
hipError_t allowDynamicLds(const void* kernel, int bytes);

// Compute units of the current device (256 on MI355X), queried once; launch sizing only.
int computeUnits();

// ------------------------------------------------------------ tensor view ---
struct TensorView {
  void* data = nullptr;
  int ndim = 0;
  int64_t shape[kMaxDims] = {0};
  int64_t stride[kMaxDims] = {0};
  diopiDtype_t dtype = diopi_dtype_unsupported;
  int64_t numel = 0;
  int64_t itemsize = 0;

  bool defined() const { return dtype != diopi_dtype_unsupported; }
  bool isContiguous() const {
    int64_t expect = 1;
    for (int i = ndim - 1; i >= 0; --i) {
      if (shape[i] == 1) continue;
      if (stride[i] != expect) return false;
      expect *= shape[i];
    }
    return true;
  }
  template <typename T>
  T* ptr() const {
    return reinterpret_cast<T*>(data);
  }
  bool aligned16() const { return (reinterpret_cast<uintptr_t>(data) & 15) == 0; }
};

int64_t dtypeSize(diopiDtype_t dt);
const char* dtypeName(diopiDtype_t dt);
inline bool isFloatDtype(diopiDtype_t dt) {
  return dt == diopi_dtype_float16 || dt == diopi_dtype_bfloat16 || dt == diopi_dtype_float32 ||
         dt == diopi_dtype_float64;
}
inline bool isIntDtype(diopiDtype_t dt) {
  return dt == diopi_dtype_int8 || dt == diopi_dtype_uint8 || dt == diopi_dtype_int16 || dt == diopi_dtype_int32 ||
         dt == diopi_dtype_int64 || dt == diopi_dtype_bool;
}

// Fills `v` from the runtime callbacks. A null handle yields an undefined view.
diopiError_t getView(diopiConstTensorHandle_t th, TensorView* v, const char* what);
diopiError_t getStream(diopiContextHandle_t ctx, hipStream_t* stream);

// Workspace on the device owned by ctx (released by the runtime when ctx dies;
// valid for kernels enqueued on ctx's stream only).
diopiError_t requireWorkspace(diopiContextHandle_t ctx, int64_t nbytes, void** ptr);
// Contiguous temporary of the given shape/dtype, as a handle plus view.
diopiError_t requireTensor(diopiContextHandle_t ctx, const int64_t* shape, int ndim, diopiDtype_t dtype,
                           diopiTensorHandle_t* th, TensorView* view);

// dst <- src with broadcasting/strides/dtype conversion (the engine behind diopiCopyInp).
diopiError_t stridedCopy(hipStream_t stream, const TensorView& src, const TensorView& dst);
// Returns `v` itself when already contiguous, else a contiguous copy in ctx workspace.
diopiError_t makeContiguous(diopiContextHandle_t ctx, hipStream_t stream, const TensorView& v, TensorView* out);

double scalarToDouble(const diopiScalar_t* s, double dflt);
bool scalarIsFloat(const diopiScalar_t* s);
int64_t scalarToInt(const diopiScalar_t* s, int64_t dflt);

inline int64_t ceilDiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

// ---------------------------------------------------------------- device ----
#if defined(__HIPCC__)

typedef __bf16 bf16_t;
typedef _Float16 half_t;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));

// buffer_load_dwordx4 ... lds: lane l of the wave fetches 16 bytes at rsrc + voffset + soffset and the
// data lands in LDS at ldsAddr + 16 * l without passing through registers. Issued as inline assembly so
// that the compiler does not order it against fragment reads of the other stage; a kernel waits for
// these loads itself (vmcnt) before the barrier that publishes a stage. The LDS address travels in M0,
// which is read when the load issues; the previous M0 is put back so the statement has no side effect
// on registers the compiler owns.
__device__ __forceinline__ void loadToLds16(u32x4 rsrc, int voffset, int soffset, unsigned ldsAddr) {
  unsigned savedM0;
  asm volatile(
      "s_mov_b32 %0, m0\n\t"
      "s_mov_b32 m0, %1\n\t"
      "s_nop 0\n\t"
      "buffer_load_dwordx4 %2, %3, %4 offen lds\n\t"
      "s_mov_b32 m0, %0"
      : "=&s"(savedM0)
      : "s"(ldsAddr), "v"(voffset), "s"(rsrc), "s"(soffset)
      : "memory");
}

// The same copy from a flat global address per lane (global_load_lds_dwordx4), for kernels that address their operands
// with 64-bit pointers instead of a buffer descriptor.
__device__ __forceinline__ void globalLoadToLds16(const void* lanePtr, unsigned ldsAddr) {
  unsigned savedM0;
  asm volatile(
      "s_mov_b32 %0, m0\n\t"
      "s_mov_b32 m0, %1\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %2, off\n\t"
      "s_mov_b32 m0, %0"
      : "=&s"(savedM0)
      : "s"(ldsAddr), "v"(lanePtr)
      : "memory");
}

// The same copy marked non-temporal: for data that is read once (a weight stream), so that it does not push
// re-used lines (the activations every workgroup reads) out of L2.
__device__ __forceinline__ void loadToLds16Stream(u32x4 rsrc, int voffset, int soffset, unsigned ldsAddr) {
  unsigned savedM0;
  asm volatile(
      "s_mov_b32 %0, m0\n\t"
      "s_mov_b32 m0, %1\n\t"
      "s_nop 0\n\t"
      "buffer_load_dwordx4 %2, %3, %4 offen nt lds\n\t"
      "s_mov_b32 m0, %0"
      : "=&s"(savedM0)
      : "s"(ldsAddr), "v"(voffset), "s"(rsrc), "s"(soffset)
      : "memory");
}

template <int... Is, typename F>
__device__ __forceinline__ void staticForImpl(std::integer_sequence<int, Is...>, F&& f) {
  (f(std::integral_constant<int, Is>{}), ...);
}
// f(std::integral_constant<int, 0>{}) ... f(std::integral_constant<int, N - 1>{}): a loop whose index is a constant
// expression in the body (register names of inline assembly, array indices that must not become run-time).
template <int N, typename F>
__device__ __forceinline__ void staticFor(F&& f) {
  staticForImpl(std::make_integer_sequence<int, N>{}, f);
}

template <typename T>
struct Vec16 {  // 16 bytes of T
  static constexpr int N = 16 / sizeof(T);
  typedef T type __attribute__((ext_vector_type(16 / sizeof(T))));
};

// Reductions over the 64 lanes of a wave, the result in every lane. All lanes of the wave must be active. Within a
// row of 16 lanes the steps are lane permutations folded into the arithmetic instruction (quad swaps, then the mirror
// images within 8 and within 16 lanes, which pair every lane with one that holds the other half of the partial
// result); the four rows are then read out of lanes 0, 16, 32 and 48 and combined the same way by every lane. No
// trips through the LDS crossbar, which a shuffle by lane index takes once per step.
template <int CTRL>
__device__ __forceinline__ float lanePermuted(float v) {  // the value of the lane CTRL pairs this one with
  const int bits = __builtin_bit_cast(int, v);
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(bits, bits, CTRL, 0xf, 0xf, false));
}
constexpr int kDppQuadSwap1 = 0xB1, kDppQuadSwap2 = 0x4E, kDppHalfMirror = 0x141, kDppMirror = 0x140;
__device__ __forceinline__ float rowOfWave(float v, int row) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 16 * row));
}
__device__ __forceinline__ float waveSum(float v) {
  v += lanePermuted<kDppQuadSwap1>(v);
  v += lanePermuted<kDppQuadSwap2>(v);
  v += lanePermuted<kDppHalfMirror>(v);
  v += lanePermuted<kDppMirror>(v);
  return (rowOfWave(v, 0) + rowOfWave(v, 1)) + (rowOfWave(v, 2) + rowOfWave(v, 3));
}
__device__ __forceinline__ float waveMax(float v) {
  v = fmaxf(v, lanePermuted<kDppQuadSwap1>(v));
  v = fmaxf(v, lanePermuted<kDppQuadSwap2>(v));
  v = fmaxf(v, lanePermuted<kDppHalfMirror>(v));
  v = fmaxf(v, lanePermuted<kDppMirror>(v));
  return fmaxf(fmaxf(rowOfWave(v, 0), rowOfWave(v, 1)), fmaxf(rowOfWave(v, 2), rowOfWave(v, 3)));
}

__device__ __forceinline__ bool isFloatDtypeDev(int dt) {
  return dt == diopi_dtype_float16 || dt == diopi_dtype_bfloat16 || dt == diopi_dtype_float32 ||
         dt == diopi_dtype_float64;
}

// Runtime-dtype element load/store used by the generic (strided / mixed dtype) paths.
template <typename C>
__device__ __forceinline__ C loadAs(const void* base, int64_t idx, int dt) {
  switch (dt) {
    case diopi_dtype_float32: return static_cast<C>(reinterpret_cast<const float*>(base)[idx]);
    case diopi_dtype_bfloat16: return static_cast<C>(static_cast<float>(reinterpret_cast<const bf16_t*>(base)[idx]));
    case diopi_dtype_float16: return static_cast<C>(static_cast<float>(reinterpret_cast<const half_t*>(base)[idx]));
    case diopi_dtype_float64: return static_cast<C>(reinterpret_cast<const double*>(base)[idx]);
    case diopi_dtype_int64: return static_cast<C>(reinterpret_cast<const int64_t*>(base)[idx]);
    case diopi_dtype_int32: return static_cast<C>(reinterpret_cast<const int32_t*>(base)[idx]);
    case diopi_dtype_int16: return static_cast<C>(reinterpret_cast<const int16_t*>(base)[idx]);
    case diopi_dtype_int8: return static_cast<C>(reinterpret_cast<const int8_t*>(base)[idx]);
    case diopi_dtype_uint8: return static_cast<C>(reinterpret_cast<const uint8_t*>(base)[idx]);
    case diopi_dtype_bool: return static_cast<C>(reinterpret_cast<const uint8_t*>(base)[idx] != 0);
    default: return C(0);
  }
}
template <typename C>
__device__ __forceinline__ void storeAs(void* base, int64_t idx, int dt, C v) {
  switch (dt) {
    case diopi_dtype_float32: reinterpret_cast<float*>(base)[idx] = static_cast<float>(v); break;
    case diopi_dtype_bfloat16: reinterpret_cast<bf16_t*>(base)[idx] = static_cast<bf16_t>(static_cast<float>(v)); break;
    case diopi_dtype_float16: reinterpret_cast<half_t*>(base)[idx] = static_cast<half_t>(static_cast<float>(v)); break;
    case diopi_dtype_float64: reinterpret_cast<double*>(base)[idx] = static_cast<double>(v); break;
    case diopi_dtype_int64: reinterpret_cast<int64_t*>(base)[idx] = static_cast<int64_t>(v); break;
    case diopi_dtype_int32: reinterpret_cast<int32_t*>(base)[idx] = static_cast<int32_t>(v); break;
    case diopi_dtype_int16: reinterpret_cast<int16_t*>(base)[idx] = static_cast<int16_t>(v); break;
    case diopi_dtype_int8: reinterpret_cast<int8_t*>(base)[idx] = static_cast<int8_t>(v); break;
    case diopi_dtype_uint8: reinterpret_cast<uint8_t*>(base)[idx] = static_cast<uint8_t>(v); break;
    case diopi_dtype_bool: reinterpret_cast<uint8_t*>(base)[idx] = (v != C(0)) ? 1 : 0; break;
    default: break;
  }
}

#endif  // __HIPCC__

}  // namespace amd
