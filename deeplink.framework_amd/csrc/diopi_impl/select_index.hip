// Selection, masking, comparison and gather-style DIOPI ops for gfx950: where, masked_fill,
// tril/triu, arange, index_select, gather and eq/ne/lt/le/gt/ge (+Scalar forms).
//
// These are the helpers a decoder layer falls back on when model code builds its causal
// mask and its rotary position tables out of primitive aten ops instead of the fused ext
// ops (dipu/scripts/autogen_diopi_wrapper/diopi_functions.yaml:405-549 comparisons,
// :1191-1197 tril, :1432-1453 masked_fill, :1566-1571 where, :1923-1933 gather and
// index_select, :2341-2347 arange, :2505-2516 triu).
//
// All of them are pure data movement or one comparison per element, so one strided,
// broadcasting, run-time-dtype kernel shape serves all: a lane owns one output element,
// walks the coalesced dims to get each operand's offset, and moves the value through a
// lossless carrier type (double for floating outputs, int64 for integral ones: every
// supported dtype round-trips exactly through its carrier, so moved values are bit-exact).
// Neighbouring lanes touch neighbouring elements whenever the innermost dim is dense.
// Out-of-range indices in index_select / gather are never dereferenced: the element is
// written as zero.
#include "common.hpp"

namespace amd {

constexpr int kSelOperands = 4;  // 0 = out, 1..3 = inputs
constexpr int kSelThreads = 256;

struct Strided4 {
  int ndim;
  int64_t shape[kMaxDims];
  int64_t st[kSelOperands][kMaxDims];
};

struct Offsets4 {
  int64_t o[kSelOperands];
};

__device__ __forceinline__ Offsets4 offsetsOf(const Strided4& s, int64_t i) {
  Offsets4 r;
#pragma unroll
  for (int k = 0; k < kSelOperands; ++k) r.o[k] = 0;
  if (s.ndim == 1) {  // everything merged into one run: no division at all
#pragma unroll
    for (int k = 0; k < kSelOperands; ++k) r.o[k] = i * s.st[k][0];
    return r;
  }
  if (i < ((int64_t)1 << 31)) {  // 32-bit divisions (an index below 2^31 has every quotient and remainder below it)
    unsigned rem = (unsigned)i;
    for (int d = s.ndim - 1; d >= 0 && rem != 0; --d) {
      const unsigned extent = s.shape[d] >= ((int64_t)1 << 31) ? 0x80000000u : (unsigned)s.shape[d];
      const unsigned q = rem / extent;
      const unsigned c = rem - q * extent;
      rem = q;
#pragma unroll
      for (int k = 0; k < kSelOperands; ++k) r.o[k] += (int64_t)c * s.st[k][d];
    }
    return r;
  }
  int64_t rem = i;
  for (int d = s.ndim - 1; d >= 0; --d) {
    int64_t q = rem / s.shape[d];
    int64_t c = rem - q * s.shape[d];
    rem = q;
#pragma unroll
    for (int k = 0; k < kSelOperands; ++k) r.o[k] += c * s.st[k][d];
  }
  return r;
}

// ------------------------------------------------------------------ kernels
// out = cond ? a : b on dense operands of one 2-byte or 4-byte dtype with a 1-byte condition: 8 elements per lane,
// moved as bits (a: tensor, or the scalar's bits in the output dtype when aBits is used).
template <typename E>
__global__ __launch_bounds__(kSelThreads) void selectVecKernel(E* __restrict__ out, const uint8_t* __restrict__ cond,
                                                               const E* __restrict__ a, const E* __restrict__ b, int64_t nvec,
                                                               int64_t condVecs, E aBits) {
  typedef E E8 __attribute__((ext_vector_type(8)));
  typedef uint8_t C8 __attribute__((ext_vector_type(8)));
  const int64_t i = (int64_t)blockIdx.x * kSelThreads + threadIdx.x;
  if (i >= nvec) return;
  // a condition that covers the trailing dims only repeats every condVecs vectors (a [s, s] mask on [b, h, s, s] scores)
  const C8 c = reinterpret_cast<const C8*>(cond)[condVecs == nvec ? i : i % condVecs];
  const E8 vb = reinterpret_cast<const E8*>(b)[i];
  E8 va;
  if (a != nullptr) {
    va = reinterpret_cast<const E8*>(a)[i];
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) va[j] = aBits;
  }
  E8 r;
#pragma unroll
  for (int j = 0; j < 8; ++j) r[j] = c[j] != 0 ? va[j] : vb[j];
  reinterpret_cast<E8*>(out)[i] = r;
}

// out = cond ? a : b. `a` is the scalar `sa` when aScalar (masked_fill with a Scalar value).
template <typename C>
__global__ __launch_bounds__(kSelThreads) void selectKernel(void* out, const void* cond, const void* a, const void* b,
                                                            int dto, int dtc, int dta, int dtb, Strided4 s, int64_t n,
                                                            C sa, bool aScalar) {
  for (int64_t i = (int64_t)blockIdx.x * kSelThreads + threadIdx.x; i < n; i += (int64_t)gridDim.x * kSelThreads) {
    Offsets4 o = offsetsOf(s, i);
    bool c = loadAs<int64_t>(cond, o.o[1], dtc) != 0;
    C v;
    if (c)
      v = aScalar ? sa : loadAs<C>(a, o.o[2], dta);
    else
      v = loadAs<C>(b, o.o[3], dtb);
    storeAs<C>(out, o.o[0], dto, v);
  }
}

enum CmpOp : int { kEq = 0, kNe, kLt, kLe, kGt, kGe };

__device__ __forceinline__ bool compareOne(float x, float y, int cmp) {
  switch (cmp) {
    case kEq: return x == y;
    case kNe: return x != y;
    case kLt: return x < y;
    case kLe: return x <= y;
    case kGt: return x > y;
    default: return x >= y;
  }
}

// out = a CMP b on dense operands of one floating dtype (b may be the scalar sb, already rounded to that dtype) into a
// dense 1-byte output: 8 elements per lane.
template <typename T>
__global__ __launch_bounds__(kSelThreads) void compareVecKernel(uint8_t* __restrict__ out, const T* __restrict__ a,
                                                                const T* __restrict__ b, int64_t nvec, int cmp, float sb) {
  typedef T T8 __attribute__((ext_vector_type(8)));
  typedef uint8_t C8 __attribute__((ext_vector_type(8)));
  const int64_t i = (int64_t)blockIdx.x * kSelThreads + threadIdx.x;
  if (i >= nvec) return;
  const T8 va = reinterpret_cast<const T8*>(a)[i];
  T8 vb;
  if (b != nullptr) vb = reinterpret_cast<const T8*>(b)[i];
  C8 r;
#pragma unroll
  for (int j = 0; j < 8; ++j)
    r[j] = compareOne(static_cast<float>(va[j]), b != nullptr ? static_cast<float>(vb[j]) : sb, cmp) ? 1 : 0;
  reinterpret_cast<C8*>(out)[i] = r;
}

// out = a CMP b; `b` is the scalar `sb` when bScalar.
template <typename C>
__global__ __launch_bounds__(kSelThreads) void compareKernel(void* out, const void* a, const void* b, int dto, int dta,
                                                             int dtb, Strided4 s, int64_t n, int cmp, C sb,
                                                             bool bScalar) {
  for (int64_t i = (int64_t)blockIdx.x * kSelThreads + threadIdx.x; i < n; i += (int64_t)gridDim.x * kSelThreads) {
    Offsets4 o = offsetsOf(s, i);
    C x = loadAs<C>(a, o.o[1], dta);
    C y = bScalar ? sb : loadAs<C>(b, o.o[2], dtb);
    bool r;
    switch (cmp) {
      case kEq: r = x == y; break;
      case kNe: r = x != y; break;
      case kLt: r = x < y; break;
      case kLe: r = x <= y; break;
      case kGt: r = x > y; break;
      default: r = x >= y; break;
    }
    storeAs<int64_t>(out, o.o[0], dto, r ? 1 : 0);
  }
}

// The last two dims of `s` are (row, col); out = keep(row, col) ? x : 0 with
// keep = col - row <= diag (lower) or col - row >= diag (upper).
template <typename C>
__global__ __launch_bounds__(kSelThreads) void triangleKernel(void* out, const void* x, int dto, int dtx, Strided4 s,
                                                              int64_t n, int64_t diag, bool lower) {
  const int64_t cols = s.shape[s.ndim - 1], rows = s.shape[s.ndim - 2];
  for (int64_t i = (int64_t)blockIdx.x * kSelThreads + threadIdx.x; i < n; i += (int64_t)gridDim.x * kSelThreads) {
    Offsets4 o = offsetsOf(s, i);
    int64_t c = i % cols, r = (i / cols) % rows;
    bool keep = lower ? (c - r <= diag) : (c - r >= diag);
    C v = keep ? loadAs<C>(x, o.o[1], dtx) : C(0);
    storeAs<C>(out, o.o[0], dto, v);
  }
}

// tril / triu on dense [..., rows, cols] of one 2-byte or 4-byte dtype, cols a multiple of 8: 8 elements per lane as bits.
template <typename E>
__global__ __launch_bounds__(kSelThreads) void triangleVecKernel(E* __restrict__ out, const E* __restrict__ x, int64_t nvec,
                                                                 int rowVecs, int64_t rows, int64_t diag, bool lower) {
  typedef E E8 __attribute__((ext_vector_type(8)));
  const int64_t i = (int64_t)blockIdx.x * kSelThreads + threadIdx.x;
  if (i >= nvec) return;
  const int64_t rowAll = i / rowVecs, c0 = (i - rowAll * rowVecs) * 8, r = rowAll % rows;
  // the whole piece on the zero side: no load
  const bool allZero = lower ? (c0 - r > diag) : (c0 + 7 - r < diag);
  E8 v;
  if (allZero) {
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = 0;
  } else {
    v = reinterpret_cast<const E8*>(x)[i];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int64_t d = c0 + j - r;
      if (!(lower ? d <= diag : d >= diag)) v[j] = 0;
    }
  }
  reinterpret_cast<E8*>(out)[i] = v;
}

template <typename C>
__global__ __launch_bounds__(kSelThreads) void arangeKernel(void* out, int dto, int64_t stride, int64_t n, C start,
                                                            C step) {
  for (int64_t i = (int64_t)blockIdx.x * kSelThreads + threadIdx.x; i < n; i += (int64_t)gridDim.x * kSelThreads)
    storeAs<C>(out, i * stride, dto, start + static_cast<C>(i) * step);
}

// out[idx] = src[idx with idx[dim] := index[...]]. st[1] holds src strides with the entry for `dim`
// zeroed (the index supplies that coordinate), st[2] the index tensor's strides (gather: the full
// index coordinates; index_select: only `dim` moves through the 1-d index).
template <typename C>
__global__ __launch_bounds__(kSelThreads) void gatherKernel(void* out, const void* src, const void* index, int dto,
                                                            int dts, int dti, Strided4 s, int64_t n, int64_t dimStride,
                                                            int64_t dimSize) {
  for (int64_t i = (int64_t)blockIdx.x * kSelThreads + threadIdx.x; i < n; i += (int64_t)gridDim.x * kSelThreads) {
    Offsets4 o = offsetsOf(s, i);
    int64_t j = loadAs<int64_t>(index, o.o[2], dti);
    C v = C(0);
    if (j >= 0 && j < dimSize) v = loadAs<C>(src, o.o[1] + j * dimStride, dts);
    storeAs<C>(out, o.o[0], dto, v);
  }
}

// index_select of dense blocks: out[o, i, :] = src[o, index[i], :] with `inner` contiguous 16-byte vectors per block
// (an embedding lookup is outer = 1, inner = the hidden size). One workgroup per output block; an index outside the
// source writes zeros, as the one-element kernel does.
template <typename IDX>
__global__ __launch_bounds__(256) void selectRowsKernel(u32x4* __restrict__ out, const u32x4* __restrict__ src,
                                                        const IDX* __restrict__ index, int64_t indexStride, int64_t nIndex,
                                                        int64_t dimSize, int64_t innerVecs) {
  const int64_t blk = blockIdx.x, o = blk / nIndex, i = blk - o * nIndex;
  const int64_t j = static_cast<int64_t>(index[i * indexStride]);
  const bool ok = j >= 0 && j < dimSize;
  const u32x4* s = src + (o * dimSize + (ok ? j : 0)) * innerVecs;
  u32x4* d = out + blk * innerVecs;
  for (int64_t v = threadIdx.x; v < innerVecs; v += 256) d[v] = ok ? s[v] : u32x4{0, 0, 0, 0};
}

// --------------------------------------------------------------------- host
static void clearStrided(Strided4* s, const TensorView& out) {
  s->ndim = out.ndim;
  for (int d = 0; d < kMaxDims; ++d) {
    s->shape[d] = 1;
    for (int k = 0; k < kSelOperands; ++k) s->st[k][d] = 0;
  }
  for (int d = 0; d < out.ndim; ++d) {
    s->shape[d] = out.shape[d];
    s->st[0][d] = out.shape[d] == 1 ? 0 : out.stride[d];
  }
}

// Right-aligns `v` against `out`; stride 0 wherever v has extent 1 or no dim at all.
static diopiError_t broadcastInto(const TensorView& out, const TensorView& v, int64_t* strides, const char* what) {
  AMD_CHECK(v.ndim <= out.ndim, "%s: rank %d cannot broadcast to output rank %d", what, v.ndim, out.ndim);
  int shift = out.ndim - v.ndim;
  for (int d = 0; d < out.ndim; ++d) {
    if (d < shift) {
      strides[d] = 0;
      continue;
    }
    int64_t e = v.shape[d - shift];
    AMD_CHECK(e == out.shape[d] || e == 1, "%s: extent %ld at dim %d cannot broadcast to %ld", what, (long)e,
              d - shift, (long)out.shape[d]);
    strides[d] = (e == 1) ? 0 : v.stride[d - shift];
  }
  return diopiSuccess;
}

// Merges neighbouring dims that are jointly dense for every operand; keeps the last `keepTail`
// dims as they are (the triangle kernel needs row and col separate).
static void coalesce(Strided4* s, int keepTail) {
  int w = 0;
  const int fixedFrom = s->ndim - keepTail;
  for (int d = 0; d < s->ndim; ++d) {
    bool fixed = d >= fixedFrom;
    if (s->shape[d] == 1 && !fixed) continue;
    bool merge = w > 0 && !fixed;  // fixed dims come last, so everything written so far is mergeable
    if (merge)
      for (int k = 0; k < kSelOperands; ++k) merge = merge && s->st[k][w - 1] == s->st[k][d] * s->shape[d];
    if (merge) {
      s->shape[w - 1] *= s->shape[d];
      for (int k = 0; k < kSelOperands; ++k) s->st[k][w - 1] = s->st[k][d];
    } else {
      s->shape[w] = s->shape[d];
      for (int k = 0; k < kSelOperands; ++k) s->st[k][w] = s->st[k][d];
      ++w;
    }
  }
  if (w == 0) {
    s->shape[0] = 1;
    for (int k = 0; k < kSelOperands; ++k) s->st[k][0] = 0;
    w = 1;
  }
  s->ndim = w;
}

static unsigned gridFor(int64_t n) {
  int64_t blocks = ceilDiv(n, kSelThreads);
  return (unsigned)(blocks > 65536 ? 65536 : blocks);
}

static bool supportedDtype(diopiDtype_t dt) { return isFloatDtype(dt) || isIntDtype(dt); }

static diopiError_t runSelect(diopiContextHandle_t ctx, diopiTensorHandle_t outH, diopiConstTensorHandle_t condH,
                              diopiConstTensorHandle_t aH, const diopiScalar_t* aScalar, diopiConstTensorHandle_t bH,
                              const char* name) {
  hipStream_t stream;
  AMD_TRY(getStream(ctx, &stream));
  TensorView out, cond, a, b;
  AMD_TRY(getView(outH, &out, "out"));
  AMD_TRY(getView(condH, &cond, "condition"));
  AMD_TRY(getView(bH, &b, "other"));
  AMD_CHECK(out.defined() && cond.defined() && b.defined(), "%s: null tensor", name);
  AMD_CHECK(supportedDtype(out.dtype) && supportedDtype(b.dtype), "%s: unsupported dtype %s", name,
            dtypeName(out.dtype));
  AMD_CHECK(isIntDtype(cond.dtype), "%s: condition must be bool or integral, got %s", name, dtypeName(cond.dtype));
  if (!aScalar) {
    AMD_TRY(getView(aH, &a, "input"));
    AMD_CHECK(a.defined() && supportedDtype(a.dtype), "%s: null or unsupported value tensor", name);
  }
  if (out.numel == 0) return diopiSuccess;
  Strided4 s;
  clearStrided(&s, out);
  AMD_TRY(broadcastInto(out, cond, s.st[1], "condition"));
  if (!aScalar) AMD_TRY(broadcastInto(out, a, s.st[2], "input"));
  AMD_TRY(broadcastInto(out, b, s.st[3], "other"));
  coalesce(&s, 0);
  const int dta = aScalar ? (int)out.dtype : (int)a.dtype;
  // Everything dense, one dtype of 2 or 4 bytes, a 1-byte condition: values move as bits, 8 per lane
  // ([8192, 4096] bf16 masked_fill: 100 us one element per lane).
  {
    auto dense = [&](const TensorView& t) {
      if (!t.isContiguous() || t.ndim != out.ndim) return false;
      for (int d = 0; d < out.ndim; ++d)
        if (t.shape[d] != out.shape[d]) return false;
      return true;
    };
    // the condition: dense like the output, or dense over the trailing dims and broadcast over all the leading ones
    auto trailing = [&](const TensorView& t) {
      if (!t.isContiguous() || t.ndim > out.ndim || t.numel % 8 != 0 || t.numel == 0) return false;
      int64_t covered = 1;
      bool lead = false;  // once a dim is broadcast, every dim before it must be too
      for (int d = out.ndim - 1; d >= 0; --d) {
        const int td = d - (out.ndim - t.ndim);
        const int64_t e = td >= 0 ? t.shape[td] : 1;
        if (lead) {
          if (e != 1) return false;
        } else if (e == out.shape[d]) {
          covered *= e;
        } else if (e == 1) {
          lead = true;
        } else {
          return false;
        }
      }
      return covered == t.numel;
    };
    const bool floatScalarIntoInt = aScalar && scalarIsFloat(aScalar) && !isFloatDtype(out.dtype);
    if ((out.itemsize == 2 || out.itemsize == 4) && out.numel % 8 == 0 && out.isContiguous() && out.aligned16() &&
        (dense(cond) || trailing(cond)) && cond.itemsize == 1 && (reinterpret_cast<uintptr_t>(cond.data) & 7) == 0 && dense(b) && b.dtype == out.dtype && b.aligned16() &&
        (aScalar ? !floatScalarIntoInt : (dense(a) && a.dtype == out.dtype && a.aligned16()))) {
      // the scalar in the output dtype's bits, through the same conversion the one-element path applies
      uint32_t bits = 0;
      if (aScalar) {
        if (out.dtype == diopi_dtype_bfloat16) {
          const bf16_t v = static_cast<bf16_t>(static_cast<float>(scalarToDouble(aScalar, 0.0)));
          bits = __builtin_bit_cast(uint16_t, v);
        } else if (out.dtype == diopi_dtype_float16) {
          const half_t v = static_cast<half_t>(static_cast<float>(scalarToDouble(aScalar, 0.0)));
          bits = __builtin_bit_cast(uint16_t, v);
        } else if (out.dtype == diopi_dtype_float32) {
          bits = __builtin_bit_cast(uint32_t, static_cast<float>(scalarToDouble(aScalar, 0.0)));
        } else {
          bits = (uint32_t)scalarToInt(aScalar, 0);
        }
      }
      const int64_t nvec = out.numel / 8, blocks = ceilDiv(nvec, kSelThreads), condVecs = cond.numel / 8;
      AMD_CHECK(blocks <= 0x7fffffff, "%s: %ld elements exceed the grid limit", name, (long)out.numel);
      if (out.itemsize == 2)
        hipLaunchKernelGGL((selectVecKernel<uint16_t>), dim3((unsigned)blocks), dim3(kSelThreads), 0, stream, out.ptr<uint16_t>(),
                           cond.ptr<uint8_t>(), aScalar ? nullptr : a.ptr<uint16_t>(), b.ptr<uint16_t>(), nvec, condVecs,
                           (uint16_t)bits);
      else
        hipLaunchKernelGGL((selectVecKernel<uint32_t>), dim3((unsigned)blocks), dim3(kSelThreads), 0, stream, out.ptr<uint32_t>(),
                           cond.ptr<uint8_t>(), aScalar ? nullptr : a.ptr<uint32_t>(), b.ptr<uint32_t>(), nvec, condVecs, bits);
      AMD_LAUNCH_CHECK();
      return diopiSuccess;
    }
  }
  if (isFloatDtype(out.dtype)) {
    hipLaunchKernelGGL((selectKernel<double>), dim3(gridFor(out.numel)), dim3(kSelThreads), 0, stream, out.data,
                       cond.data, aScalar ? nullptr : a.data, b.data, (int)out.dtype, (int)cond.dtype, dta,
                       (int)b.dtype, s, out.numel, scalarToDouble(aScalar, 0.0), aScalar != nullptr);
  } else {
    int64_t sv = aScalar ? (scalarIsFloat(aScalar) ? (int64_t)scalarToDouble(aScalar, 0.0) : scalarToInt(aScalar, 0))
                         : 0;
    hipLaunchKernelGGL((selectKernel<int64_t>), dim3(gridFor(out.numel)), dim3(kSelThreads), 0, stream, out.data,
                       cond.data, aScalar ? nullptr : a.data, b.data, (int)out.dtype, (int)cond.dtype, dta,
                       (int)b.dtype, s, out.numel, sv, aScalar != nullptr);
  }
  AMD_LAUNCH_CHECK();
  return diopiSuccess;
}

static diopiError_t runCompare(diopiContextHandle_t ctx, diopiTensorHandle_t outH, diopiConstTensorHandle_t aH,
                               diopiConstTensorHandle_t bH, const diopiScalar_t* bScalar, int cmp, const char* name) {
  hipStream_t stream;
  AMD_TRY(getStream(ctx, &stream));
  TensorView out, a, b;
  AMD_TRY(getView(outH, &out, "out"));
  AMD_TRY(getView(aH, &a, "input"));
  AMD_CHECK(out.defined() && a.defined(), "%s: null tensor", name);
  AMD_CHECK(supportedDtype(out.dtype) && supportedDtype(a.dtype), "%s: unsupported dtype", name);
  if (!bScalar) {
    AMD_TRY(getView(bH, &b, "other"));
    AMD_CHECK(b.defined() && supportedDtype(b.dtype), "%s: null or unsupported other tensor", name);
  }
  if (out.numel == 0) return diopiSuccess;
  Strided4 s;
  clearStrided(&s, out);
  AMD_TRY(broadcastInto(out, a, s.st[1], "input"));
  if (!bScalar) AMD_TRY(broadcastInto(out, b, s.st[2], "other"));
  coalesce(&s, 0);
  // compare as floating point as soon as either side is; integers compare exactly as int64
  const bool asFloat = isFloatDtype(a.dtype) || (bScalar ? scalarIsFloat(bScalar) : isFloatDtype(b.dtype));
  const int dtb = bScalar ? (int)a.dtype : (int)b.dtype;
  // A scalar compared with a floating tensor is first rounded to the tensor's dtype, as ATen's type promotion has it
  // (a bfloat16 tensor holding bfloat16(0.1) is equal to the scalar 0.1).
  double sbFloat = scalarToDouble(bScalar, 0.0);
  if (bScalar) {
    if (a.dtype == diopi_dtype_bfloat16) sbFloat = static_cast<float>(static_cast<bf16_t>(static_cast<float>(sbFloat)));
    else if (a.dtype == diopi_dtype_float16) sbFloat = static_cast<float>(static_cast<half_t>(static_cast<float>(sbFloat)));
    else if (a.dtype == diopi_dtype_float32) sbFloat = static_cast<float>(sbFloat);
  }
  // dense, one floating dtype on the input side, a 1-byte output: 8 elements per lane
  {
    auto dense = [&](const TensorView& t) {
      if (!t.isContiguous() || t.ndim != out.ndim) return false;
      for (int d = 0; d < out.ndim; ++d)
        if (t.shape[d] != out.shape[d]) return false;
      return true;
    };
    const bool vecType = a.dtype == diopi_dtype_bfloat16 || a.dtype == diopi_dtype_float16 || a.dtype == diopi_dtype_float32;
    if (vecType && out.itemsize == 1 && out.numel % 8 == 0 && out.isContiguous() && (reinterpret_cast<uintptr_t>(out.data) & 7) == 0 &&
        dense(a) && a.aligned16() && (bScalar || (dense(b) && b.dtype == a.dtype && b.aligned16()))) {
      const int64_t nvec = out.numel / 8, blocks = ceilDiv(nvec, kSelThreads);
      AMD_CHECK(blocks <= 0x7fffffff, "%s: %ld elements exceed the grid limit", name, (long)out.numel);
      const dim3 grid((unsigned)blocks), block(kSelThreads);
      if (a.dtype == diopi_dtype_bfloat16)
        hipLaunchKernelGGL((compareVecKernel<bf16_t>), grid, block, 0, stream, out.ptr<uint8_t>(), a.ptr<bf16_t>(),
                           bScalar ? nullptr : b.ptr<bf16_t>(), nvec, cmp, (float)sbFloat);
      else if (a.dtype == diopi_dtype_float16)
        hipLaunchKernelGGL((compareVecKernel<half_t>), grid, block, 0, stream, out.ptr<uint8_t>(), a.ptr<half_t>(),
                           bScalar ? nullptr : b.ptr<half_t>(), nvec, cmp, (float)sbFloat);
      else
        hipLaunchKernelGGL((compareVecKernel<float>), grid, block, 0, stream, out.ptr<uint8_t>(), a.ptr<float>(),
                           bScalar ? nullptr : b.ptr<float>(), nvec, cmp, (float)sbFloat);
      AMD_LAUNCH_CHECK();
      return diopiSuccess;
    }
  }
  if (asFloat) {
    hipLaunchKernelGGL((compareKernel<double>), dim3(gridFor(out.numel)), dim3(kSelThreads), 0, stream, out.data,
                       a.data, bScalar ? nullptr : b.data, (int)out.dtype, (int)a.dtype, dtb, s, out.numel, cmp,
                       sbFloat, bScalar != nullptr);
  } else {
    hipLaunchKernelGGL((compareKernel<int64_t>), dim3(gridFor(out.numel)), dim3(kSelThreads), 0, stream, out.data,
                       a.data, bScalar ? nullptr : b.data, (int)out.dtype, (int)a.dtype, dtb, s, out.numel, cmp,
                       scalarToInt(bScalar, 0), bScalar != nullptr);
  }
  AMD_LAUNCH_CHECK();
  return diopiSuccess;
}

static diopiError_t runTriangle(diopiContextHandle_t ctx, diopiTensorHandle_t outH, diopiConstTensorHandle_t xH,
                                int64_t diagonal, bool lower, const char* name) {
  hipStream_t stream;
  AMD_TRY(getStream(ctx, &stream));
  TensorView out, x;
  AMD_TRY(getView(outH, &out, "out"));
  AMD_TRY(getView(xH, &x, "input"));
  AMD_CHECK(out.defined() && x.defined(), "%s: null tensor", name);
  AMD_CHECK(supportedDtype(out.dtype) && supportedDtype(x.dtype), "%s: unsupported dtype", name);
  AMD_CHECK(x.ndim >= 2 && x.ndim == out.ndim, "%s: needs matching tensors of rank >= 2, got %d and %d", name, x.ndim,
            out.ndim);
  for (int d = 0; d < x.ndim; ++d)
    AMD_CHECK(x.shape[d] == out.shape[d], "%s: shape mismatch at dim %d (%ld vs %ld)", name, d, (long)x.shape[d],
              (long)out.shape[d]);
  if (out.numel == 0) return diopiSuccess;
  Strided4 s;
  clearStrided(&s, out);
  for (int d = 0; d < x.ndim; ++d) s.st[1][d] = x.shape[d] == 1 ? 0 : x.stride[d];
  coalesce(&s, 2);
  {
    const int64_t cols = out.shape[out.ndim - 1], rows = out.shape[out.ndim - 2];
    if (x.dtype == out.dtype && (out.itemsize == 2 || out.itemsize == 4) && out.isContiguous() && x.isContiguous() && out.aligned16() &&
        x.aligned16() && cols % 8 == 0 && cols / 8 < ((int64_t)1 << 31)) {
      const int64_t nvec = out.numel / 8, blocks = ceilDiv(nvec, kSelThreads);
      AMD_CHECK(blocks <= 0x7fffffff, "%s: %ld elements exceed the grid limit", name, (long)out.numel);
      if (out.itemsize == 2)
        hipLaunchKernelGGL((triangleVecKernel<uint16_t>), dim3((unsigned)blocks), dim3(kSelThreads), 0, stream, out.ptr<uint16_t>(),
                           x.ptr<uint16_t>(), nvec, (int)(cols / 8), rows, diagonal, lower);
      else
        hipLaunchKernelGGL((triangleVecKernel<uint32_t>), dim3((unsigned)blocks), dim3(kSelThreads), 0, stream, out.ptr<uint32_t>(),
                           x.ptr<uint32_t>(), nvec, (int)(cols / 8), rows, diagonal, lower);
      AMD_LAUNCH_CHECK();
      return diopiSuccess;
    }
  }
  if (isFloatDtype(out.dtype))
    hipLaunchKernelGGL((triangleKernel<double>), dim3(gridFor(out.numel)), dim3(kSelThreads), 0, stream, out.data,
                       x.data, (int)out.dtype, (int)x.dtype, s, out.numel, diagonal, lower);
  else
    hipLaunchKernelGGL((triangleKernel<int64_t>), dim3(gridFor(out.numel)), dim3(kSelThreads), 0, stream, out.data,
                       x.data, (int)out.dtype, (int)x.dtype, s, out.numel, diagonal, lower);
  AMD_LAUNCH_CHECK();
  return diopiSuccess;
}

static diopiError_t runGather(diopiContextHandle_t ctx, diopiTensorHandle_t outH, diopiConstTensorHandle_t srcH,
                              int64_t dim, diopiConstTensorHandle_t indexH, bool select, const char* name) {
  hipStream_t stream;
  AMD_TRY(getStream(ctx, &stream));
  TensorView out, src, index;
  AMD_TRY(getView(outH, &out, "out"));
  AMD_TRY(getView(srcH, &src, "input"));
  AMD_TRY(getView(indexH, &index, "index"));
  AMD_CHECK(out.defined() && src.defined() && index.defined(), "%s: null tensor", name);
  AMD_CHECK(supportedDtype(out.dtype) && supportedDtype(src.dtype), "%s: unsupported dtype", name);
  AMD_CHECK(index.dtype == diopi_dtype_int64 || index.dtype == diopi_dtype_int32, "%s: index must be int32 or int64",
            name);
  // a 0-d source is treated as one element along dim 0, as aten does
  const int rank = src.ndim == 0 ? 1 : src.ndim;
  if (dim < 0) dim += rank;
  AMD_CHECK(dim >= 0 && dim < rank, "%s: dim out of range for rank %d", name, rank);
  TensorView s1 = src;
  if (src.ndim == 0) s1.ndim = 1, s1.shape[0] = 1, s1.stride[0] = 1;
  TensorView o1 = out;
  if (out.ndim == 0) o1.ndim = 1, o1.shape[0] = 1, o1.stride[0] = 1;
  AMD_CHECK(o1.ndim == rank, "%s: output rank %d does not match input rank %d", name, o1.ndim, rank);
  Strided4 s;
  clearStrided(&s, o1);
  if (select) {
    AMD_CHECK(index.ndim <= 1, "%s: index must be 0-d or 1-d", name);
    AMD_CHECK(o1.shape[dim] == index.numel, "%s: output extent %ld at dim %ld must equal index length %ld", name,
              (long)o1.shape[dim], (long)dim, (long)index.numel);
    for (int d = 0; d < rank; ++d) {
      if (d == dim) continue;
      AMD_CHECK(o1.shape[d] == s1.shape[d], "%s: shape mismatch at dim %d", name, d);
      s.st[1][d] = s1.shape[d] == 1 ? 0 : s1.stride[d];
    }
    s.st[2][dim] = index.ndim == 1 ? index.stride[0] : 0;
  } else {
    TensorView i1 = index;
    if (index.ndim == 0) i1.ndim = 1, i1.shape[0] = 1, i1.stride[0] = 1;
    AMD_CHECK(i1.ndim == rank, "%s: index rank %d does not match input rank %d", name, i1.ndim, rank);
    for (int d = 0; d < rank; ++d) {
      AMD_CHECK(o1.shape[d] == i1.shape[d], "%s: output and index shapes differ at dim %d", name, d);
      AMD_CHECK(d == dim || i1.shape[d] <= s1.shape[d], "%s: index extent exceeds input at dim %d", name, d);
      if (d != dim) s.st[1][d] = s1.stride[d];
      s.st[2][d] = i1.shape[d] == 1 ? 0 : i1.stride[d];
    }
  }
  if (out.numel == 0) return diopiSuccess;
  const int64_t dimStride = s1.stride[dim], dimSize = s1.shape[dim];
  // index_select on dense tensors of one dtype whose blocks behind `dim` are whole 16-byte vectors: block copies
  // ([32000, 4096] bf16, 8192 indices: 122 us one element per lane)
  if (select && src.dtype == out.dtype && src.isContiguous() && out.isContiguous() && src.aligned16() && out.aligned16() &&
      src.ndim == out.ndim) {
    int64_t outer = 1, inner = 1;
    for (int d = 0; d < (int)dim; ++d) outer *= s1.shape[d];
    for (int d = (int)dim + 1; d < rank; ++d) inner *= s1.shape[d];
    const int64_t blockBytes = inner * src.itemsize, blocks = outer * index.numel;
    if (blockBytes % 16 == 0 && blockBytes >= 256 && blocks < ((int64_t)1 << 31)) {
      const int64_t istr = index.ndim == 1 ? index.stride[0] : 0;
      if (index.dtype == diopi_dtype_int64)
        hipLaunchKernelGGL((selectRowsKernel<int64_t>), dim3((unsigned)blocks), dim3(256), 0, stream, out.ptr<u32x4>(),
                           src.ptr<u32x4>(), index.ptr<int64_t>(), istr, index.numel, dimSize, blockBytes / 16);
      else
        hipLaunchKernelGGL((selectRowsKernel<int32_t>), dim3((unsigned)blocks), dim3(256), 0, stream, out.ptr<u32x4>(),
                           src.ptr<u32x4>(), index.ptr<int32_t>(), istr, index.numel, dimSize, blockBytes / 16);
      AMD_LAUNCH_CHECK();
      return diopiSuccess;
    }
  }
  // no coalescing: `dim` has to stay a dim of its own for both operand tables
  if (isFloatDtype(out.dtype))
    hipLaunchKernelGGL((gatherKernel<double>), dim3(gridFor(out.numel)), dim3(kSelThreads), 0, stream, out.data,
                       src.data, index.data, (int)out.dtype, (int)src.dtype, (int)index.dtype, s, out.numel, dimStride,
                       dimSize);
  else
    hipLaunchKernelGGL((gatherKernel<int64_t>), dim3(gridFor(out.numel)), dim3(kSelThreads), 0, stream, out.data,
                       src.data, index.data, (int)out.dtype, (int)src.dtype, (int)index.dtype, s, out.numel, dimStride,
                       dimSize);
  AMD_LAUNCH_CHECK();
  return diopiSuccess;
}

}  // namespace amd

using namespace amd;

#define SEL_EXPORT extern "C" __attribute__((visibility("default")))

SEL_EXPORT diopiError_t diopiWhere(diopiContextHandle_t ctx, diopiTensorHandle_t out,
                                   diopiConstTensorHandle_t condition, diopiConstTensorHandle_t input,
                                   diopiConstTensorHandle_t other) {
  return runSelect(ctx, out, condition, input, nullptr, other, "diopiWhere");
}

// value is a 0-d (or broadcastable) device tensor: out = mask ? value : input
SEL_EXPORT diopiError_t diopiMaskedFill(diopiContextHandle_t ctx, diopiTensorHandle_t out,
                                        diopiConstTensorHandle_t input, diopiConstTensorHandle_t mask,
                                        diopiConstTensorHandle_t value) {
  return runSelect(ctx, out, mask, value, nullptr, input, "diopiMaskedFill");
}
SEL_EXPORT diopiError_t diopiMaskedFillInp(diopiContextHandle_t ctx, diopiTensorHandle_t input,
                                           diopiConstTensorHandle_t mask, diopiConstTensorHandle_t value) {
  return runSelect(ctx, input, mask, value, nullptr, input, "diopiMaskedFillInp");
}
SEL_EXPORT diopiError_t diopiMaskedFillScalar(diopiContextHandle_t ctx, diopiTensorHandle_t out,
                                              diopiConstTensorHandle_t input, diopiConstTensorHandle_t mask,
                                              const diopiScalar_t* value) {
  AMD_CHECK(value != nullptr, "diopiMaskedFillScalar: null scalar");
  return runSelect(ctx, out, mask, nullptr, value, input, "diopiMaskedFillScalar");
}
SEL_EXPORT diopiError_t diopiMaskedFillInpScalar(diopiContextHandle_t ctx, diopiTensorHandle_t input,
                                                 diopiConstTensorHandle_t mask, const diopiScalar_t* value) {
  AMD_CHECK(value != nullptr, "diopiMaskedFillInpScalar: null scalar");
  return runSelect(ctx, input, mask, nullptr, value, input, "diopiMaskedFillInpScalar");
}

SEL_EXPORT diopiError_t diopiTril(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input,
                                  int64_t diagonal) {
  return runTriangle(ctx, out, input, diagonal, true, "diopiTril");
}
SEL_EXPORT diopiError_t diopiTriu(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input,
                                  int64_t diagonal) {
  return runTriangle(ctx, out, input, diagonal, false, "diopiTriu");
}
SEL_EXPORT diopiError_t diopiTriuInp(diopiContextHandle_t ctx, diopiTensorHandle_t input, int64_t diagonal) {
  return runTriangle(ctx, input, input, diagonal, false, "diopiTriuInp");
}

SEL_EXPORT diopiError_t diopiArange(diopiContextHandle_t ctx, diopiTensorHandle_t outH, const diopiScalar_t* start,
                                    const diopiScalar_t* end, const diopiScalar_t* step) {
  hipStream_t stream;
  AMD_TRY(getStream(ctx, &stream));
  TensorView out;
  AMD_TRY(getView(outH, &out, "out"));
  AMD_CHECK(out.defined() && supportedDtype(out.dtype), "diopiArange: null or unsupported output");
  AMD_CHECK(start && end && step, "diopiArange: null scalar");
  AMD_CHECK(out.ndim <= 1, "diopiArange: output must be 1-d, got rank %d", out.ndim);
  const double st = scalarToDouble(step, 1.0), lo = scalarToDouble(start, 0.0), hi = scalarToDouble(end, 0.0);
  AMD_CHECK(st != 0.0 && (hi - lo) / st >= 0.0, "diopiArange: step %g does not lead from %g to %g", st, lo, hi);
  // the caller sized `out`; it may hold at most the ceil((end - start) / step) values of the range
  const int64_t count = (int64_t)ceil((hi - lo) / st);
  AMD_CHECK(out.numel <= count, "diopiArange: output has %ld elements, the range only %ld", (long)out.numel,
            (long)count);
  if (out.numel == 0) return diopiSuccess;
  const int64_t stride = out.ndim == 1 ? out.stride[0] : 1;
  const bool integral =
      !isFloatDtype(out.dtype) && !scalarIsFloat(start) && !scalarIsFloat(step);
  if (integral)
    hipLaunchKernelGGL((arangeKernel<int64_t>), dim3(gridFor(out.numel)), dim3(kSelThreads), 0, stream, out.data,
                       (int)out.dtype, stride, out.numel, scalarToInt(start, 0), scalarToInt(step, 1));
  else
    hipLaunchKernelGGL((arangeKernel<double>), dim3(gridFor(out.numel)), dim3(kSelThreads), 0, stream, out.data,
                       (int)out.dtype, stride, out.numel, lo, st);
  AMD_LAUNCH_CHECK();
  return diopiSuccess;
}

SEL_EXPORT diopiError_t diopiIndexSelect(diopiContextHandle_t ctx, diopiTensorHandle_t out,
                                         diopiConstTensorHandle_t input, int64_t dim,
                                         diopiConstTensorHandle_t index) {
  return runGather(ctx, out, input, dim, index, true, "diopiIndexSelect");
}
SEL_EXPORT diopiError_t diopiGather(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input,
                                    int64_t dim, diopiConstTensorHandle_t index) {
  return runGather(ctx, out, input, dim, index, false, "diopiGather");
}

#define SEL_COMPARE(Name, OP)                                                                                       \
  SEL_EXPORT diopiError_t diopi##Name(diopiContextHandle_t ctx, diopiTensorHandle_t out,                            \
                                      diopiConstTensorHandle_t input, diopiConstTensorHandle_t other) {             \
    return runCompare(ctx, out, input, other, nullptr, OP, "diopi" #Name);                                          \
  }                                                                                                                 \
  SEL_EXPORT diopiError_t diopi##Name##Scalar(diopiContextHandle_t ctx, diopiTensorHandle_t out,                    \
                                              diopiConstTensorHandle_t input, const diopiScalar_t* other) {         \
    AMD_CHECK(other != nullptr, "diopi" #Name "Scalar: null scalar");                                               \
    return runCompare(ctx, out, input, nullptr, other, OP, "diopi" #Name "Scalar");                                 \
  }
SEL_COMPARE(Eq, kEq)
SEL_COMPARE(Ne, kNe)
SEL_COMPARE(Lt, kLt)
SEL_COMPARE(Le, kLe)
SEL_COMPARE(Gt, kGt)
SEL_COMPARE(Ge, kGe)
#undef SEL_COMPARE
