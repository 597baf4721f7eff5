// diopiRotaryEmbedding, diopiDestIndexCopyKV and diopiIndexPutInp for gfx950.
//
// Rotary: x viewed as [tokens, heads, d]; each lane rotates 8 (bf16/fp16) or 4 (fp32)
// pairs: one 16-byte load from each half of the head row (half-split layout) or one
// 16-byte load of adjacent pairs (interleaved layout), one cos and one sin vector that
// all heads of the token share (served by L2 after the first head), fp32 math, 16-byte
// stores. Algorithmic traffic = 2 * |x| + |cos| + |sin|.
//   half-split : dicp/dicp/vendor/AscendGraph/ext_ops.py:24-33
//   interleaved: dicp/test/model/llama/model.py:58-69 (complex multiply by cos + i sin)
//
// DestIndexCopyKV: out[dest_loc[i], :, :] = k[i, :, :], a pure byte move done with the
// widest vector the row size and pointers allow; one workgroup per token row.
#include "gemm.hpp"

namespace amd {

// ------------------------------------------------------------------ rotary ---
constexpr int kRotaryTokensPerLane = 1;

template <typename CT, int K>
__device__ __forceinline__ void loadAngles(const CT* __restrict__ p, bool vec, float (&f)[K]) {
  constexpr int BYTES = K * (int)sizeof(CT);
  CT tmp[K];
  if (vec && BYTES % 16 == 0) {
#pragma unroll
    for (int i = 0; i < BYTES / 16; ++i) reinterpret_cast<u32x4*>(tmp)[i] = reinterpret_cast<const u32x4*>(p)[i];
  } else if (vec && BYTES == 8) {
    *reinterpret_cast<u32x2*>(tmp) = *reinterpret_cast<const u32x2*>(p);
  } else {
#pragma unroll
    for (int k = 0; k < K; ++k) tmp[k] = p[k];
  }
#pragma unroll
  for (int k = 0; k < K; ++k) f[k] = static_cast<float>(tmp[k]);
}

// The vector form, laid out by token: a workgroup takes tokPerWg whole tokens (one when a token has 256 work items or
// more, e.g. 32 heads x 128), so a lane finds its (token, head, piece) with 32-bit arithmetic on small numbers, a
// token's table row is shared by the lanes next to each other, and the table entries of a lane are one vector load.
// x is loaded non-temporally like the other streaming kernels' operands: at [8192, 32, 128] bf16 that moved the
// cold figure from 24.1 to 23.1 us and the hot one (x resident in the memory-side cache) from 20.1 to 21.8. Two
// tokens per lane with all loads issued first: 25.0 us cold, not kept.
template <typename T, typename CT, bool INTERLEAVED>
__global__ __launch_bounds__(256) void rotaryTokenKernel(T* __restrict__ out, const T* __restrict__ x,
                                                          const CT* __restrict__ cosT, const CT* __restrict__ sinT,
                                                          int64_t tokens, int heads, int d, int64_t tableRows,
                                                          int tableCols, float sinSign, int64_t xTok, int64_t xHead,
                                                          int64_t oTok, int64_t oHead, int tokPerWg, bool tabVec) {
  using V = typename Vec16<T>::type;
  constexpr int N = Vec16<T>::N;
  constexpr int U = kRotaryTokensPerLane;  // tokens per lane, all their loads issued before the first is used
  constexpr int A = INTERLEAVED ? N / 2 : N;  // angles per work item
  const int half = d / 2;
  const int perHead = INTERLEAVED ? d / N : half / N;
  const int perTok = heads * perHead;
  int local = 0, first = threadIdx.x;
  if (tokPerWg > 1) {
    local = threadIdx.x / perTok, first = threadIdx.x - local * perTok;
    if (local >= tokPerWg) return;
  }
  const int64_t t0 = (int64_t)blockIdx.x * tokPerWg * U + local;
  const bool wide = INTERLEAVED && tableCols == d;  // full-width tables hold the pair's angle at 2 i
  for (int w = first; w < perTok; w += 256) {
    const int hh = w / perHead, j = w - hh * perHead;
    V a[U], b[U];
    float c[U][A], sn[U][A];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t t = t0 + (int64_t)u * tokPerWg;
      if (t >= tokens) continue;
      const T* xr = x + t * xTok + hh * xHead;
      const int64_t trow = (t % tableRows) * tableCols;
      a[u] = __builtin_nontemporal_load(reinterpret_cast<const V*>(xr + j * N));
      if constexpr (!INTERLEAVED) b[u] = __builtin_nontemporal_load(reinterpret_cast<const V*>(xr + half + j * N));
      if (wide) {
#pragma unroll
        for (int e = 0; e < A; ++e) {
          c[u][e] = static_cast<float>(cosT[trow + (j * A + e) * 2]);
          sn[u][e] = static_cast<float>(sinT[trow + (j * A + e) * 2]);
        }
      } else {
        loadAngles<CT, A>(cosT + trow + j * A, tabVec, c[u]);
        loadAngles<CT, A>(sinT + trow + j * A, tabVec, sn[u]);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t t = t0 + (int64_t)u * tokPerWg;
      if (t >= tokens) continue;
      T* outr = out + t * oTok + hh * oHead;
      if constexpr (!INTERLEAVED) {
        V oa, ob;
#pragma unroll
        for (int e = 0; e < N; ++e) {
          const float sg = sn[u][e] * sinSign;
          const float x0 = static_cast<float>(a[u][e]), x1 = static_cast<float>(b[u][e]);
          oa[e] = static_cast<T>(x0 * c[u][e] - x1 * sg);
          ob[e] = static_cast<T>(x0 * sg + x1 * c[u][e]);
        }
        __builtin_nontemporal_store(oa, reinterpret_cast<V*>(outr + j * N));
        __builtin_nontemporal_store(ob, reinterpret_cast<V*>(outr + half + j * N));
      } else {
        V o;
#pragma unroll
        for (int e = 0; e < N / 2; ++e) {
          const float sg = sn[u][e] * sinSign;
          const float x0 = static_cast<float>(a[u][2 * e]), x1 = static_cast<float>(a[u][2 * e + 1]);
          o[2 * e] = static_cast<T>(x0 * c[u][e] - x1 * sg);
          o[2 * e + 1] = static_cast<T>(x0 * sg + x1 * c[u][e]);
        }
        __builtin_nontemporal_store(o, reinterpret_cast<V*>(outr + j * N));
      }
    }
  }
}

template <typename T, typename CT>
__global__ __launch_bounds__(256) void rotaryScalarKernel(T* out, const T* x, const CT* cosT, const CT* sinT,
                                                           int64_t tokens, int heads, int d, int64_t tableRows,
                                                           int tableCols, float sinSign, bool interleaved, int64_t xTok,
                                                           int64_t xHead, int64_t oTok, int64_t oHead) {
  const int half = d / 2;
  const int64_t total = tokens * heads * half;
  for (int64_t w = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; w < total; w += (int64_t)gridDim.x * blockDim.x) {
    const int p = (int)(w % half);
    const int64_t th = w / half;
    const int64_t t = th / heads, hh = th - t * heads;
    const int64_t trow = t % tableRows;
    const T* xr = x + t * xTok + hh * xHead;
    T* outr = out + t * oTok + hh * oHead;
    const int i0 = interleaved ? 2 * p : p, i1 = interleaved ? 2 * p + 1 : p + half;
    const int tc = (interleaved && tableCols == d) ? 2 * p : p;
    float c = static_cast<float>(cosT[trow * tableCols + tc]);
    float s = static_cast<float>(sinT[trow * tableCols + tc]) * sinSign;
    float x0 = static_cast<float>(xr[i0]), x1 = static_cast<float>(xr[i1]);
    outr[i0] = static_cast<T>(x0 * c - x1 * s);
    outr[i1] = static_cast<T>(x0 * s + x1 * c);
  }
}

template <typename T, typename CT>
static diopiError_t launchRotary(hipStream_t stream, const TensorView& out, const TensorView& x, const TensorView& c,
                                 const TensorView& s, int64_t tokens, int heads, int d, int64_t tableRows,
                                 int tableCols, bool conj, bool interleaved, int64_t xTok, int64_t xHead, int64_t oTok,
                                 int64_t oHead) {
  constexpr int N = Vec16<T>::N;
  const float sign = conj ? -1.f : 1.f;
  const int half = d / 2;
  if (tokens == 0 || heads == 0 || d == 0) return diopiSuccess;
  bool vec = x.aligned16() && out.aligned16() && (interleaved ? d % N == 0 : half % N == 0) && xTok % N == 0 &&
             xHead % N == 0 && oTok % N == 0 && oHead % N == 0 && (int64_t)heads * d < ((int64_t)1 << 24) &&
             tokens < ((int64_t)1 << 31);
  if (vec) {
    const int perHead = interleaved ? d / N : half / N;
    const int64_t perTok = (int64_t)heads * perHead;
    const int tokPerWg = perTok >= 256 ? 1 : (int)(256 / perTok);
    const int64_t blocks = ceilDiv(tokens, (int64_t)tokPerWg * kRotaryTokensPerLane);
    // table entries of a lane as one vector: N (half-split) or N / 2 (interleaved, half-width tables) entries
    const int entries = interleaved ? N / 2 : N, align = entries * (int)sizeof(CT) >= 16 ? 16 : 8;
    const bool tabVec = (reinterpret_cast<uintptr_t>(c.data) % align) == 0 && (reinterpret_cast<uintptr_t>(s.data) % align) == 0 &&
                        ((int64_t)tableCols * (int64_t)sizeof(CT)) % align == 0;
    if (interleaved) {
      hipLaunchKernelGGL((rotaryTokenKernel<T, CT, true>), dim3((unsigned)blocks), dim3(256), 0, stream, out.ptr<T>(), x.ptr<T>(),
                         c.ptr<CT>(), s.ptr<CT>(), tokens, heads, d, tableRows, tableCols, sign, xTok, xHead, oTok, oHead, tokPerWg, tabVec);
    } else {
      hipLaunchKernelGGL((rotaryTokenKernel<T, CT, false>), dim3((unsigned)blocks), dim3(256), 0, stream, out.ptr<T>(), x.ptr<T>(),
                         c.ptr<CT>(), s.ptr<CT>(), tokens, heads, d, tableRows, tableCols, sign, xTok, xHead, oTok, oHead, tokPerWg, tabVec);
    }
  } else {
    int64_t total = tokens * heads * half;
    int64_t blocks = ceilDiv(total, 256);
    if (blocks > (1 << 20)) blocks = 1 << 20;
    hipLaunchKernelGGL((rotaryScalarKernel<T, CT>), dim3((unsigned)blocks), dim3(256), 0, stream, out.ptr<T>(),
                       x.ptr<T>(), c.ptr<CT>(), s.ptr<CT>(), tokens, heads, d, tableRows, tableCols, sign,
                       interleaved, xTok, xHead, oTok, oHead);
  }
  AMD_LAUNCH_CHECK();
  return diopiSuccess;
}

// ---------------------------------------------------------------- KV scatter --
// One workgroup per (token, pool): grid.y walks the pools of a call, so the K and the V row of a new token go out in
// one launch (the op is all launch latency: 64 rows of 8 KiB).
struct KvScatterPool {
  void* out;
  const void* src;
  int64_t outRowStrideVecs, srcRowStrideVecs, slots;
};
struct KvScatterArgs {
  KvScatterPool pool[2];
  const void* destLoc;
  int64_t tokens, rowVecs;
};

template <typename VEC, typename IDX>
__global__ __launch_bounds__(256) void destIndexCopyKernel(KvScatterArgs a) {
  const int64_t t = blockIdx.x;
  if (t >= a.tokens) return;
  const KvScatterPool& p = a.pool[blockIdx.y];
  int64_t slot = static_cast<int64_t>(static_cast<const IDX*>(a.destLoc)[t]);
  if (slot < 0) slot += p.slots;             // python-style negative index
  if (slot < 0 || slot >= p.slots) return;   // an out-of-range slot is dropped, never written
  const VEC* s = static_cast<const VEC*>(p.src) + t * p.srcRowStrideVecs;
  VEC* o = static_cast<VEC*>(p.out) + slot * p.outRowStrideVecs;
  for (int64_t i = threadIdx.x; i < a.rowVecs; i += blockDim.x) o[i] = s[i];
}

// Strides in `a` arrive in bytes and are scaled here to the widest vector every pointer, row length and stride allows.
template <typename IDX>
static diopiError_t launchDestCopy(hipStream_t stream, KvScatterArgs a, int pools, int64_t rowBytes) {
  uintptr_t bits = (uintptr_t)rowBytes;
  for (int i = 0; i < pools; ++i)
    bits |= reinterpret_cast<uintptr_t>(a.pool[i].out) | reinterpret_cast<uintptr_t>(a.pool[i].src) |
            (uintptr_t)a.pool[i].outRowStrideVecs | (uintptr_t)a.pool[i].srcRowStrideVecs;
#define KV_LAUNCH(VEC)                                                                                                   \
  do {                                                                                                                   \
    a.rowVecs = rowBytes / (int64_t)sizeof(VEC);                                                                         \
    for (int i = 0; i < pools; ++i)                                                                                      \
      a.pool[i].outRowStrideVecs /= (int64_t)sizeof(VEC), a.pool[i].srcRowStrideVecs /= (int64_t)sizeof(VEC);            \
    hipLaunchKernelGGL((destIndexCopyKernel<VEC, IDX>), dim3((unsigned)a.tokens, (unsigned)pools), dim3(256), 0, stream, a); \
  } while (0)
  if ((bits & 15) == 0) KV_LAUNCH(u32x4);
  else if ((bits & 7) == 0) KV_LAUNCH(u32x2);
  else if ((bits & 3) == 0) KV_LAUNCH(uint32_t);
  else if ((bits & 1) == 0) KV_LAUNCH(uint16_t);
  else KV_LAUNCH(uint8_t);
#undef KV_LAUNCH
  AMD_LAUNCH_CHECK();
  return diopiSuccess;
}

// ---------------------------------------------------------------- index_put --
// input[i0[r], i1[r], ..., :] (=|+=) values[r, :]; rows of `inner` elements.
struct IndexTables {  // passed by value as a kernel argument
  const void* ptrs[kMaxDims];
  int64_t sizes[kMaxDims];
  int64_t strides[kMaxDims];
};

// *addr += v for a 16-bit float: compare-and-swap on the aligned 32-bit word that holds it (the sum is rounded to
// the element type after every addition, as a 16-bit accumulate does).
template <typename T>
__device__ __forceinline__ void atomicAdd16(T* addr, float v) {
  const uintptr_t a = reinterpret_cast<uintptr_t>(addr);
  unsigned* word = reinterpret_cast<unsigned*>(a & ~uintptr_t(3));
  const int shift = (int)(a & 2) * 8;
  unsigned old = *word, assumed;
  do {
    assumed = old;
    const unsigned short curBits = (unsigned short)(assumed >> shift);
    const T next = static_cast<T>(static_cast<float>(__builtin_bit_cast(T, curBits)) + v);
    const unsigned repl = (assumed & ~(0xffffu << shift)) | ((unsigned)__builtin_bit_cast(unsigned short, next) << shift);
    old = atomicCAS(word, assumed, repl);
  } while (old != assumed);
}

template <typename IDX>
__global__ __launch_bounds__(256) void indexPutKernel(void* input, const void* values, int dtIn, int dtVal,
                                                       IndexTables tab, int nIdx, int64_t rows, int64_t inner,
                                                       int64_t valRowStride, bool accumulate) {
  const int64_t total = rows * inner;
  for (int64_t w = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; w < total; w += (int64_t)gridDim.x * blockDim.x) {
    int64_t r = w / inner, c = w - r * inner;
    int64_t off = 0;
    bool ok = true;
    for (int k = 0; k < nIdx; ++k) {
      int64_t v = static_cast<int64_t>(reinterpret_cast<const IDX*>(tab.ptrs[k])[r]);
      if (v < 0) v += tab.sizes[k];
      ok = ok && v >= 0 && v < tab.sizes[k];
      off += v * tab.strides[k];
    }
    if (!ok) continue;
    off += c;
    if (!accumulate) {
      if (isFloatDtypeDev(dtIn)) storeAs<double>(input, off, dtIn, loadAs<double>(values, r * valRowStride + c, dtVal));
      else storeAs<int64_t>(input, off, dtIn, loadAs<int64_t>(values, r * valRowStride + c, dtVal));
    } else {
      if (dtIn == diopi_dtype_float32) {
        atomicAdd(reinterpret_cast<float*>(input) + off, loadAs<float>(values, r * valRowStride + c, dtVal));
      } else if (dtIn == diopi_dtype_int32) {
        atomicAdd(reinterpret_cast<int*>(input) + off, (int)loadAs<int64_t>(values, r * valRowStride + c, dtVal));
      } else if (dtIn == diopi_dtype_int64) {
        atomicAdd(reinterpret_cast<unsigned long long*>(input) + off,
                  (unsigned long long)loadAs<int64_t>(values, r * valRowStride + c, dtVal));
      } else if (dtIn == diopi_dtype_float64) {
        atomicAdd(reinterpret_cast<double*>(input) + off, loadAs<double>(values, r * valRowStride + c, dtVal));
      } else if (dtIn == diopi_dtype_bfloat16) {
        atomicAdd16(reinterpret_cast<bf16_t*>(input) + off, loadAs<float>(values, r * valRowStride + c, dtVal));
      } else if (dtIn == diopi_dtype_float16) {
        atomicAdd16(reinterpret_cast<half_t*>(input) + off, loadAs<float>(values, r * valRowStride + c, dtVal));
      }
    }
  }
}

}  // namespace amd

using namespace amd;

extern "C" __attribute__((visibility("default"))) diopiError_t diopiRotaryEmbedding(
    diopiContextHandle_t ctx, diopiTensorHandle_t outH, diopiConstTensorHandle_t xH, diopiConstTensorHandle_t cosH,
    diopiConstTensorHandle_t sinH, bool conj, bool interleaved) {
  hipStream_t stream;
  AMD_TRY(getStream(ctx, &stream));
  TensorView out, x, c, s;
  AMD_TRY(getView(outH, &out, "out"));
  AMD_TRY(getView(xH, &x, "x"));
  AMD_TRY(getView(cosH, &c, "cos"));
  AMD_TRY(getView(sinH, &s, "sin"));
  return amd::runRotary(ctx, stream, out, x, c, s, conj, interleaved);
}

// The body of diopiRotaryEmbedding on views (also the second pass of diopiLinearRotary's two-pass form).
diopiError_t amd::runRotary(diopiContextHandle_t ctx, hipStream_t stream, const TensorView& out, const TensorView& x,
                            const TensorView& c, const TensorView& s, bool conj, bool interleaved) {
  AMD_CHECK(out.defined() && x.defined() && c.defined() && s.defined(), "diopiRotaryEmbedding: null tensor");
  AMD_CHECK(x.ndim >= 2, "diopiRotaryEmbedding: x must be [..., heads, head_dim]");
  AMD_CHECK(out.dtype == x.dtype && out.ndim == x.ndim, "diopiRotaryEmbedding: out must match x");
  for (int d = 0; d < x.ndim; ++d) AMD_CHECK(out.shape[d] == x.shape[d], "diopiRotaryEmbedding: shape mismatch at dim %d", d);
  AMD_CHECK(c.dtype == s.dtype && c.numel == s.numel, "diopiRotaryEmbedding: cos and sin differ in dtype or size");
  if (x.numel == 0) return diopiSuccess;
  const int d = (int)x.shape[x.ndim - 1];
  const int heads = (int)x.shape[x.ndim - 2];
  AMD_CHECK(d % 2 == 0, "diopiRotaryEmbedding: head_dim %d is odd", d);
  const int64_t tokens = x.numel / ((int64_t)heads * d);
  AMD_CHECK(c.ndim >= 1, "diopiRotaryEmbedding: cos must have a last dim of head_dim or head_dim/2");
  const int tableCols = (int)c.shape[c.ndim - 1];
  AMD_CHECK(tableCols == d || tableCols == d / 2, "diopiRotaryEmbedding: cos last dim %d is neither %d nor %d", tableCols,
            d, d / 2);
  const int64_t tableRows = c.numel / tableCols;
  AMD_CHECK(tableRows > 0 && tokens % tableRows == 0,
            "diopiRotaryEmbedding: %ld table rows do not divide %ld tokens", (long)tableRows, (long)tokens);
  // x / out are addressed as [tokens, heads, d] with a token stride and a head stride, so the
  // q and k slices of a fused QKV projection are rotated in place without a dense copy
  auto tokenView = [&](const TensorView& t, int64_t* tokStride, int64_t* headStride) {
    if (!(t.stride[t.ndim - 1] == 1 || d == 1)) return false;
    *headStride = heads == 1 ? d : t.stride[t.ndim - 2];
    int64_t n = 1, st = 0;
    bool have = false;
    for (int i = t.ndim - 3; i >= 0; --i) {
      if (t.shape[i] == 1) continue;
      if (!have) st = t.stride[i], have = true;
      else if (t.stride[i] != st * n) return false;
      n *= t.shape[i];
    }
    *tokStride = have ? st : (int64_t)heads * d;
    return true;
  };
  TensorView cx = x, cc, cs;
  int64_t xTok, xHead, oTok, oHead;
  if (!tokenView(x, &xTok, &xHead)) {
    AMD_TRY(makeContiguous(ctx, stream, x, &cx));
    xTok = (int64_t)heads * d, xHead = d;
  }
  AMD_TRY(makeContiguous(ctx, stream, c, &cc));
  AMD_TRY(makeContiguous(ctx, stream, s, &cs));
  TensorView cout = out;
  bool outTemp = !tokenView(out, &oTok, &oHead);
  if (outTemp) {
    diopiTensorHandle_t th;
    AMD_TRY(requireTensor(ctx, out.shape, out.ndim, out.dtype, &th, &cout));
    oTok = (int64_t)heads * d, oHead = d;
  }
  diopiError_t err;
#define ROTARY(T, CT) \
  err = launchRotary<T, CT>(stream, cout, cx, cc, cs, tokens, heads, d, tableRows, tableCols, conj, interleaved, xTok, xHead, oTok, oHead)
  if (x.dtype == diopi_dtype_bfloat16 && c.dtype == diopi_dtype_bfloat16) ROTARY(bf16_t, bf16_t);
  else if (x.dtype == diopi_dtype_bfloat16 && c.dtype == diopi_dtype_float32) ROTARY(bf16_t, float);
  else if (x.dtype == diopi_dtype_float16 && c.dtype == diopi_dtype_float16) ROTARY(half_t, half_t);
  else if (x.dtype == diopi_dtype_float16 && c.dtype == diopi_dtype_float32) ROTARY(half_t, float);
  else if (x.dtype == diopi_dtype_float32 && c.dtype == diopi_dtype_float32) ROTARY(float, float);
  else {
    setLastError("diopiRotaryEmbedding: unsupported dtypes x=%s cos=%s", dtypeName(x.dtype), dtypeName(c.dtype));
    return diopiErrorOccurred;
  }
#undef ROTARY
  AMD_TRY(err);
  if (outTemp) AMD_TRY(stridedCopy(stream, cout, out));
  return diopiSuccess;
}

// Checks one (pool, new rows) pair of the scatter and fills its part of the launch arguments (strides in bytes).
static diopiError_t kvScatterPool(diopiContextHandle_t ctx, hipStream_t stream, const char* what, const TensorView& out, const TensorView& k,
                                  int64_t tokens, KvScatterPool* pool, int64_t* rowBytes) {
  AMD_CHECK(out.defined() && k.defined(), "%s: null tensor", what);
  AMD_CHECK(out.dtype == k.dtype, "%s: out dtype %s differs from k dtype %s", what, dtypeName(out.dtype), dtypeName(k.dtype));
  AMD_CHECK(out.ndim == k.ndim && k.ndim >= 1, "%s: rank mismatch", what);
  for (int d = 1; d < k.ndim; ++d) AMD_CHECK(out.shape[d] == k.shape[d], "%s: trailing extent mismatch at dim %d", what, d);
  AMD_CHECK(k.shape[0] == tokens, "%s: dest_loc has %ld entries for %ld tokens", what, (long)tokens, (long)k.shape[0]);
  if (tokens == 0 || k.numel == 0) {
    *rowBytes = 0;
    return diopiSuccess;
  }
  AMD_CHECK(out.shape[0] > 0, "%s: empty destination pool", what);
  // rows (everything after dim 0) must be dense in both tensors; dim 0 may be strided
  TensorView rowK = k, rowO = out;
  rowK.shape[0] = rowO.shape[0] = 1;
  TensorView ck = k;
  if (!rowK.isContiguous()) AMD_TRY(makeContiguous(ctx, stream, k, &ck));
  AMD_CHECK(rowO.isContiguous(), "%s: rows of the destination pool must be dense", what);
  const int64_t rowElems = k.numel / tokens;
  *rowBytes = rowElems * k.itemsize;
  pool->out = out.data, pool->src = ck.data, pool->slots = out.shape[0];
  pool->srcRowStrideVecs = (tokens > 1 ? ck.stride[0] : rowElems) * k.itemsize;
  pool->outRowStrideVecs = (out.shape[0] > 1 ? out.stride[0] : rowElems) * out.itemsize;
  return diopiSuccess;
}

extern "C" __attribute__((visibility("default"))) diopiError_t diopiDestIndexCopyKV(diopiContextHandle_t ctx,
                                                                                    diopiTensorHandle_t outH,
                                                                                    diopiConstTensorHandle_t kH,
                                                                                    diopiConstTensorHandle_t locH) {
  hipStream_t stream;
  AMD_TRY(getStream(ctx, &stream));
  TensorView out, k, loc;
  AMD_TRY(getView(outH, &out, "out"));
  AMD_TRY(getView(kH, &k, "k"));
  AMD_TRY(getView(locH, &loc, "dest_loc"));
  AMD_CHECK(loc.defined(), "diopiDestIndexCopyKV: null tensor");
  AMD_CHECK(loc.dtype == diopi_dtype_int32 || loc.dtype == diopi_dtype_int64,
            "diopiDestIndexCopyKV: dest_loc must be int32 or int64, got %s", dtypeName(loc.dtype));
  KvScatterArgs a;
  int64_t rowBytes = 0;
  a.tokens = loc.numel;
  AMD_TRY(kvScatterPool(ctx, stream, "diopiDestIndexCopyKV", out, k, a.tokens, &a.pool[0], &rowBytes));
  if (rowBytes == 0) return diopiSuccess;
  a.pool[1] = a.pool[0];
  TensorView cloc;
  AMD_TRY(makeContiguous(ctx, stream, loc, &cloc));
  a.destLoc = cloc.data;
  return loc.dtype == diopi_dtype_int32 ? launchDestCopy<int32_t>(stream, a, 1, rowBytes) : launchDestCopy<int64_t>(stream, a, 1, rowBytes);
}

// The K and the V rows of the new tokens into their two pools in one launch (see functions_ext.h): the same result as two
// diopiDestIndexCopyKV calls with the same dest_loc.
extern "C" __attribute__((visibility("default"))) diopiError_t diopiDestIndexCopyKVPair(diopiContextHandle_t ctx, diopiTensorHandle_t outKH,
                                                                                        diopiConstTensorHandle_t kH, diopiTensorHandle_t outVH,
                                                                                        diopiConstTensorHandle_t vH, diopiConstTensorHandle_t locH) {
  hipStream_t stream;
  AMD_TRY(getStream(ctx, &stream));
  TensorView outK, k, outV, v, loc;
  AMD_TRY(getView(outKH, &outK, "out_k"));
  AMD_TRY(getView(kH, &k, "k"));
  AMD_TRY(getView(outVH, &outV, "out_v"));
  AMD_TRY(getView(vH, &v, "v"));
  AMD_TRY(getView(locH, &loc, "dest_loc"));
  AMD_CHECK(loc.defined(), "diopiDestIndexCopyKVPair: null tensor");
  AMD_CHECK(loc.dtype == diopi_dtype_int32 || loc.dtype == diopi_dtype_int64,
            "diopiDestIndexCopyKVPair: dest_loc must be int32 or int64, got %s", dtypeName(loc.dtype));
  KvScatterArgs a;
  int64_t rowBytesK = 0, rowBytesV = 0;
  a.tokens = loc.numel;
  AMD_TRY(kvScatterPool(ctx, stream, "diopiDestIndexCopyKVPair (k)", outK, k, a.tokens, &a.pool[0], &rowBytesK));
  AMD_TRY(kvScatterPool(ctx, stream, "diopiDestIndexCopyKVPair (v)", outV, v, a.tokens, &a.pool[1], &rowBytesV));
  if (rowBytesK == 0 && rowBytesV == 0) return diopiSuccess;
  TensorView cloc;
  AMD_TRY(makeContiguous(ctx, stream, loc, &cloc));
  a.destLoc = cloc.data;
  const bool i32 = loc.dtype == diopi_dtype_int32;
  if (rowBytesK != rowBytesV) {  // rows of different length (or one side empty): one launch each
    KvScatterArgs one = a;
    if (rowBytesK) AMD_TRY(i32 ? launchDestCopy<int32_t>(stream, one, 1, rowBytesK) : launchDestCopy<int64_t>(stream, one, 1, rowBytesK));
    one.pool[0] = a.pool[1];
    if (rowBytesV) AMD_TRY(i32 ? launchDestCopy<int32_t>(stream, one, 1, rowBytesV) : launchDestCopy<int64_t>(stream, one, 1, rowBytesV));
    return diopiSuccess;
  }
  return i32 ? launchDestCopy<int32_t>(stream, a, 2, rowBytesK) : launchDestCopy<int64_t>(stream, a, 2, rowBytesK);
}

extern "C" __attribute__((visibility("default"))) diopiError_t diopiIndexPutInp(
    diopiContextHandle_t ctx, diopiTensorHandle_t inputH, diopiConstTensorHandle_t valuesH,
    diopiConstTensorHandle_t* indices, int64_t nIdx, bool accumulate) {
  hipStream_t stream;
  AMD_TRY(getStream(ctx, &stream));
  TensorView in, val;
  AMD_TRY(getView(inputH, &in, "input"));
  AMD_TRY(getView(valuesH, &val, "values"));
  AMD_CHECK(in.defined() && val.defined(), "diopiIndexPutInp: null tensor");
  AMD_CHECK(nIdx >= 1 && nIdx <= in.ndim, "diopiIndexPutInp: %ld index tensors for a rank-%d input", (long)nIdx, in.ndim);
  AMD_CHECK(in.isContiguous(), "diopiIndexPutInp: input must be dense");
  if (accumulate)
    AMD_CHECK(in.dtype == diopi_dtype_float32 || in.dtype == diopi_dtype_float64 || in.dtype == diopi_dtype_int32 ||
                  in.dtype == diopi_dtype_int64 || in.dtype == diopi_dtype_bfloat16 || in.dtype == diopi_dtype_float16,
              "diopiIndexPutInp: accumulate supports float16/bfloat16/float32/float64/int32/int64 inputs, got %s",
              dtypeName(in.dtype));
  TensorView idx[kMaxDims];
  int64_t rows = -1;
  diopiDtype_t idt = diopi_dtype_int64;
  for (int64_t i = 0; i < nIdx; ++i) {
    AMD_CHECK(indices[i] != nullptr, "diopiIndexPutInp: null (slice) indices are not supported");
    TensorView t;
    AMD_TRY(getView(indices[i], &t, "index"));
    AMD_CHECK(t.dtype == diopi_dtype_int64 || t.dtype == diopi_dtype_int32, "diopiIndexPutInp: index dtype %s",
              dtypeName(t.dtype));
    if (i == 0) idt = t.dtype;
    AMD_CHECK(t.dtype == idt, "diopiIndexPutInp: mixed index dtypes");
    if (rows < 0) rows = t.numel;
    AMD_CHECK(t.numel == rows, "diopiIndexPutInp: index tensors differ in length");
    AMD_TRY(makeContiguous(ctx, stream, t, &idx[i]));
  }
  if (rows == 0) return diopiSuccess;
  int64_t inner = 1;
  for (int d = (int)nIdx; d < in.ndim; ++d) inner *= in.shape[d];
  // values: [rows, inner...] or anything broadcastable to it
  TensorView cval;
  AMD_TRY(makeContiguous(ctx, stream, val, &cval));
  int64_t valRowStride;
  if (cval.numel == rows * inner) valRowStride = inner;
  else if (cval.numel == inner) valRowStride = 0;
  else if (cval.numel == 1) valRowStride = 0;
  else {
    setLastError("diopiIndexPutInp: values with %ld elements cannot fill %ld rows of %ld", (long)cval.numel, (long)rows,
                 (long)inner);
    return diopiErrorOccurred;
  }
  if (cval.numel == 1 && inner != 1) {
    // scalar value broadcast over whole rows: expand through the generic copy
    diopiTensorHandle_t th;
    TensorView expanded;
    int64_t shp[1] = {inner};
    AMD_TRY(requireTensor(ctx, shp, 1, val.dtype, &th, &expanded));
    TensorView one = cval;
    one.ndim = 1;
    one.shape[0] = 1;
    one.stride[0] = 0;
    AMD_TRY(stridedCopy(stream, one, expanded));
    cval = expanded;
  }
  // Whole rows of the leading dim replaced by rows of the same dtype (how a KV cache is written through index_put):
  // the byte mover of diopiDestIndexCopyKV, a workgroup per row with the widest vector the rows allow, instead of an
  // element per lane through a lossless carrier (8192 rows of 8 KiB: 94 -> 24 us). Negative indices wrap and rows out
  // of range are dropped, as in the generic form.
  if (!accumulate && nIdx == 1 && cval.dtype == in.dtype && valRowStride == inner && inner * in.itemsize >= 512 &&
      rows <= 0x7fffffff) {
    KvScatterArgs a;
    a.pool[0].out = in.data, a.pool[0].src = cval.data, a.pool[0].slots = in.shape[0];
    a.pool[0].outRowStrideVecs = in.stride[0] * in.itemsize, a.pool[0].srcRowStrideVecs = inner * in.itemsize;
    a.pool[1] = a.pool[0];
    a.destLoc = idx[0].data, a.tokens = rows;
    return idt == diopi_dtype_int64 ? launchDestCopy<int64_t>(stream, a, 1, inner * in.itemsize)
                                    : launchDestCopy<int32_t>(stream, a, 1, inner * in.itemsize);
  }
  IndexTables tab;
  for (int i = 0; i < kMaxDims; ++i) tab.ptrs[i] = nullptr, tab.sizes[i] = 1, tab.strides[i] = 0;
  for (int64_t i = 0; i < nIdx; ++i) {
    tab.ptrs[i] = idx[i].data;
    tab.sizes[i] = in.shape[i];
    tab.strides[i] = in.stride[i];
  }
  int64_t total = rows * inner;
  int64_t blocks = ceilDiv(total, 256);
  if (blocks > 65536) blocks = 65536;
  if (idt == diopi_dtype_int64) {
    hipLaunchKernelGGL(indexPutKernel<int64_t>, dim3((unsigned)blocks), dim3(256), 0, stream, in.data, cval.data,
                       (int)in.dtype, (int)cval.dtype, tab, (int)nIdx, rows, inner, valRowStride, accumulate);
  } else {
    hipLaunchKernelGGL(indexPutKernel<int32_t>, dim3((unsigned)blocks), dim3(256), 0, stream, in.data, cval.data,
                       (int)in.dtype, (int)cval.dtype, tab, (int)nIdx, rows, inner, valRowStride, accumulate);
  }
  AMD_LAUNCH_CHECK();
  return diopiSuccess;
}
