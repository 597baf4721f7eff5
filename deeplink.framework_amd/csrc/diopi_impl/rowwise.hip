// Row reductions for gfx950: diopiSoftmax, diopiRMSNorm, diopiMean.
//
// Fast path (rows along the last, dense dim; row length a multiple of the 16-byte vector
// and at most 64 lanes * 16 vectors): ONE WAVEFRONT PER ROW. Each lane keeps its slice of
// the row in registers (up to 16 x 16-byte vectors), the max / sum / sum-of-squares are
// wave64 butterfly reductions, and the row makes exactly one trip from and one trip to
// HBM: algorithmic traffic = 2 * rows * cols * itemsize (+ the weight vector once).
// No LDS, no barrier. Waves are persistent (16 per CU): each walks its rows with the
// next row's loads in flight while the current one is reduced, and keeps its slice of the
// RMSNorm weight in registers.
//
// Short rows (at most 32 vectors) share a wave, 2 to 8 rows at a time; rows longer than a wave's registers (up to 8192
// vectors) take a workgroup per row with the row packed in the threads' registers.
//
// Generic path: one workgroup per row, LDS-staged block reduction, rows of any length or alignment;
// softmax over a non-last dim walks the reduced dim with a stride (one lane per column).
//
// Semantics: softmax as at::softmax on CPU (dipu/torch_dipu/csrc_dipu/aten/ops/CustomFallbackFunctions.hpp:466-474);
// RMSNorm as dicp/dicp/vendor/AscendGraph/ext_ops.py:47-49 with fp32 accumulation
// (dicp/test/model/llama/model.py:34-39).
#include <algorithm>

#include "common.hpp"

namespace amd {

constexpr float kLog2e = 1.4426950408889634f;

// ------------------------------------------------------------ wave-per-row ---
enum RowOp { kRowSoftmax = 0, kRowRmsNorm = 1 };

template <typename T, int NV, int OP, typename WT>
__global__ __launch_bounds__(256) void rowWaveKernel(T* __restrict__ out, const T* __restrict__ in,
                                                      const WT* __restrict__ weight, const WT* __restrict__ bias,
                                                      float* __restrict__ invRmsOut, int64_t rows, int cols,
                                                      int64_t inRowStride, int64_t outRowStride, float eps) {
  using V = typename Vec16<T>::type;
  using WV = typename Vec16<WT>::type;
  constexpr int N = Vec16<T>::N;
  constexpr int WN = Vec16<WT>::N;
  const int lane = threadIdx.x & 63;
  const int nvec = cols / N;
  // Persistent waves: wave w handles rows w, w + W, w + 2W, ... and fetches the next row
  // while it reduces the current one, so every resident wave keeps loads in flight until
  // the last row (no tail of half-empty CUs).
  const int64_t nWaves = (int64_t)gridDim.x * 4;
  int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  // RMSNorm: the weight vector is staged once per workgroup in LDS (NV KiB) and read from there
  // for every row, which keeps it out of both the register file and the L1/L2 request stream.
  constexpr int WPER = (N + WN - 1) / WN;
  __shared__ WV wlds[OP == kRowRmsNorm ? 64 * NV * WPER : 1];
  // The first row's loads go out before the weights are staged, so the two latencies overlap.
  V pre[NV];
  if (row < rows) {
    const V* src = reinterpret_cast<const V*>(in + row * inRowStride);
#pragma unroll
    for (int i = 0; i < NV; ++i)
      if (lane + 64 * i < nvec) pre[i] = __builtin_nontemporal_load(src + lane + 64 * i);
  }
  if (OP == kRowRmsNorm && weight != nullptr) {
    for (int i = threadIdx.x; i < nvec * WPER; i += 256) wlds[i] = reinterpret_cast<const WV*>(weight)[i];
  }
  if (OP == kRowRmsNorm) __syncthreads();  // before the early exit below: every wave of the block arrives
  if (row >= rows) return;
  for (; row < rows; row += nWaves) {
  V* dst = reinterpret_cast<V*>(out + row * outRowStride);
  V cur[NV];
  if (OP == kRowRmsNorm) {
#pragma unroll
    for (int i = 0; i < NV; ++i) cur[i] = pre[i];
    if (row + nWaves < rows) {  // next row in flight while this one is reduced
      // (ordinary loads here, non-temporal ones for a wave's first row: measured on [8192, 4096] bf16, cold, 22.4 us
      // against 24.0 with both non-temporal and 24.2 with both ordinary)
      const V* src = reinterpret_cast<const V*>(in + (row + nWaves) * inRowStride);
#pragma unroll
      for (int i = 0; i < NV; ++i)
        if (lane + 64 * i < nvec) pre[i] = src[lane + 64 * i];
    }
  }

  if constexpr (OP == kRowSoftmax) {
    float f[NV][N];
    float m = -INFINITY;
#pragma unroll
    for (int i = 0; i < NV; ++i)
      if (lane + 64 * i < nvec) {
#pragma unroll
        for (int j = 0; j < N; ++j) {
          f[i][j] = static_cast<float>(pre[i][j]);
          m = fmaxf(m, f[i][j]);
        }
      }
    if (row + nWaves < rows) {  // next row in flight while this one is reduced (ordinary loads, as for RMSNorm: 22.7 -> 21.1 us cold)
      const V* src = reinterpret_cast<const V*>(in + (row + nWaves) * inRowStride);
#pragma unroll
      for (int i = 0; i < NV; ++i)
        if (lane + 64 * i < nvec) pre[i] = src[lane + 64 * i];
    }
    m = waveMax(m);
    const float mScaled = (m == -INFINITY) ? 0.f : m * kLog2e;  // all -inf row -> nan like the CPU kernel
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i)
      if (lane + 64 * i < nvec) {
#pragma unroll
        for (int j = 0; j < N; ++j) {
          f[i][j] = __builtin_amdgcn_exp2f(fmaf(f[i][j], kLog2e, -mScaled));
          s += f[i][j];
        }
      }
    s = waveSum(s);
    const float inv = 1.f / s;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      int idx = lane + 64 * i;
      if (idx < nvec) {
        V v;
#pragma unroll
        for (int j = 0; j < N; ++j) v[j] = static_cast<T>(f[i][j] * inv);
        __builtin_nontemporal_store(v, dst + idx);
      }
    }
  } else {
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i)
      if (lane + 64 * i < nvec) {
#pragma unroll
        for (int j = 0; j < N; ++j) {
          float x = static_cast<float>(cur[i][j]);
          ss += x * x;
        }
      }
    ss = waveSum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)cols + eps);
    if (invRmsOut != nullptr && lane == 0) invRmsOut[row] = inv;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      int idx = lane + 64 * i;
      if (idx < nvec) {
        V v;
        V xv = cur[i];
        asm volatile("" : "+v"(xv));  // re-convert from the packed row instead of keeping an fp32 copy alive
        // weight/bias vectors hold WN elements per 16 bytes; N elements of T need N/WN of them
        float w[N], b[N];
        if (weight != nullptr) {
#pragma unroll
          for (int p = 0; p < WPER; ++p) {
            WV wv = wlds[idx * WPER + p];
#pragma unroll
            for (int j = 0; j < WN && p * WN + j < N; ++j) w[p * WN + j] = static_cast<float>(wv[j]);
          }
        }
        if (bias != nullptr) {
          constexpr int PER = (N + WN - 1) / WN;
#pragma unroll
          for (int p = 0; p < PER; ++p) {
            WV bv = reinterpret_cast<const WV*>(bias)[idx * PER + p];
#pragma unroll
            for (int j = 0; j < WN && p * WN + j < N; ++j) b[p * WN + j] = static_cast<float>(bv[j]);
          }
        }
#pragma unroll
        for (int j = 0; j < N; ++j) {
          float r = static_cast<float>(xv[j]) * inv;
          if (weight != nullptr) r *= w[j];
          if (bias != nullptr) r += b[j];
          v[j] = static_cast<T>(r);
        }
        __builtin_nontemporal_store(v, dst + idx);
      }
    }
  }
  }  // persistent row loop
}

// ------------------------------------------------- several short rows per wave ---
// Rows of at most 32 vectors (256 elements of a 16-bit type): a wave-per-row kernel would leave most lanes without a
// vector. Here LPR lanes share a row, a wave takes 64 / LPR rows at a time, one vector per lane, and the reductions are
// butterflies within the LPR lanes. Four such row groups per iteration keep four loads per lane in flight.
template <int LPR>
__device__ __forceinline__ float groupReduce(float v, bool isMax) {
  // within a row of 16 lanes: permutations folded into the arithmetic (see waveSum); 32 lanes: one shuffle more
  auto step = [&](float other) { v = isMax ? fmaxf(v, other) : v + other; };
  step(lanePermuted<kDppQuadSwap1>(v));
  step(lanePermuted<kDppQuadSwap2>(v));
  step(lanePermuted<kDppHalfMirror>(v));
  if (LPR >= 16) step(lanePermuted<kDppMirror>(v));
  if (LPR >= 32) step(__shfl_xor(v, 16, 64));
  return v;
}

template <typename T, int LPR, int OP, typename WT>
__global__ __launch_bounds__(256) void rowSubWaveKernel(T* __restrict__ out, const T* __restrict__ in,
                                                         const WT* __restrict__ weight, const WT* __restrict__ bias,
                                                         float* __restrict__ invRmsOut, int64_t rows, int cols,
                                                         int64_t inRowStride, int64_t outRowStride, float eps) {
  using V = typename Vec16<T>::type;
  using WV = typename Vec16<WT>::type;
  constexpr int N = Vec16<T>::N, WN = Vec16<WT>::N, WPER = (N + WN - 1) / WN;
  constexpr int RPW = 64 / LPR, U = 4;
  const int lane = threadIdx.x & 63, sub = lane % LPR, r = lane / LPR;
  const bool active = sub < cols / N;
  float w[N], b[N];
#pragma unroll
  for (int j = 0; j < N; ++j) w[j] = 1.f, b[j] = 0.f;
  if (OP == kRowRmsNorm && active) {
#pragma unroll
    for (int p = 0; p < WPER; ++p) {
      if (weight != nullptr) {
        const WV wv = reinterpret_cast<const WV*>(weight)[sub * WPER + p];
#pragma unroll
        for (int j = 0; j < WN && p * WN + j < N; ++j) w[p * WN + j] = static_cast<float>(wv[j]);
      }
      if (bias != nullptr) {
        const WV bv = reinterpret_cast<const WV*>(bias)[sub * WPER + p];
#pragma unroll
        for (int j = 0; j < WN && p * WN + j < N; ++j) b[p * WN + j] = static_cast<float>(bv[j]);
      }
    }
  }
  const int64_t nWaves = (int64_t)gridDim.x * 4, step = nWaves * RPW * U;
  for (int64_t base = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * RPW * U; base < rows; base += step) {
    V x[U];
    bool ok[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t row = base + u * RPW + r;
      ok[u] = active && row < rows;
      if (ok[u]) x[u] = __builtin_nontemporal_load(reinterpret_cast<const V*>(in + row * inRowStride) + sub);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t row = base + u * RPW + r;
      float f[N];
      V v;
      if constexpr (OP == kRowSoftmax) {
        float m = -INFINITY;
#pragma unroll
        for (int j = 0; j < N; ++j) {
          f[j] = ok[u] ? static_cast<float>(x[u][j]) : -INFINITY;
          m = fmaxf(m, f[j]);
        }
        m = groupReduce<LPR>(m, true);
        const float mScaled = (m == -INFINITY) ? 0.f : m * kLog2e;  // all -inf row -> nan like the CPU kernel
        float sum = 0.f;
#pragma unroll
        for (int j = 0; j < N; ++j) {
          f[j] = ok[u] ? __builtin_amdgcn_exp2f(fmaf(f[j], kLog2e, -mScaled)) : 0.f;
          sum += f[j];
        }
        sum = groupReduce<LPR>(sum, false);
        const float inv = 1.f / sum;
#pragma unroll
        for (int j = 0; j < N; ++j) v[j] = static_cast<T>(f[j] * inv);
      } else {
        float ss = 0.f;
#pragma unroll
        for (int j = 0; j < N; ++j) {
          f[j] = ok[u] ? static_cast<float>(x[u][j]) : 0.f;
          ss += f[j] * f[j];
        }
        ss = groupReduce<LPR>(ss, false);
        const float inv = 1.0f / sqrtf(ss / (float)cols + eps);
        if (invRmsOut != nullptr && sub == 0 && row < rows) invRmsOut[row] = inv;
#pragma unroll
        for (int j = 0; j < N; ++j) {
          float t = f[j] * inv;
          if (weight != nullptr) t *= w[j];
          if (bias != nullptr) t += b[j];
          v[j] = static_cast<T>(t);
        }
      }
      if (ok[u]) __builtin_nontemporal_store(v, reinterpret_cast<V*>(out + row * outRowStride) + sub);
    }
  }
}

// --------------------------------------------------------- block-per-row ----
__device__ __forceinline__ float blockReduce(float v, bool isMax, float* smem) {
  v = isMax ? waveMax(v) : waveSum(v);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = blockDim.x >> 6;
  __syncthreads();
  if (lane == 0) smem[wave] = v;
  __syncthreads();
  float r = isMax ? -INFINITY : 0.f;
  for (int i = 0; i < nw; ++i) r = isMax ? fmaxf(r, smem[i]) : r + smem[i];
  return r;
}

// Rows of any length / alignment. The row is staged in LDS as fp32 when it fits
// (`stage` elements), otherwise re-read from global memory.
template <typename T, int OP, typename WT>
__global__ __launch_bounds__(256) void rowBlockKernel(T* out, const T* in, const WT* weight, const WT* bias,
                                                       float* invRmsOut, int64_t rows, int64_t cols,
                                                       int64_t inRowStride, int64_t outRowStride, float eps,
                                                       int stage) {
  extern __shared__ float lds[];
  float* red = lds;         // 4 floats for the cross-wave step
  float* rowBuf = lds + 8;  // `stage` floats
  const int64_t row = blockIdx.x;
  const T* src = in + row * inRowStride;
  T* dst = out + row * outRowStride;
  const bool staged = cols <= stage;
  if constexpr (OP == kRowSoftmax) {
    float m = -INFINITY;
    for (int64_t c = threadIdx.x; c < cols; c += blockDim.x) {
      float v = static_cast<float>(src[c]);
      if (staged) rowBuf[c] = v;
      m = fmaxf(m, v);
    }
    m = blockReduce(m, true, red);
    const float mScaled = (m == -INFINITY) ? 0.f : m * kLog2e;
    float s = 0.f;
    for (int64_t c = threadIdx.x; c < cols; c += blockDim.x) {
      float v = staged ? rowBuf[c] : static_cast<float>(src[c]);
      v = exp2f(v * kLog2e - mScaled);
      if (staged) rowBuf[c] = v;
      s += v;
    }
    s = blockReduce(s, false, red);
    const float inv = 1.f / s;
    for (int64_t c = threadIdx.x; c < cols; c += blockDim.x) {
      float v = staged ? rowBuf[c] : exp2f(static_cast<float>(src[c]) * kLog2e - mScaled);
      dst[c] = static_cast<T>(v * inv);
    }
  } else {
    float ss = 0.f;
    for (int64_t c = threadIdx.x; c < cols; c += blockDim.x) {
      float v = static_cast<float>(src[c]);
      if (staged) rowBuf[c] = v;
      ss += v * v;
    }
    ss = blockReduce(ss, false, red);
    const float inv = 1.0f / sqrtf(ss / (float)cols + eps);
    if (invRmsOut != nullptr && threadIdx.x == 0) invRmsOut[row] = inv;
    for (int64_t c = threadIdx.x; c < cols; c += blockDim.x) {
      float v = (staged ? rowBuf[c] : static_cast<float>(src[c])) * inv;
      if (weight != nullptr) v *= static_cast<float>(weight[c]);
      if (bias != nullptr) v += static_cast<float>(bias[c]);
      dst[c] = static_cast<T>(v);
    }
  }
}

// Rows too long for one wave's registers (more than 1024 vectors), 16-byte aligned: a workgroup per row, every thread
// keeps NVT vectors of the row packed in registers, so the row still makes one trip from and one trip to memory;
// the two reductions of a row go through LDS. Workgroups walk the rows with a stride.
template <typename T, int NVT, int OP, typename WT>
__global__ __launch_bounds__(256) void rowBlockVecKernel(T* __restrict__ out, const T* __restrict__ in,
                                                          const WT* __restrict__ weight, const WT* __restrict__ bias,
                                                          float* __restrict__ invRmsOut, int64_t rows, int cols,
                                                          int64_t inRowStride, int64_t outRowStride, float eps) {
  using V = typename Vec16<T>::type;
  using WV = typename Vec16<WT>::type;
  constexpr int N = Vec16<T>::N, WN = Vec16<WT>::N, WPER = (N + WN - 1) / WN;
  __shared__ float red[8];
  const int nvec = cols / N, tid = threadIdx.x;
  // RMSNorm: this thread's pieces of the weight stay in registers for all the rows of the workgroup when they fit
  // next to the row
  constexpr bool kEarly = OP == kRowRmsNorm && NVT * WPER <= 16;
  WV wEarly[kEarly ? NVT * WPER : 1];
  if constexpr (kEarly) {
    if (weight != nullptr) {
#pragma unroll
      for (int i = 0; i < NVT; ++i)
        if (tid + 256 * i < nvec) {
#pragma unroll
          for (int p = 0; p < WPER; ++p) wEarly[i * WPER + p] = reinterpret_cast<const WV*>(weight)[(tid + 256 * i) * WPER + p];
        }
    }
  }
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const V* src = reinterpret_cast<const V*>(in + row * inRowStride);
    V* dst = reinterpret_cast<V*>(out + row * outRowStride);
    V x[NVT];
#pragma unroll
    for (int i = 0; i < NVT; ++i)
      if (tid + 256 * i < nvec) x[i] = __builtin_nontemporal_load(src + tid + 256 * i);
    if constexpr (OP == kRowSoftmax) {
      float m = -INFINITY;
#pragma unroll
      for (int i = 0; i < NVT; ++i)
        if (tid + 256 * i < nvec) {
#pragma unroll
          for (int j = 0; j < N; ++j) m = fmaxf(m, static_cast<float>(x[i][j]));
        }
      m = blockReduce(m, true, red);
      const float mScaled = (m == -INFINITY) ? 0.f : m * kLog2e;
      float sum = 0.f;
#pragma unroll
      for (int i = 0; i < NVT; ++i)
        if (tid + 256 * i < nvec) {
#pragma unroll
          for (int j = 0; j < N; ++j) sum += __builtin_amdgcn_exp2f(fmaf(static_cast<float>(x[i][j]), kLog2e, -mScaled));
        }
      sum = blockReduce(sum, false, red);
      const float inv = 1.f / sum;
#pragma unroll
      for (int i = 0; i < NVT; ++i)
        if (tid + 256 * i < nvec) {
          V v;
#pragma unroll
          for (int j = 0; j < N; ++j)
            v[j] = static_cast<T>(__builtin_amdgcn_exp2f(fmaf(static_cast<float>(x[i][j]), kLog2e, -mScaled)) * inv);
          __builtin_nontemporal_store(v, dst + tid + 256 * i);
        }
    } else {
      float ss = 0.f;
#pragma unroll
      for (int i = 0; i < NVT; ++i)
        if (tid + 256 * i < nvec) {
#pragma unroll
          for (int j = 0; j < N; ++j) {
            const float f = static_cast<float>(x[i][j]);
            ss += f * f;
          }
        }
      ss = blockReduce(ss, false, red);
      const float inv = 1.0f / sqrtf(ss / (float)cols + eps);
      if (invRmsOut != nullptr && tid == 0) invRmsOut[row] = inv;
#pragma unroll
      for (int i = 0; i < NVT; ++i) {
        const int idx = tid + 256 * i;
        if (idx < nvec) {
          float w[N], b[N];
#pragma unroll
          for (int p = 0; p < WPER; ++p) {
            if (weight != nullptr) {
              WV wv;
              if constexpr (kEarly) wv = wEarly[i * WPER + p];
              else wv = reinterpret_cast<const WV*>(weight)[idx * WPER + p];
#pragma unroll
              for (int j = 0; j < WN && p * WN + j < N; ++j) w[p * WN + j] = static_cast<float>(wv[j]);
            }
            if (bias != nullptr) {
              const WV bv = reinterpret_cast<const WV*>(bias)[idx * WPER + p];
#pragma unroll
              for (int j = 0; j < WN && p * WN + j < N; ++j) b[p * WN + j] = static_cast<float>(bv[j]);
            }
          }
          V v;
#pragma unroll
          for (int j = 0; j < N; ++j) {
            float t = static_cast<float>(x[i][j]) * inv;
            if (weight != nullptr) t *= w[j];
            if (bias != nullptr) t += b[j];
            v[j] = static_cast<T>(t);
          }
          __builtin_nontemporal_store(v, dst + idx);
        }
      }
    }
  }
}

// Rows too long for a workgroup's registers (a softmax over a vocabulary of more than 65 536 entries), or long and not
// 16-byte aligned: a workgroup of 1024 threads per row streams the row twice, the second time mostly out of the caches
// the first pass filled. Pass one keeps a running maximum and a sum rescaled to it per thread (softmax) or the sum of
// squares (RMSNorm); pass two writes. VEC: 16-byte pieces (cols a multiple of the vector, aligned rows), else single
// elements.
template <typename T, int OP, typename WT, bool VEC>
__global__ __launch_bounds__(1024) void rowStreamKernel(T* __restrict__ out, const T* __restrict__ in,
                                                         const WT* __restrict__ weight, const WT* __restrict__ bias,
                                                         float* __restrict__ invRmsOut, int64_t rows, int64_t cols,
                                                         int64_t inRowStride, int64_t outRowStride, float eps) {
  using V = typename Vec16<T>::type;
  constexpr int N = VEC ? Vec16<T>::N : 1;
  __shared__ float red[16];
  const int64_t pieces = cols / N;
  auto load = [&](const T* src, int64_t i, float (&f)[N]) {
    if constexpr (VEC) {
      const V v = reinterpret_cast<const V*>(src)[i];
#pragma unroll
      for (int j = 0; j < N; ++j) f[j] = static_cast<float>(v[j]);
    } else {
      f[0] = static_cast<float>(src[i]);
    }
  };
  auto store = [&](T* dst, int64_t i, const float (&f)[N]) {
    if constexpr (VEC) {
      V v;
#pragma unroll
      for (int j = 0; j < N; ++j) v[j] = static_cast<T>(f[j]);
      __builtin_nontemporal_store(v, reinterpret_cast<V*>(dst) + i);
    } else {
      dst[i] = static_cast<T>(f[0]);
    }
  };
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const T* src = in + row * inRowStride;
    T* dst = out + row * outRowStride;
    if constexpr (OP == kRowSoftmax) {
      float m = -INFINITY, sum = 0.f;  // in units of log2
      for (int64_t i = threadIdx.x; i < pieces; i += 1024) {
        float f[N];
        load(src, i, f);
        float pm = f[0];
#pragma unroll
        for (int j = 1; j < N; ++j) pm = fmaxf(pm, f[j]);
        pm *= kLog2e;
        if (pm > m) {
          sum *= __builtin_amdgcn_exp2f(m - pm);  // (m = -inf: sum is still 0, and exp2(-inf) = 0)
          m = pm;
        }
        if (m != -INFINITY) {
#pragma unroll
          for (int j = 0; j < N; ++j) sum += __builtin_amdgcn_exp2f(fmaf(f[j], kLog2e, -m));
        }
      }
      const float rowMax = blockReduce(m, true, red);
      const float mScaled = (rowMax == -INFINITY) ? 0.f : rowMax;  // all -inf row: the sum is 0 and every output 0 * inf = nan, like the CPU kernel
      sum = (m == -INFINITY) ? 0.f : sum * __builtin_amdgcn_exp2f(m - mScaled);
      const float total = blockReduce(sum, false, red);
      const float inv = 1.f / total;
      for (int64_t i = threadIdx.x; i < pieces; i += 1024) {
        float f[N];
        load(src, i, f);
#pragma unroll
        for (int j = 0; j < N; ++j) f[j] = __builtin_amdgcn_exp2f(fmaf(f[j], kLog2e, -mScaled)) * inv;
        store(dst, i, f);
      }
    } else {
      float ss = 0.f;
      for (int64_t i = threadIdx.x; i < pieces; i += 1024) {
        float f[N];
        load(src, i, f);
#pragma unroll
        for (int j = 0; j < N; ++j) ss += f[j] * f[j];
      }
      ss = blockReduce(ss, false, red);
      const float inv = 1.0f / sqrtf(ss / (float)cols + eps);
      if (invRmsOut != nullptr && threadIdx.x == 0) invRmsOut[row] = inv;
      for (int64_t i = threadIdx.x; i < pieces; i += 1024) {
        float f[N];
        load(src, i, f);
#pragma unroll
        for (int j = 0; j < N; ++j) {
          float t = f[j] * inv;
          if (weight != nullptr) t *= static_cast<float>(weight[i * N + j]);
          if (bias != nullptr) t += static_cast<float>(bias[i * N + j]);
          f[j] = t;
        }
        store(dst, i, f);
      }
    }
  }
}

// softmax along a non-last dim of a dense tensor [outer, dim, inner]: one lane per
// (outer, inner) column, lanes adjacent along `inner` so every step is coalesced.
template <typename T>
__global__ __launch_bounds__(256) void softmaxStridedKernel(T* out, const T* in, int64_t outer, int64_t dim,
                                                             int64_t inner) {
  int64_t col = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (col >= outer * inner) return;
  int64_t o = col / inner, i = col - o * inner;
  const T* src = in + o * dim * inner + i;
  T* dst = out + o * dim * inner + i;
  float m = -INFINITY;
  for (int64_t d = 0; d < dim; ++d) m = fmaxf(m, static_cast<float>(src[d * inner]));
  const float mScaled = (m == -INFINITY) ? 0.f : m * kLog2e;
  float s = 0.f;
  for (int64_t d = 0; d < dim; ++d) s += exp2f(static_cast<float>(src[d * inner]) * kLog2e - mScaled);
  const float inv = 1.f / s;
  for (int64_t d = 0; d < dim; ++d)
    dst[d * inner] = static_cast<T>(exp2f(static_cast<float>(src[d * inner]) * kLog2e - mScaled) * inv);
}

// The same softmax for long columns: a workgroup of 1024 takes 32 adjacent `inner` positions of one outer index, its 32
// row lanes split the `dim` entries (each keeps an online (max, sum) over its share), the shares meet in LDS, and a
// second pass writes. One lane per column leaves a [8192, 4096] softmax over dim 0 with 4096 lanes in flight, each
// walking 8192 entries three times: 6.3 ms against 0.1 ms in this form.
template <typename T>
__global__ __launch_bounds__(1024) void softmaxStridedTileKernel(T* out, const T* in, int64_t dim, int64_t inner,
                                                                  int64_t innerBlocks) {
  __shared__ float sm[32][33], ss[32][33];
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  const int64_t o = blockIdx.x / innerBlocks, col = (blockIdx.x - o * innerBlocks) * 32 + tx;
  const bool live = col < inner;
  const T* src = in + o * dim * inner + col;
  T* dst = out + o * dim * inner + col;
  // differences are taken before the scaling by log2 e: the rounding of that product then grows with the distance
  // from the maximum, not with the size of the entry
  float m = -INFINITY, s = 0.f;
  if (live)
    for (int64_t d = ty; d < dim; d += 32) {
      const float v = static_cast<float>(src[d * inner]);
      const float mn = fmaxf(m, v);
      if (mn != -INFINITY) s = s * exp2f((m - mn) * kLog2e) + exp2f((v - mn) * kLog2e);
      m = mn;
    }
  sm[ty][tx] = m;
  ss[ty][tx] = s;
  __syncthreads();
  float mAll = -INFINITY, sAll = 0.f;
#pragma unroll
  for (int r = 0; r < 32; ++r) mAll = fmaxf(mAll, sm[r][tx]);
  if (mAll != -INFINITY) {
#pragma unroll
    for (int r = 0; r < 32; ++r) sAll += ss[r][tx] * exp2f((sm[r][tx] - mAll) * kLog2e);
  }
  const float inv = 1.f / sAll;  // a column of -inf: (-inf) - (-inf) below and 1 / 0 here give NaN, as the one-lane form does
  if (live)
    for (int64_t d = ty; d < dim; d += 32)
      dst[d * inner] = static_cast<T>(exp2f((static_cast<float>(src[d * inner]) - mAll) * kLog2e) * inv);
}

// mean of each dense row (one wave per row), fp32 accumulation
template <typename T>
__global__ __launch_bounds__(256) void rowMeanKernel(T* out, const T* in, int64_t rows, int64_t cols) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const T* src = in + row * cols;
  float s = 0.f;
  // 16-byte loads where the row allows (a lane reading one 2-byte element per step keeps a wave at 128 bytes per load:
  // [8192, 4096] bf16 took 22.8 us, as long as the fp32 tensor of twice the bytes)
  using V = typename Vec16<T>::type;
  constexpr int N = Vec16<T>::N;
  int64_t done = 0;
  if ((reinterpret_cast<uintptr_t>(src) & 15) == 0) {
    const int64_t nvec = cols / N;
    for (int64_t v = lane; v < nvec; v += 64) {
      const V x = reinterpret_cast<const V*>(src)[v];
#pragma unroll
      for (int j = 0; j < N; ++j) s += static_cast<float>(x[j]);
    }
    done = nvec * N;
  }
  for (int64_t c = done + lane; c < cols; c += 64) s += static_cast<float>(src[c]);
  s = waveSum(s);
  if (lane == 0) out[row] = static_cast<T>(s / (float)cols);
}

// Sums over the middle dim of a dense [outer, R, inner] tensor, inner > 1 (a mean over leading dims: the kept elements
// lie next to each other). A workgroup owns lpr VEC adjacent columns of one `outer` (lpr lanes per row, a power of two
// up to 64, so a wave load covers 64 / lpr rows of a narrow tensor) and one share of the R rows; its four waves take
// turns at the rows of the share with one VEC-wide load per lane (whole 1 KiB pieces of a row when VEC fills 16 bytes
// and lpr is 64), two loads ahead, and meet in LDS. With one share per column (partial == nullptr) the mean goes
// straight to `out`; otherwise the fp32 sums of share s go to partial[(o * shares + s) * inner + c] and
// finishMeanKernel adds them up. [8192, 4096] bf16 over dim 0: 13 + 4 us, against 50 us as a transposing copy followed
// by row means; all of it (one row of 33 M elements, rowShareSumKernel): 12 + 4 us.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void columnSumKernel(T* __restrict__ out, float* __restrict__ partial,
                                                       const T* __restrict__ in, int64_t R, int64_t inner,
                                                       int64_t rowsPerShare, int shares, int colTiles, int lpr, float scale) {
  __shared__ float red[4][64 * VEC];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int rpw = 64 / lpr, sub = lane / lpr, cl = lane & (lpr - 1);  // rows per wave load, this lane's row and column piece
  const int64_t flat = blockIdx.x;
  const int tile = (int)(flat % colTiles);
  const int share = (int)((flat / colTiles) % shares);
  const int64_t o = flat / ((int64_t)colTiles * shares);
  const int64_t c0 = ((int64_t)tile * lpr + cl) * VEC;
  const int64_t r0 = (int64_t)share * rowsPerShare, r1 = min(R, r0 + rowsPerShare);
  float s[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) s[j] = 0.f;
  if (c0 < inner) {  // inner is a multiple of VEC: a lane's columns are all live or all past the end
    const T* src = in + (o * R) * inner + c0;
    struct alignas(sizeof(T) * VEC) Piece { T v[VEC]; };
    const int step = 4 * rpw;
    int64_t r = r0 + wave * rpw + sub;
    for (; r + step < r1; r += 2 * step) {
      const Piece a = *reinterpret_cast<const Piece*>(src + r * inner);
      const Piece b = *reinterpret_cast<const Piece*>(src + (r + step) * inner);
#pragma unroll
      for (int j = 0; j < VEC; ++j) s[j] += static_cast<float>(a.v[j]) + static_cast<float>(b.v[j]);
    }
    if (r < r1) {
      const Piece a = *reinterpret_cast<const Piece*>(src + r * inner);
#pragma unroll
      for (int j = 0; j < VEC; ++j) s[j] += static_cast<float>(a.v[j]);
    }
  }
#pragma unroll
  for (int j = 0; j < VEC; ++j) red[wave][lane * VEC + j] = s[j];
  __syncthreads();
  // thread t finishes columns t, t + 256, ... of the tile: four waves times rpw rows of lanes each
  for (int c = threadIdx.x; c < lpr * VEC; c += 256) {
    const int64_t col = (int64_t)tile * lpr * VEC + c;
    if (col >= inner) break;
    float v = 0.f;
    for (int q = 0; q < rpw; ++q) {
      const int at = q * lpr * VEC + c;
      v += red[0][at] + red[1][at] + red[2][at] + red[3][at];
    }
    if (partial) partial[(o * shares + share) * inner + col] = v;
    else out[o * inner + col] = static_cast<T>(v * scale);
  }
}

// Sums of one share of each dense row, for a few very long rows (a mean over everything is one row): workgroup
// (row, share) adds its piece of the row with 16-byte loads where the piece allows and writes one fp32 sum.
template <typename T>
__global__ __launch_bounds__(256) void rowShareSumKernel(float* __restrict__ partial, const T* __restrict__ in,
                                                         int64_t cols, int64_t colsPerShare, int shares) {
  __shared__ float red[4];
  using V = typename Vec16<T>::type;
  constexpr int N = Vec16<T>::N;
  const int64_t row = blockIdx.x / shares;
  const int share = (int)(blockIdx.x % shares);
  const int64_t c0 = min(cols, (int64_t)share * colsPerShare), c1 = min(cols, c0 + colsPerShare);
  const T* src = in + row * cols;
  float s = 0.f;
  int64_t c = c0;
  if ((reinterpret_cast<uintptr_t>(src + c0) & 15) == 0) {
    const int64_t nvec = (c1 - c0) / N;
    const V* vs = reinterpret_cast<const V*>(src + c0);
    for (int64_t v = threadIdx.x; v < nvec; v += 256) {
      const V x = vs[v];
#pragma unroll
      for (int j = 0; j < N; ++j) s += static_cast<float>(x[j]);
    }
    c = c0 + nvec * N;
  }
  for (c += threadIdx.x; c < c1; c += 256) s += static_cast<float>(src[c]);
  s = waveSum(s);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0) partial[blockIdx.x] = red[0] + red[1] + red[2] + red[3];
}

// out[o, c] = scale * sum over s of partial[(o * shares + s) * inner + c]. A workgroup takes cpb adjacent columns (a
// power of two, at most 64) of one o; its 256 threads split the shares 256 / cpb ways and meet in LDS. (One thread
// per output walking the shares one after the other took 60 us for 256 shares of 4096 columns, 64 columns per
// workgroup with 64 shares per thread 12 us.)
template <typename T>
__global__ __launch_bounds__(256) void finishMeanKernel(T* __restrict__ out, const float* __restrict__ partial,
                                                        int64_t inner, int shares, int cpb, int colBlocks, float scale) {
  __shared__ float red[256];
  const int c = threadIdx.x & (cpb - 1), kg = threadIdx.x / cpb, kgs = 256 / cpb;
  const int64_t o = blockIdx.x / colBlocks;
  const int64_t col = (int64_t)(blockIdx.x % colBlocks) * cpb + c;
  float s = 0.f;
  if (col < inner) {
    const float* p = partial + (o * shares) * inner + col;
    for (int k = kg; k < shares; k += kgs) s += p[(int64_t)k * inner];
  }
  red[threadIdx.x] = s;
  __syncthreads();
  for (int stride = 128; stride >= cpb; stride >>= 1) {
    if ((int)threadIdx.x < stride) red[threadIdx.x] += red[threadIdx.x + stride];
    __syncthreads();
  }
  if ((int)threadIdx.x < cpb && col < inner) out[o * inner + col] = static_cast<T>(red[threadIdx.x] * scale);
}

template <typename T>
static void launchFinishMean(hipStream_t stream, T* out, const float* partial, int64_t outer, int64_t inner, int shares,
                             float scale) {
  // about eight shares per thread: many shares want few columns per workgroup (and so more workgroups)
  int cpb = 1;
  while (cpb < 64 && cpb * 2 <= inner && cpb * 2 * shares <= 2048) cpb *= 2;
  const int64_t colBlocks = ceilDiv(inner, (int64_t)cpb);
  hipLaunchKernelGGL(finishMeanKernel<T>, dim3((unsigned)(outer * colBlocks)), dim3(256), 0, stream, out, partial, inner,
                     shares, cpb, (int)colBlocks, scale);
}

template <typename T>
static diopiError_t launchColumnMean(diopiContextHandle_t ctx, hipStream_t stream, T* out, const T* in, int64_t outer,
                                     int64_t R, int64_t inner) {
  constexpr int N = Vec16<T>::N;
  const bool vec = inner % N == 0 && (reinterpret_cast<uintptr_t>(in) & 15) == 0;
  const int64_t pieces = vec ? inner / N : inner;  // per row
  int lpr = 1;
  while (lpr < 64 && lpr < pieces) lpr *= 2;
  const int64_t colTiles = ceilDiv(pieces, (int64_t)lpr);
  const int rowsPerPass = 4 * (64 / lpr);  // of the four waves together
  // two workgroups per CU where the rows allow, no share under sixteen passes (two to sixteen per CU and four to
  // sixteen passes all read 12.9 - 14.5 us on [8192, 4096] bf16; fewer shares leave less for the second kernel)
  const int64_t want = ceilDiv((int64_t)computeUnits() * 2, outer * colTiles);
  const int shares = (int)std::max<int64_t>(1, std::min<int64_t>(want, R / (16 * rowsPerPass)));
  const int64_t rowsPerShare = ceilDiv(R, (int64_t)shares);
  const int64_t wgs = outer * colTiles * shares;
  AMD_CHECK(wgs <= INT32_MAX && colTiles <= INT32_MAX, "diopiMean: %ld workgroups", (long)wgs);
  float* partial = nullptr;
  if (shares > 1) {
    void* ws = nullptr;
    AMD_TRY(requireWorkspace(ctx, outer * shares * inner * 4, &ws));
    partial = static_cast<float*>(ws);
  }
  const float scale = 1.f / (float)R;
  if (vec)
    hipLaunchKernelGGL((columnSumKernel<T, N>), dim3((unsigned)wgs), dim3(256), 0, stream, out, partial, in, R, inner,
                       rowsPerShare, shares, (int)colTiles, lpr, scale);
  else
    hipLaunchKernelGGL((columnSumKernel<T, 1>), dim3((unsigned)wgs), dim3(256), 0, stream, out, partial, in, R, inner,
                       rowsPerShare, shares, (int)colTiles, lpr, scale);
  AMD_LAUNCH_CHECK();
  if (partial) {
    launchFinishMean<T>(stream, out, partial, outer, inner, shares, scale);
    AMD_LAUNCH_CHECK();
  }
  return diopiSuccess;
}

// A few rows far longer than a wave's worth: shares of each row summed by separate workgroups, then added up.
template <typename T>
static diopiError_t launchLongRowMean(diopiContextHandle_t ctx, hipStream_t stream, T* out, const T* in, int64_t rows,
                                      int64_t cols) {
  constexpr int N = Vec16<T>::N;
  const int64_t want = ceilDiv((int64_t)computeUnits() * 8, rows);
  const int shares = (int)std::max<int64_t>(1, std::min<int64_t>(want, cols / 4096));
  // whole vectors per share, so every share of an aligned row starts aligned
  const int64_t colsPerShare = ceilDiv(ceilDiv(cols, (int64_t)shares), (int64_t)N) * N;
  void* ws = nullptr;
  AMD_TRY(requireWorkspace(ctx, rows * shares * 4, &ws));
  float* partial = static_cast<float*>(ws);
  hipLaunchKernelGGL(rowShareSumKernel<T>, dim3((unsigned)(rows * shares)), dim3(256), 0, stream, partial, in, cols,
                     colsPerShare, shares);
  AMD_LAUNCH_CHECK();
  launchFinishMean<T>(stream, out, partial, rows, 1, shares, 1.f / (float)cols);
  AMD_LAUNCH_CHECK();
  return diopiSuccess;
}

// ------------------------------------------------------------- dispatch ------
template <typename T, int OP, typename WT>
static diopiError_t launchRows(hipStream_t stream, T* out, const T* in, const WT* weight, const WT* bias,
                               float* invRms, int64_t rows, int64_t cols, int64_t inStride, int64_t outStride,
                               float eps, bool vectorOk) {
  constexpr int N = Vec16<T>::N;
  if (rows == 0 || cols == 0) return diopiSuccess;
  if (vectorOk && cols % N == 0 && cols / N <= 32 && rows >= 16) {
    const int nvec = (int)(cols / N), lpr = nvec <= 8 ? 8 : (nvec <= 16 ? 16 : 32);
    // 16 waves per CU, every wave 4 row groups of 64 / lpr rows per iteration
    const int64_t groups = ceilDiv(rows, (int64_t)(64 / lpr) * 4);
    dim3 grid((unsigned)std::min<int64_t>(ceilDiv(groups, 4), (int64_t)computeUnits() * 4)), block(256);
#define SUB_LAUNCH(LPR)                                                                                               \
  hipLaunchKernelGGL((rowSubWaveKernel<T, LPR, OP, WT>), grid, block, 0, stream, out, in, weight, bias, invRms, rows, \
                     (int)cols, inStride, outStride, eps)
    if (lpr == 8) SUB_LAUNCH(8);
    else if (lpr == 16) SUB_LAUNCH(16);
    else SUB_LAUNCH(32);
#undef SUB_LAUNCH
  } else if (vectorOk && cols % N == 0 && cols / N >= 256 && cols / N <= 64 * 16 && rows * 4 <= computeUnits()) {
    // A handful of long rows (the norms of a decode step): a workgroup per row shortens the chain load - reduce - store
    // that a single wave walks with eight vectors per lane.
    const int nvt = (int)ceilDiv(cols / N, 256);
    dim3 grid((unsigned)rows), block(256);
#define FEW_LAUNCH(NVT)                                                                                                \
  hipLaunchKernelGGL((rowBlockVecKernel<T, NVT, OP, WT>), grid, block, 0, stream, out, in, weight, bias, invRms, rows, \
                     (int)cols, inStride, outStride, eps)
    if (nvt <= 1) FEW_LAUNCH(1);
    else if (nvt <= 2) FEW_LAUNCH(2);
    else FEW_LAUNCH(4);
#undef FEW_LAUNCH
  } else if (vectorOk && cols % N == 0 && cols / N <= 64 * 8) {
    // (up to 8 vectors per lane; with 9 - 16 a wave holds the row and the next in 128 registers and up, and a workgroup
    // per row is as fast or faster: [6553, 5120] bf16 RMSNorm 26.4 -> 24.8 us, [4681, 7168] softmax 27.7 -> 23.2 us)
    int nvec = (int)(cols / N);
    int nv = (nvec + 63) / 64;
    // persistent waves: the kernels hold 16 waves per CU (4 per SIMD, <= 128 registers); give every
    // wave the same number of rows so that no CU idles in a last partial round
    const int64_t capacity = (int64_t)computeUnits() * 16;
    const int64_t rowsPerWave = ceilDiv(rows, capacity);
    dim3 grid((unsigned)ceilDiv(ceilDiv(rows, rowsPerWave), 4)), block(256);
#define ROW_LAUNCH(NV)                                                                                            \
  hipLaunchKernelGGL((rowWaveKernel<T, NV, OP, WT>), grid, block, 0, stream, out, in, weight, bias, invRms, rows, \
                     (int)cols, inStride, outStride, eps)
    if (nv <= 1) ROW_LAUNCH(1);
    else if (nv <= 2) ROW_LAUNCH(2);
    else if (nv <= 4) ROW_LAUNCH(4);
    else ROW_LAUNCH(8);
#undef ROW_LAUNCH
  } else if (vectorOk && cols % N == 0 && cols / N <= 256 * 32) {
    const int nvt = (int)ceilDiv(cols / N, 256);
    dim3 grid((unsigned)std::min<int64_t>(rows, (int64_t)computeUnits() * 8)), block(256);
#define BLOCK_LAUNCH(NVT)                                                                                               \
  hipLaunchKernelGGL((rowBlockVecKernel<T, NVT, OP, WT>), grid, block, 0, stream, out, in, weight, bias, invRms, rows, \
                     (int)cols, inStride, outStride, eps)
    if (nvt <= 2) BLOCK_LAUNCH(2);
    else if (nvt <= 4) BLOCK_LAUNCH(4);
    else if (nvt <= 8) BLOCK_LAUNCH(8);
    else if (nvt <= 16) BLOCK_LAUNCH(16);
    else BLOCK_LAUNCH(32);
#undef BLOCK_LAUNCH
  } else if (cols > 12288) {
    // longer than the register and LDS forms hold: two streaming passes, in 16-byte pieces where the rows allow them
    dim3 grid((unsigned)std::min<int64_t>(rows, (int64_t)computeUnits() * 2)), block(1024);
    if (vectorOk && cols % N == 0)
      hipLaunchKernelGGL((rowStreamKernel<T, OP, WT, true>), grid, block, 0, stream, out, in, weight, bias, invRms, rows, cols,
                         inStride, outStride, eps);
    else
      hipLaunchKernelGGL((rowStreamKernel<T, OP, WT, false>), grid, block, 0, stream, out, in, weight, bias, invRms, rows, cols,
                         inStride, outStride, eps);
  } else {
    int stage = (int)cols;  // at most 48 KiB of fp32 staging
    size_t lds = (8 + (size_t)stage) * sizeof(float);
    hipLaunchKernelGGL((rowBlockKernel<T, OP, WT>), dim3((unsigned)rows), dim3(256), lds, stream, out, in, weight,
                       bias, invRms, rows, cols, inStride, outStride, eps, stage);
  }
  AMD_LAUNCH_CHECK();
  return diopiSuccess;
}

}  // namespace amd

using namespace amd;

extern "C" __attribute__((visibility("default"))) diopiError_t diopiSoftmax(diopiContextHandle_t ctx,
                                                                            diopiTensorHandle_t outH,
                                                                            diopiConstTensorHandle_t inH,
                                                                            int64_t dim) {
  hipStream_t stream;
  AMD_TRY(getStream(ctx, &stream));
  TensorView out, in;
  AMD_TRY(getView(outH, &out, "out"));
  AMD_TRY(getView(inH, &in, "input"));
  AMD_CHECK(out.defined() && in.defined(), "diopiSoftmax: null tensor");
  AMD_CHECK(out.dtype == in.dtype, "diopiSoftmax: out dtype %s differs from input dtype %s", dtypeName(out.dtype),
            dtypeName(in.dtype));
  AMD_CHECK(out.ndim == in.ndim, "diopiSoftmax: rank mismatch");
  for (int d = 0; d < in.ndim; ++d) AMD_CHECK(out.shape[d] == in.shape[d], "diopiSoftmax: shape mismatch at dim %d", d);
  if (in.numel == 0) return diopiSuccess;
  if (in.ndim == 0) {  // softmax of a scalar is 1
    diopiScalar_t one;
    one.stype = diopi_dtype_float64;
    one.fval = 1.0;
    return diopiFill(ctx, outH, &one);
  }
  if (dim < 0) dim += in.ndim;
  AMD_CHECK(dim >= 0 && dim < in.ndim, "diopiSoftmax: dim out of range");
  AMD_CHECK(in.dtype == diopi_dtype_bfloat16 || in.dtype == diopi_dtype_float16 || in.dtype == diopi_dtype_float32,
            "diopiSoftmax: unsupported dtype %s", dtypeName(in.dtype));
  TensorView cin;
  AMD_TRY(makeContiguous(ctx, stream, in, &cin));
  // a non-dense output is produced densely and copied back
  TensorView cout = out;
  bool outTemp = !out.isContiguous();
  if (outTemp) {
    diopiTensorHandle_t th;
    AMD_TRY(requireTensor(ctx, out.shape, out.ndim, out.dtype, &th, &cout));
  }
  int64_t outer = 1, inner = 1, n = in.shape[dim];
  for (int d = 0; d < dim; ++d) outer *= in.shape[d];
  for (int d = (int)dim + 1; d < in.ndim; ++d) inner *= in.shape[d];
  diopiError_t err = diopiSuccess;
  if (inner == 1) {
    bool vecOk = cin.aligned16() && cout.aligned16() && (n * in.itemsize) % 16 == 0;
    switch (in.dtype) {
      case diopi_dtype_bfloat16:
        err = launchRows<bf16_t, kRowSoftmax, bf16_t>(stream, cout.ptr<bf16_t>(), cin.ptr<bf16_t>(), nullptr, nullptr,
                                                      nullptr, outer, n, n, n, 0.f, vecOk);
        break;
      case diopi_dtype_float16:
        err = launchRows<half_t, kRowSoftmax, half_t>(stream, cout.ptr<half_t>(), cin.ptr<half_t>(), nullptr, nullptr,
                                                      nullptr, outer, n, n, n, 0.f, vecOk);
        break;
      default:
        err = launchRows<float, kRowSoftmax, float>(stream, cout.ptr<float>(), cin.ptr<float>(), nullptr, nullptr,
                                                    nullptr, outer, n, n, n, 0.f, vecOk);
        break;
    }
  } else if (n >= 128 && inner >= 16 && outer * ceilDiv(inner, 32) < ((int64_t)1 << 31)) {
    const int64_t innerBlocks = ceilDiv(inner, 32);
    dim3 grid((unsigned)(outer * innerBlocks)), block(1024);
    switch (in.dtype) {
      case diopi_dtype_bfloat16:
        hipLaunchKernelGGL(softmaxStridedTileKernel<bf16_t>, grid, block, 0, stream, cout.ptr<bf16_t>(), cin.ptr<bf16_t>(), n,
                           inner, innerBlocks);
        break;
      case diopi_dtype_float16:
        hipLaunchKernelGGL(softmaxStridedTileKernel<half_t>, grid, block, 0, stream, cout.ptr<half_t>(), cin.ptr<half_t>(), n,
                           inner, innerBlocks);
        break;
      default:
        hipLaunchKernelGGL(softmaxStridedTileKernel<float>, grid, block, 0, stream, cout.ptr<float>(), cin.ptr<float>(), n,
                           inner, innerBlocks);
        break;
    }
    AMD_LAUNCH_CHECK();
  } else {
    int64_t colsTotal = outer * inner;
    dim3 grid((unsigned)ceilDiv(colsTotal, 256)), block(256);
    switch (in.dtype) {
      case diopi_dtype_bfloat16:
        hipLaunchKernelGGL(softmaxStridedKernel<bf16_t>, grid, block, 0, stream, cout.ptr<bf16_t>(), cin.ptr<bf16_t>(),
                           outer, n, inner);
        break;
      case diopi_dtype_float16:
        hipLaunchKernelGGL(softmaxStridedKernel<half_t>, grid, block, 0, stream, cout.ptr<half_t>(), cin.ptr<half_t>(),
                           outer, n, inner);
        break;
      default:
        hipLaunchKernelGGL(softmaxStridedKernel<float>, grid, block, 0, stream, cout.ptr<float>(), cin.ptr<float>(),
                           outer, n, inner);
        break;
    }
    AMD_LAUNCH_CHECK();
  }
  AMD_TRY(err);
  if (outTemp) AMD_TRY(stridedCopy(stream, cout, out));
  return diopiSuccess;
}

template <typename T>
static diopiError_t rmsNormTyped(hipStream_t stream, const TensorView& out, const TensorView& in,
                                 const TensorView& w, const TensorView& b, float* invRms, int64_t rows, int64_t cols,
                                 float eps) {
  bool vecOk = in.aligned16() && out.aligned16() && (cols * in.itemsize) % 16 == 0;
  diopiDtype_t wdt = w.defined() ? w.dtype : (b.defined() ? b.dtype : in.dtype);
  if (w.defined()) vecOk = vecOk && w.aligned16();
  if (b.defined()) vecOk = vecOk && b.aligned16();
  if (wdt == in.dtype) {
    return launchRows<T, kRowRmsNorm, T>(stream, out.ptr<T>(), in.ptr<T>(), w.ptr<T>(), b.ptr<T>(), invRms, rows, cols,
                                         cols, cols, eps, vecOk);
  }
  AMD_CHECK(wdt == diopi_dtype_float32, "diopiRMSNorm: weight dtype %s must equal the input dtype or be float32",
            dtypeName(wdt));
  return launchRows<T, kRowRmsNorm, float>(stream, out.ptr<T>(), in.ptr<T>(), w.ptr<float>(), b.ptr<float>(), invRms,
                                           rows, cols, cols, cols, eps, vecOk);
}

extern "C" __attribute__((visibility("default"))) diopiError_t diopiRMSNorm(
    diopiContextHandle_t ctx, diopiTensorHandle_t outH, diopiTensorHandle_t invRmsH, diopiConstTensorHandle_t inH,
    diopiSize_t normalizedShape, diopiConstTensorHandle_t weightH, diopiConstTensorHandle_t biasH, double eps) {
  hipStream_t stream;
  AMD_TRY(getStream(ctx, &stream));
  TensorView out, inv, in, w, b;
  AMD_TRY(getView(outH, &out, "out"));
  AMD_TRY(getView(invRmsH, &inv, "inv_rms"));
  AMD_TRY(getView(inH, &in, "input"));
  AMD_TRY(getView(weightH, &w, "weight"));
  AMD_TRY(getView(biasH, &b, "bias"));
  AMD_CHECK(out.defined() && in.defined(), "diopiRMSNorm: null tensor");
  AMD_CHECK(out.dtype == in.dtype, "diopiRMSNorm: out dtype differs from input dtype");
  AMD_CHECK(out.ndim == in.ndim, "diopiRMSNorm: rank mismatch");
  for (int d = 0; d < in.ndim; ++d) AMD_CHECK(out.shape[d] == in.shape[d], "diopiRMSNorm: shape mismatch at dim %d", d);
  AMD_CHECK(normalizedShape.len >= 1 && normalizedShape.len <= in.ndim, "diopiRMSNorm: bad normalized_shape rank");
  int64_t cols = 1;
  for (int64_t i = 0; i < normalizedShape.len; ++i) {
    int64_t e = in.shape[in.ndim - normalizedShape.len + i];
    AMD_CHECK(normalizedShape.data[i] == e, "diopiRMSNorm: normalized_shape[%ld]=%ld but input extent is %ld", (long)i,
              (long)normalizedShape.data[i], (long)e);
    cols *= e;
  }
  if (in.numel == 0) return diopiSuccess;
  int64_t rows = in.numel / cols;
  if (w.defined()) AMD_CHECK(w.numel == cols, "diopiRMSNorm: weight has %ld elements, expected %ld", (long)w.numel, (long)cols);
  if (b.defined()) AMD_CHECK(b.numel == cols, "diopiRMSNorm: bias has %ld elements, expected %ld", (long)b.numel, (long)cols);
  if (w.defined() && b.defined()) AMD_CHECK(w.dtype == b.dtype, "diopiRMSNorm: weight and bias dtypes differ");
  AMD_CHECK(in.dtype == diopi_dtype_bfloat16 || in.dtype == diopi_dtype_float16 || in.dtype == diopi_dtype_float32,
            "diopiRMSNorm: unsupported dtype %s", dtypeName(in.dtype));
  TensorView cin, cw, cb;
  AMD_TRY(makeContiguous(ctx, stream, in, &cin));
  if (w.defined()) AMD_TRY(makeContiguous(ctx, stream, w, &cw));
  if (b.defined()) AMD_TRY(makeContiguous(ctx, stream, b, &cb));
  TensorView cout = out;
  bool outTemp = !out.isContiguous();
  if (outTemp) {
    diopiTensorHandle_t th;
    AMD_TRY(requireTensor(ctx, out.shape, out.ndim, out.dtype, &th, &cout));
  }
  // inv_rms is produced as fp32 [rows]; other dtypes/layouts are converted afterwards
  float* invPtr = nullptr;
  TensorView invTmp;
  bool invDirect = false;
  if (inv.defined()) {
    AMD_CHECK(inv.numel == rows, "diopiRMSNorm: inv_rms has %ld elements, expected %ld", (long)inv.numel, (long)rows);
    invDirect = inv.dtype == diopi_dtype_float32 && inv.isContiguous();
    if (invDirect) {
      invPtr = inv.ptr<float>();
    } else {
      diopiTensorHandle_t th;
      AMD_TRY(requireTensor(ctx, inv.shape, inv.ndim, diopi_dtype_float32, &th, &invTmp));
      invPtr = invTmp.ptr<float>();
    }
  }
  diopiError_t err;
  switch (in.dtype) {
    case diopi_dtype_bfloat16: err = rmsNormTyped<bf16_t>(stream, cout, cin, cw, cb, invPtr, rows, cols, (float)eps); break;
    case diopi_dtype_float16: err = rmsNormTyped<half_t>(stream, cout, cin, cw, cb, invPtr, rows, cols, (float)eps); break;
    default: err = rmsNormTyped<float>(stream, cout, cin, cw, cb, invPtr, rows, cols, (float)eps); break;
  }
  AMD_TRY(err);
  if (outTemp) AMD_TRY(stridedCopy(stream, cout, out));
  if (inv.defined() && !invDirect) AMD_TRY(stridedCopy(stream, invTmp, inv));
  return diopiSuccess;
}

// mean over `dims`. Reduced dims that lie next to each other in a dense input with kept dims after them are summed
// down the columns where they lie; otherwise the kept dims are moved to the front (a strided view, made dense if it
// is not) and each row of prod(reduced) elements is averaged by one wave, or by many workgroups when the rows are few
// and long.
extern "C" __attribute__((visibility("default"))) diopiError_t diopiMean(diopiContextHandle_t ctx,
                                                                         diopiTensorHandle_t outH,
                                                                         diopiConstTensorHandle_t inH,
                                                                         diopiSize_t dims) {
  hipStream_t stream;
  AMD_TRY(getStream(ctx, &stream));
  TensorView out, in;
  AMD_TRY(getView(outH, &out, "out"));
  AMD_TRY(getView(inH, &in, "input"));
  AMD_CHECK(out.defined() && in.defined(), "diopiMean: null tensor");
  AMD_CHECK(out.dtype == in.dtype, "diopiMean: dtype conversion is not supported");
  AMD_CHECK(in.dtype == diopi_dtype_bfloat16 || in.dtype == diopi_dtype_float16 || in.dtype == diopi_dtype_float32,
            "diopiMean: unsupported dtype %s", dtypeName(in.dtype));
  bool reduced[kMaxDims] = {false};
  if (dims.len == 0) {
    for (int d = 0; d < in.ndim; ++d) reduced[d] = true;
  }
  for (int64_t i = 0; i < dims.len; ++i) {
    int64_t d = dims.data[i] < 0 ? dims.data[i] + in.ndim : dims.data[i];
    AMD_CHECK(d >= 0 && d < in.ndim, "diopiMean: dim %ld out of range", (long)dims.data[i]);
    reduced[d] = true;
  }
  TensorView perm = in;
  int w = 0;
  int64_t rows = 1, cols = 1;
  for (int d = 0; d < in.ndim; ++d)
    if (!reduced[d]) perm.shape[w] = in.shape[d], perm.stride[w] = in.stride[d], rows *= in.shape[d], ++w;
  for (int d = 0; d < in.ndim; ++d)
    if (reduced[d]) perm.shape[w] = in.shape[d], perm.stride[w] = in.stride[d], cols *= in.shape[d], ++w;
  AMD_CHECK(out.numel == rows, "diopiMean: output has %ld elements, expected %ld", (long)out.numel, (long)rows);
  if (rows == 0) return diopiSuccess;
  TensorView cout = out;
  bool outTemp = !out.isContiguous();
  if (outTemp) {
    diopiTensorHandle_t th;
    AMD_TRY(requireTensor(ctx, out.shape, out.ndim, out.dtype, &th, &cout));
  }
  // The reduced dims of a dense input next to each other, kept dims after them: [outer, R, inner] summed over R where
  // it lies (no transposing copy).
  int firstRed = -1, lastRed = -1, nRed = 0;
  for (int d = 0; d < in.ndim; ++d)
    if (reduced[d]) firstRed = firstRed < 0 ? d : firstRed, lastRed = d, ++nRed;
  const bool oneRun = nRed > 0 && lastRed - firstRed + 1 == nRed && in.isContiguous() && cols > 0;
  int64_t inner = 1;
  for (int d = lastRed + 1; oneRun && d < in.ndim; ++d) inner *= in.shape[d];
#define MEAN_BY_DTYPE(CALL)                                                           \
  switch (in.dtype) {                                                                 \
    case diopi_dtype_bfloat16: { using T = bf16_t; AMD_TRY(CALL); break; }            \
    case diopi_dtype_float16: { using T = half_t; AMD_TRY(CALL); break; }             \
    default: { using T = float; AMD_TRY(CALL); break; }                               \
  }
  if (oneRun && inner > 1) {
    MEAN_BY_DTYPE((launchColumnMean<T>(ctx, stream, cout.ptr<T>(), in.ptr<T>(), rows / inner, cols, inner)));
    if (outTemp) AMD_TRY(stridedCopy(stream, cout, out));
    return diopiSuccess;
  }
  TensorView cin;
  AMD_TRY(makeContiguous(ctx, stream, perm, &cin));
  if (rows * 4 <= computeUnits() && cols >= 65536) {
    MEAN_BY_DTYPE((launchLongRowMean<T>(ctx, stream, cout.ptr<T>(), cin.ptr<T>(), rows, cols)));
    if (outTemp) AMD_TRY(stridedCopy(stream, cout, out));
    return diopiSuccess;
  }
#undef MEAN_BY_DTYPE
  dim3 grid((unsigned)ceilDiv(rows, 4)), block(256);
  switch (in.dtype) {
    case diopi_dtype_bfloat16:
      hipLaunchKernelGGL(rowMeanKernel<bf16_t>, grid, block, 0, stream, cout.ptr<bf16_t>(), cin.ptr<bf16_t>(), rows, cols);
      break;
    case diopi_dtype_float16:
      hipLaunchKernelGGL(rowMeanKernel<half_t>, grid, block, 0, stream, cout.ptr<half_t>(), cin.ptr<half_t>(), rows, cols);
      break;
    default:
      hipLaunchKernelGGL(rowMeanKernel<float>, grid, block, 0, stream, cout.ptr<float>(), cin.ptr<float>(), rows, cols);
      break;
  }
  AMD_LAUNCH_CHECK();
  if (outTemp) AMD_TRY(stridedCopy(stream, cout, out));
  return diopiSuccess;
}
