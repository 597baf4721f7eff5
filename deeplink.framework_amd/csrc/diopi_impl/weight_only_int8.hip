// diopiWeightOnlyInt8Linear for gfx950: out[M,N] = x[M,K] . (W_int8[N,K] * scale[N])^T + bias.
//
// Skinny-M (decode) shape: the int8 weight matrix is streamed from HBM exactly once and is
// the only traffic of size (K*N bytes); everything else (x, scale, out) is tiny and stays
// in L2. The kernel is a GEMV-shaped MFMA kernel:
//   * a workgroup owns 16 output channels; its 4 waves split K four ways; each
//     wave keeps 8 weight + 16 activation vectors per lane in flight;
//   * v_mfma_f32_16x16x32_{bf16,f16}: the B operand is the weight tile -- lane (n = lane%16,
//     kgrp = lane/16) loads 32 consecutive int8 of row n (two 16-byte loads; the 4 kgrps of a
//     row cover 128 contiguous bytes) and converts them to bf16/fp16 in registers while
//     the next loads are in flight: the dequantisation is fused into the operand load;
//   * the A operand is x (rows beyond M are clamped and discarded), read with the same
//     K permutation as the weights, so no shuffle is needed;
//   * fp32 accumulators of the 4 waves are summed through LDS; the per-channel scale is
//     applied to the fp32 sum (identical to scaling the weights first, one rounding fewer),
//     then bias, then one conversion to the output dtype.
// Rows of x beyond 16 are handled by more workgroups along grid.y (weights are then re-read
// per group of 16 rows; large-M prefill should dequantise once and use the dense GEMM).
#include "common.hpp"

namespace amd {

template <typename T>
struct W8Mfma;
template <>
struct W8Mfma<bf16_t> {
  typedef bf16x8 Frag;
  static __device__ __forceinline__ f32x4 run(Frag a, Frag b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};
template <>
struct W8Mfma<half_t> {
  typedef f16x8 Frag;
  static __device__ __forceinline__ f32x4 run(Frag a, Frag b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};

struct W8Args {
  const void* x;
  const int8_t* w;
  const void* scale;
  const void* bias;
  void* out;
  int64_t ldx, ldw, ldo;
  int M, N, K;
  int scaleDtype, biasDtype;
};

// converts 8 consecutive int8 (two dwords) to an MFMA operand fragment
template <typename T>
__device__ __forceinline__ typename W8Mfma<T>::Frag cvt8(uint32_t lo, uint32_t hi) {
  typename W8Mfma<T>::Frag f;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    f[j] = static_cast<T>(static_cast<float>(static_cast<int8_t>((lo >> (8 * j)) & 0xff)));
    f[4 + j] = static_cast<T>(static_cast<float>(static_cast<int8_t>((hi >> (8 * j)) & 0xff)));
  }
  return f;
}

constexpr int kW8Block = 128;  // K elements one wave consumes per step (4 kgrps x 32)
constexpr int kW8Unroll = 4;   // steps in flight
constexpr int kW8Waves = 4;    // waves per workgroup = K splits (8 measured slower for M > 1)

template <typename T>
__global__ __launch_bounds__(kW8Waves * 64) void w8LinearKernel(W8Args a) {
  using Frag = typename W8Mfma<T>::Frag;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r16 = lane & 15, kgrp = lane >> 4;
  const int n0 = blockIdx.x * 16, m0 = blockIdx.y * 16;
  const int n = min(n0 + r16, a.N - 1);
  const int m = min(m0 + r16, a.M - 1);
  const int8_t* wrow = a.w + (int64_t)n * a.ldw + kgrp * 32;
  const T* xrow = reinterpret_cast<const T*>(a.x) + (int64_t)m * a.ldx + kgrp * 32;
  // K is split in kW8Waves contiguous parts (rounded to the 128-element step), one per wave; at
  // K = 4096 a wave owns 4 steps, i.e. every load of the wave is issued in one go
  const int steps = (a.K + kW8Block - 1) / kW8Block;
  const int per = (steps + kW8Waves - 1) / kW8Waves;
  const int sBegin = wave * per, sEnd = min(steps, sBegin + per);
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int s = sBegin; s < sEnd; s += kW8Unroll) {
    u32x4 wv[kW8Unroll][2];
    Frag xv[kW8Unroll][4];
#pragma unroll
    for (int u = 0; u < kW8Unroll; ++u) {
      const int k = (s + u) * kW8Block;
      // K % 128 == 0 is guaranteed by the host, so a step is entirely inside or outside
      const bool in = s + u < sEnd;
      const int kk = in ? k : 0;
      wv[u][0] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wrow + kk));
      wv[u][1] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wrow + kk + 16));
#pragma unroll
      for (int j = 0; j < 4; ++j) xv[u][j] = *reinterpret_cast<const Frag*>(xrow + kk + j * 8);
    }
#pragma unroll
    for (int u = 0; u < kW8Unroll; ++u) {
      if (s + u < sEnd) {
        acc = W8Mfma<T>::run(xv[u][0], cvt8<T>(wv[u][0][0], wv[u][0][1]), acc);
        acc = W8Mfma<T>::run(xv[u][1], cvt8<T>(wv[u][0][2], wv[u][0][3]), acc);
        acc = W8Mfma<T>::run(xv[u][2], cvt8<T>(wv[u][1][0], wv[u][1][1]), acc);
        acc = W8Mfma<T>::run(xv[u][3], cvt8<T>(wv[u][1][2], wv[u][1][3]), acc);
      }
    }
  }
  __shared__ float red[kW8Waves][64][4];
#pragma unroll
  for (int r = 0; r < 4; ++r) red[wave][lane][r] = acc[r];
  __syncthreads();
  if (wave == 0) {
    const int col = n0 + r16;
    if (col < a.N) {
      const float sc = loadAs<float>(a.scale, col, a.scaleDtype);
      const float bv = a.bias ? loadAs<float>(a.bias, col, a.biasDtype) : 0.f;
      T* out = reinterpret_cast<T*>(a.out);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = m0 + kgrp * 4 + r;
        if (row < a.M) {
          float v = 0.f;
#pragma unroll
          for (int w = 0; w < kW8Waves; ++w) v += red[w][lane][r];
          out[(int64_t)row * a.ldo + col] = static_cast<T>(v * sc + bv);
        }
      }
    }
  }
}

// Any K / alignment: one lane per output element, fp32 accumulate (correctness path).
template <typename T>
__global__ __launch_bounds__(256) void w8LinearScalarKernel(W8Args a) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (int64_t)a.M * a.N) return;
  const int m = (int)(idx / a.N), n = (int)(idx % a.N);
  const T* x = reinterpret_cast<const T*>(a.x) + (int64_t)m * a.ldx;
  const int8_t* w = a.w + (int64_t)n * a.ldw;
  float acc = 0.f;
  for (int k = 0; k < a.K; ++k) acc += static_cast<float>(x[k]) * static_cast<float>(w[k]);
  float v = acc * loadAs<float>(a.scale, n, a.scaleDtype);
  if (a.bias) v += loadAs<float>(a.bias, n, a.biasDtype);
  reinterpret_cast<T*>(a.out)[(int64_t)m * a.ldo + n] = static_cast<T>(v);
}

}  // namespace amd

using namespace amd;

extern "C" __attribute__((visibility("default"))) diopiError_t diopiWeightOnlyInt8Linear(
    diopiContextHandle_t ctx, diopiTensorHandle_t outH, diopiConstTensorHandle_t inH, diopiConstTensorHandle_t wH,
    diopiConstTensorHandle_t scaleH, diopiConstTensorHandle_t biasH) {
  hipStream_t stream;
  AMD_TRY(getStream(ctx, &stream));
  TensorView out, in, w, sc, bias;
  AMD_TRY(getView(outH, &out, "out"));
  AMD_TRY(getView(inH, &in, "input"));
  AMD_TRY(getView(wH, &w, "weight"));
  AMD_TRY(getView(scaleH, &sc, "scale"));
  AMD_TRY(getView(biasH, &bias, "bias"));
  AMD_CHECK(out.defined() && in.defined() && w.defined() && sc.defined(), "diopiWeightOnlyInt8Linear: null tensor");
  AMD_CHECK(w.dtype == diopi_dtype_int8 && w.ndim == 2, "diopiWeightOnlyInt8Linear: weight must be int8 [N, K]");
  AMD_CHECK(in.dtype == diopi_dtype_bfloat16 || in.dtype == diopi_dtype_float16,
            "diopiWeightOnlyInt8Linear: input must be bfloat16 or float16, got %s", dtypeName(in.dtype));
  AMD_CHECK(out.dtype == in.dtype, "diopiWeightOnlyInt8Linear: out dtype differs from input dtype");
  AMD_CHECK(in.ndim >= 1 && out.ndim == in.ndim, "diopiWeightOnlyInt8Linear: out must be shaped like input");
  const int64_t N = w.shape[0], K = w.shape[1];
  AMD_CHECK(in.shape[in.ndim - 1] == K, "diopiWeightOnlyInt8Linear: input last dim %ld differs from K=%ld",
            (long)in.shape[in.ndim - 1], (long)K);
  AMD_CHECK(out.shape[out.ndim - 1] == N, "diopiWeightOnlyInt8Linear: out last dim %ld differs from N=%ld",
            (long)out.shape[out.ndim - 1], (long)N);
  AMD_CHECK(sc.numel == N && isFloatDtype(sc.dtype) && sc.dtype != diopi_dtype_float64,
            "diopiWeightOnlyInt8Linear: scale must hold N fp16/bf16/fp32 values");
  if (bias.defined())
    AMD_CHECK(bias.numel == N && isFloatDtype(bias.dtype) && bias.dtype != diopi_dtype_float64,
              "diopiWeightOnlyInt8Linear: bias must hold N fp16/bf16/fp32 values");
  const int64_t M = K > 0 ? in.numel / K : 0;
  AMD_CHECK(out.numel == M * N, "diopiWeightOnlyInt8Linear: out has %ld elements, expected %ld", (long)out.numel, (long)(M * N));
  if (M == 0 || N == 0) return diopiSuccess;
  TensorView cin, cw, csc, cb;
  AMD_TRY(makeContiguous(ctx, stream, in, &cin));
  AMD_TRY(makeContiguous(ctx, stream, sc, &csc));
  if (bias.defined()) AMD_TRY(makeContiguous(ctx, stream, bias, &cb));
  cw = w;
  if (!(w.stride[1] == 1 || K == 1)) AMD_TRY(makeContiguous(ctx, stream, w, &cw));
  TensorView cout = out;
  bool outTemp = !out.isContiguous();
  if (outTemp) {
    diopiTensorHandle_t th;
    AMD_TRY(requireTensor(ctx, out.shape, out.ndim, out.dtype, &th, &cout));
  }
  W8Args a;
  a.x = cin.data, a.w = cw.ptr<int8_t>(), a.scale = csc.data, a.bias = bias.defined() ? cb.data : nullptr, a.out = cout.data;
  a.ldx = K, a.ldw = N > 1 ? cw.stride[0] : K, a.ldo = N;
  a.M = (int)M, a.N = (int)N, a.K = (int)K;
  a.scaleDtype = csc.dtype, a.biasDtype = bias.defined() ? cb.dtype : diopi_dtype_float32;
  const bool fast = K % kW8Block == 0 && cin.aligned16() && cw.aligned16() && a.ldw % 16 == 0 && ceilDiv(M, 16) <= 65535;
  if (fast) {
    dim3 grid((unsigned)ceilDiv(N, 16), (unsigned)ceilDiv(M, 16));
    if (in.dtype == diopi_dtype_bfloat16) hipLaunchKernelGGL(w8LinearKernel<bf16_t>, grid, dim3(kW8Waves * 64), 0, stream, a);
    else hipLaunchKernelGGL(w8LinearKernel<half_t>, grid, dim3(kW8Waves * 64), 0, stream, a);
  } else {
    dim3 grid((unsigned)ceilDiv(M * N, 256));
    if (in.dtype == diopi_dtype_bfloat16) hipLaunchKernelGGL(w8LinearScalarKernel<bf16_t>, grid, dim3(256), 0, stream, a);
    else hipLaunchKernelGGL(w8LinearScalarKernel<half_t>, grid, dim3(256), 0, stream, a);
  }
  AMD_LAUNCH_CHECK();
  if (outTemp) AMD_TRY(stridedCopy(stream, cout, out));
  return diopiSuccess;
}
