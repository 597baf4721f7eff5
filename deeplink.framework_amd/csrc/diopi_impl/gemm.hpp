// Internal GEMM interface shared by the dense (diopiMm/Bmm/Matmul/Addmm/Baddbmm/Linear)
// entry points. One problem description, two engines:
//   * the MFMA engine (bf16/fp16, fp32 accumulate) for K-contiguous operands,
//   * a strided fp32-accumulate FMA engine for everything else (fp32, odd shapes).
#pragma once

#include "common.hpp"

namespace amd {

// out[b, m, n] = alpha * sum_k A[b, m, k] * B[b, n, k]  +  beta * Cin[b, m, n]  +  bias[n]
// All strides in elements. B is described in [N, K] orientation whatever its storage order.
struct GemmProblem {
  diopiDtype_t dtype = diopi_dtype_unsupported;  // A, B, out (and Cin/bias) element type
  int64_t batch = 1, M = 0, N = 0, K = 0;
  const void* A = nullptr;
  int64_t sAb = 0, sAm = 0, sAk = 0;
  const void* B = nullptr;
  int64_t sBb = 0, sBn = 0, sBk = 0;
  void* out = nullptr;
  int64_t sOb = 0, sOm = 0;  // out: n-contiguous
  const void* Cin = nullptr;
  int64_t sCb = 0, sCm = 0, sCn = 0;
  const void* bias = nullptr;
  float alpha = 1.f, beta = 0.f;
  // out[m, n] = alpha * sum * colScale[n] + colBias[n], one rounding: N values each of their own dtype (fp16 / bf16 /
  // fp32), colBias optional. Only for problems gemmAppliesColumnScale accepts (no addend, no `bias`).
  const void* colScale = nullptr;
  diopiDtype_t colScaleDtype = diopi_dtype_float32;
  const void* colBias = nullptr;
  diopiDtype_t colBiasDtype = diopi_dtype_float32;
};

diopiError_t runGemm(diopiContextHandle_t ctx, hipStream_t stream, GemmProblem p);

// Whether runGemm would send p to the kernel whose epilogue can multiply every column by a scale of its own (the
// 4-wave large-tile kernel): the caller sets colScale only then, and applies the scale in a pass of its own otherwise.
bool gemmAppliesColumnScale(const GemmProblem& p);

// diopiRotaryEmbedding on views (rotary_kv.hip): out and x of shape [..., heads, head_dim], strided views allowed.
diopiError_t runRotary(diopiContextHandle_t ctx, hipStream_t stream, const TensorView& out, const TensorView& x,
                       const TensorView& cosT, const TensorView& sinT, bool conj, bool interleaved);

// dst[b, c, r] = src[b, r, c] for 2-byte or 4-byte elements (64 x 64 tiles through LDS): src is [rows, cols] with the
// element strides given, dst dense [cols, rows] per batch.
diopiError_t transposeCopy(hipStream_t stream, void* dst, const void* src, int itemsize, int64_t batch, int64_t rows,
                           int64_t cols, int64_t sRow, int64_t sCol, int64_t sBatch);

}  // namespace amd
