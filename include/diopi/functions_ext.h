/*
 * DIOPI extension entry points for transformer inference (MI355X backend).
 *
 * None of these has a call site in the reference: DIPU's op adapter
 * (dipu/scripts/autogen_diopi_wrapper/diopi_functions.yaml,
 * dipu/SupportedDiopiFunctions.txt:1-262) wraps no RMSNorm / rotary / KV-scatter /
 * attention / weight-only function; the DeepLink ecosystem binds them from a
 * separate repository pinned only as a CI clone (dipu/scripts/ci/ci_benchmark.sh:35).
 * The SIGNATURES therefore follow upstream DIOPI's functions_ext.h as recalled and
 * are unverifiable here ("parity unpinned at the ABI"); the SEMANTICS each one
 * implements are pinned by the pure-PyTorch definitions the reference does hold,
 * cited per function below (dicp/dicp/vendor/AscendGraph/ext_ops.py and
 * dicp/test/model/llama/model.py).
 */
#ifndef DIOPI_FUNCTIONS_EXT_H_
#define DIOPI_FUNCTIONS_EXT_H_

#include <diopi/diopirt.h>

/* out = input * rsqrt(mean(input^2 over normalized_shape) + eps) * weight (+ bias).
 * Semantics: dicp/dicp/vendor/AscendGraph/ext_ops.py:47-49. Accumulation is fp32
 * (dicp/test/model/llama/model.py:34-39 normalises in fp32). inv_rms (nullable) receives
 * rsqrt(mean+eps) per row as fp32 (or input dtype), shape = input.shape minus normalized dims.
 * weight / bias may be null. */
DIOPI_API diopiError_t diopiRMSNorm(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiTensorHandle_t inv_rms,
                                    diopiConstTensorHandle_t input, diopiSize_t normalized_shape,
                                    diopiConstTensorHandle_t weight, diopiConstTensorHandle_t bias, double eps);

/* Rotary position embedding, out and x of shape [..., head_dim], cos/sin broadcastable to
 * x after unsqueezing the head dim: [tokens, d/2] or [tokens, d] (or [tokens,1,d/2|d]).
 *   interleaved == false: half-split pairs (x[i], x[i+d/2])  -- ext_ops.py:24-33
 *   interleaved == true : adjacent pairs (x[2i], x[2i+1])     -- model.py:58-69 (complex multiply)
 *   conj: rotate by the negative angle (backward pass).
 * When cos/sin carry the full head_dim, the first d/2 entries of each row are used for
 * the half-split layout and entries 2i for the interleaved one. */
DIOPI_API diopiError_t diopiRotaryEmbedding(diopiContextHandle_t ctx, diopiTensorHandle_t out,
                                            diopiConstTensorHandle_t x, diopiConstTensorHandle_t cos,
                                            diopiConstTensorHandle_t sin, bool conj, bool interleaved);

/* out[dest_loc[i], :, :] = k[i, :, :]; bit-exact move. dest_loc is int32 or int64.
 * Nearest reference semantics: index_put on the leading dim (diopi_functions.yaml:2370-2382)
 * and the contiguous-range form ext_ops.py:146-149. */
DIOPI_API diopiError_t diopiDestIndexCopyKV(diopiContextHandle_t ctx, diopiTensorHandle_t out,
                                            diopiConstTensorHandle_t k, diopiConstTensorHandle_t dest_loc);

/* Decode attention, first half: attention_out[h, b_start_loc[b] + t] = q[b,h,:] . k[slot,h,:] / sqrt(d)
 * for t in [0, b_seq_len[b]), slot = b_loc[b, max_input_len - b_seq_len[b] + t] (right-aligned slot table).
 * q [batch, heads, d]; k [slots, kv_heads, d]; attention_out [heads, total_tokens] (fp32 or q dtype).
 * In all three decode entry points a b_seq_len[b] outside [0, max_input_len] is cut to that range (the table row
 * holds no more), and slots outside the pool are skipped, never dereferenced. q, k, v are float32, float16 or
 * bfloat16 with a contiguous head dimension; head rows of 128, 256 or 512 bytes at 16-byte aligned strides take the
 * streaming kernels, any other head size up to 1024 elements a plain kernel (one workgroup per sequence and head).
 * Semantics: the q.K^T/sqrt(d) step of ext_ops.py:100-133. */
DIOPI_API diopiError_t diopiTokenAttentionInference(diopiContextHandle_t ctx, diopiTensorHandle_t attention_out,
                                                    diopiConstTensorHandle_t q, diopiConstTensorHandle_t k,
                                                    diopiConstTensorHandle_t b_loc,
                                                    diopiConstTensorHandle_t b_start_loc,
                                                    diopiConstTensorHandle_t b_seq_len, int max_input_len);

/* Decode attention, second half: out[b,h,:] = softmax_t(logics[h, start_b + t]) . v[slot_t, h, :].
 * Semantics: the softmax / .V step of ext_ops.py:120-131. other_kv_index is accepted for
 * signature fidelity and ignored (it only pads vendor kernels upstream). */
DIOPI_API diopiError_t diopiTokenSoftmaxReduceVInference(diopiContextHandle_t ctx, diopiTensorHandle_t out,
                                                         diopiConstTensorHandle_t logics, diopiConstTensorHandle_t v,
                                                         diopiConstTensorHandle_t b_loc,
                                                         diopiConstTensorHandle_t b_start_loc,
                                                         diopiConstTensorHandle_t b_seq_len, int max_input_len,
                                                         int other_kv_index);

/* Prefill (context) causal attention over packed sequences:
 * q [total_tokens, heads, d], k/v [total_tokens, kv_heads, d]; sequence b occupies rows
 * [b_start_loc[b], b_start_loc[b] + b_seq_len[b]); out = softmax(q k^T / sqrt(d) + causal) v in fp32.
 * Semantics: ext_ops.py:62-87 (grouped kv heads via num_key_value_heads). */
DIOPI_API diopiError_t diopiContextAttentionInference(diopiContextHandle_t ctx, diopiTensorHandle_t out,
                                                      diopiConstTensorHandle_t q, diopiConstTensorHandle_t k,
                                                      diopiConstTensorHandle_t v,
                                                      diopiConstTensorHandle_t b_start_loc,
                                                      diopiConstTensorHandle_t b_seq_len, int max_input_len);

/* ---- extensions defined by this backend (no upstream precedent) ----------- */

/* Fused decode attention: both halves above in one pass over the paged KV pool
 * (split-KV partial softmax + merge), never materialising the logits.
 * Same arguments as the two-call form minus the logits tensor. ext_ops.py:100-133. */
DIOPI_API diopiError_t diopiTokenDecodeAttentionInference(diopiContextHandle_t ctx, diopiTensorHandle_t out,
                                                          diopiConstTensorHandle_t q, diopiConstTensorHandle_t k,
                                                          diopiConstTensorHandle_t v, diopiConstTensorHandle_t b_loc,
                                                          diopiConstTensorHandle_t b_start_loc,
                                                          diopiConstTensorHandle_t b_seq_len, int max_input_len);

/* The K row and the V row of every new token into their two pools in one launch: the same result, bit for bit, as
 * diopiDestIndexCopyKV(out_k, k, dest_loc) followed by diopiDestIndexCopyKV(out_v, v, dest_loc). The scatter of a
 * decode step moves a few hundred KiB and costs one launch latency per call; this halves it. The reference runs the two
 * calls (lightllm's destindex_copy_kv for K and for V). */
DIOPI_API diopiError_t diopiDestIndexCopyKVPair(diopiContextHandle_t ctx, diopiTensorHandle_t out_k,
                                                diopiConstTensorHandle_t k, diopiTensorHandle_t out_v,
                                                diopiConstTensorHandle_t v, diopiConstTensorHandle_t dest_loc);

/* diopiTokenDecodeAttentionInference for callers that cannot allocate (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): same arguments, same kernels, same result bit for bit, but the split-KV
 * partial results live in a 32 MiB device array inside the library instead of workspace from diopiRequireBuffer, and
 * the call makes no hipMalloc, hipFree or workspace request. It has no counterpart in the reference. Fails with a
 * clear error when batch x heads x splits x (2 + head_dim) x 4 bytes exceeds 32 MiB (splits = ceil(max_input_len /
 * 512), at most 64; batch 64 x 32 heads x head_dim 128 fits up to max_input_len 15872). Every call on a device
 * shares that device's array: calls that overlap on one device (two streams, two threads) race, and so do replays of
 * graphs that hold this call when they run at the same time on different streams (every graph recorded on a device
 * points at the same array). The array's device address is looked up by the first call of this function or of
 * diopiTokenDecodeAttentionInference on a device: make that first call eagerly, outside stream capture, before
 * recording this one into a graph. */
DIOPI_API diopiError_t diopiTokenDecodeAttentionInferenceNoAlloc(diopiContextHandle_t ctx, diopiTensorHandle_t out,
                                                                 diopiConstTensorHandle_t q, diopiConstTensorHandle_t k,
                                                                 diopiConstTensorHandle_t v, diopiConstTensorHandle_t b_loc,
                                                                 diopiConstTensorHandle_t b_start_loc,
                                                                 diopiConstTensorHandle_t b_seq_len, int max_input_len);

/* out[M,N] = input[M,K] @ (weight[N,K] (int8) * scale[N])^T + bias[N].
 * input/out bf16 or fp16; scale fp16/bf16/fp32 per output channel; bias nullable.
 * The int8 -> bf16/fp16 conversion happens while the MFMA operand tile is loaded; the
 * per-channel scale multiplies the fp32 accumulator. Absent from the whole reference. */
DIOPI_API diopiError_t diopiWeightOnlyInt8Linear(diopiContextHandle_t ctx, diopiTensorHandle_t out,
                                                 diopiConstTensorHandle_t input, diopiConstTensorHandle_t weight,
                                                 diopiConstTensorHandle_t scale, diopiConstTensorHandle_t bias);

/* out = silu(gate) * up, one pass (the SiLU-gated FFN's elementwise stage;
 * reference runs it as diopiSilu + diopiMul, diopi_functions.yaml:1767-1775,181-196). */
DIOPI_API diopiError_t diopiSiluMul(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t gate,
                                    diopiConstTensorHandle_t up);

/* out[..., F] = silu(input @ w_gate^T) * (input @ w_up^T): the SiLU-gated FFN's two projections and its
 * elementwise stage in one pass; gate and up never reach memory. weight is [2F, K] and holds w_gate [F, K] and
 * w_up [F, K] interleaved in blocks of 32 rows: rows [64 b, 64 b + 32) = w_gate[32 b : 32 b + 32],
 * rows [64 b + 32, 64 b + 64) = w_up[32 b : 32 b + 32] (a load-time permutation of the checkpoint, like stacking
 * q, k and v). F must be a multiple of 32. The reference model runs two linears, silu and mul
 * (dicp/test/model/llama/model.py:196-200). */
DIOPI_API diopiError_t diopiLinearSiluMul(diopiContextHandle_t ctx, diopiTensorHandle_t out,
                                          diopiConstTensorHandle_t input, diopiConstTensorHandle_t weight);

/* out[..., N] = input @ weight^T + bias, followed by diopiRotaryEmbedding on the first rotary_cols columns of out
 * viewed as heads of head_dim columns: the q and k heads of a stacked [q; k; v] projection come out rotated, v passes
 * through, and the rotary pass over q and k (read + write) disappears. cos / sin are [t, head_dim / 2] with t
 * dividing the rows of the flattened input (row r uses table row r % t, as diopiRotaryEmbedding does); conj and interleaved as in diopiRotaryEmbedding. With interleaved == true
 * (adjacent pairs, dicp/test/model/llama/model.py:58-69) and a large problem this is one GEMM launch; otherwise the
 * projection and the rotation run as two passes with the same result. A checkpoint in the half-split convention
 * (dicp/dicp/vendor/AscendGraph/ext_ops.py:24-33) can use the single-launch form after a load-time permutation of
 * the q and k weight rows of every head (row 2 i <- row i, row 2 i + 1 <- row i + head_dim / 2): q . k is
 * invariant under a permutation of the head dim applied to both. bias may be null. The reference model runs the
 * projections and the rotation as separate steps (model.py:108-160). */
DIOPI_API diopiError_t diopiLinearRotary(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input,
                                         diopiConstTensorHandle_t weight, diopiConstTensorHandle_t bias,
                                         diopiConstTensorHandle_t cos, diopiConstTensorHandle_t sin, int64_t rotary_cols,
                                         int64_t head_dim, bool conj, bool interleaved);

#endif /* DIOPI_FUNCTIONS_EXT_H_ */
