/*
 * DIOPI operator entry points exported by libdiopi_impl.so (MI355X backend).
 *
 * Each declaration names the reference call site whose argument order it
 * follows: the `interface:` lines of
 *   dipu/scripts/autogen_diopi_wrapper/diopi_functions.yaml
 * (abbreviated "yaml:LINE" below). Pointer-ness of scalars/handles follows the
 * wrapper generator, dipu/scripts/autogen_diopi_wrapper/autogen_diopi_wrapper.py:878-961:
 * tensors are opaque handles, at::Scalar becomes `const diopiScalar_t*`,
 * optional tensors become nullable handles, int lists become diopiSize_t by value.
 *
 * Convention: (ctx, outputs..., inputs..., attributes...). Every function
 * enqueues on diopiGetStream(ctx), never synchronises, and returns diopiSuccess
 * or an error whose text diopiGetLastErrorString() reports
 * (autogen_diopi_wrapper.py:1001).
 */
#ifndef DIOPI_FUNCTIONS_H_
#define DIOPI_FUNCTIONS_H_

#include <diopi/diopirt.h>

/* autogen_diopi_wrapper.py:1001 */
DIOPI_API const char* diopiGetLastErrorString(void);

/* ---- elementwise arithmetic -------------------------------------------- */
/* out = input + alpha * other, broadcasting, out dtype = promoted dtype. yaml:49-63 */
DIOPI_API diopiError_t diopiAdd(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input,
                                diopiConstTensorHandle_t other, const diopiScalar_t* alpha);
/* yaml:40-47 */
DIOPI_API diopiError_t diopiAddInp(diopiContextHandle_t ctx, diopiTensorHandle_t input, diopiConstTensorHandle_t other,
                                   const diopiScalar_t* alpha);
/* yaml:31-32 */
DIOPI_API diopiError_t diopiAddScalar(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input,
                                      const diopiScalar_t* other, const diopiScalar_t* alpha);
/* yaml:34-38 */
DIOPI_API diopiError_t diopiAddInpScalar(diopiContextHandle_t ctx, diopiTensorHandle_t input,
                                         const diopiScalar_t* other, const diopiScalar_t* alpha);
/* out = input - alpha * other. yaml:1374 (rsub passes operands swapped), yaml:72-80 */
DIOPI_API diopiError_t diopiSub(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input,
                                diopiConstTensorHandle_t other, const diopiScalar_t* alpha);
DIOPI_API diopiError_t diopiSubScalar(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input,
                                      const diopiScalar_t* other, const diopiScalar_t* alpha);
/* yaml:181-196 */
DIOPI_API diopiError_t diopiMul(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input,
                                diopiConstTensorHandle_t other);
/* yaml:169-179 */
DIOPI_API diopiError_t diopiMulInp(diopiContextHandle_t ctx, diopiTensorHandle_t input, diopiConstTensorHandle_t other);
/* yaml:159-167 */
DIOPI_API diopiError_t diopiMulScalar(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input,
                                      const diopiScalar_t* other);
DIOPI_API diopiError_t diopiMulInpScalar(diopiContextHandle_t ctx, diopiTensorHandle_t input,
                                         const diopiScalar_t* other);
/* yaml:94-151; only RoundModeNone/Floor/Trunc on floating outputs */
DIOPI_API diopiError_t diopiDiv(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input,
                                diopiConstTensorHandle_t other, diopiRoundMode_t rounding_mode);
DIOPI_API diopiError_t diopiDivScalar(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input,
                                      const diopiScalar_t* other, diopiRoundMode_t rounding_mode);

/* ---- unary ---------------------------------------------------------------- */
/* x * sigmoid(x). yaml:1767-1775, in-place yaml:1785-1786 */
DIOPI_API diopiError_t diopiSilu(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input);
DIOPI_API diopiError_t diopiSiluInp(diopiContextHandle_t ctx, diopiTensorHandle_t input);
/* yaml:1950-1953 */
DIOPI_API diopiError_t diopiSigmoid(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input);
/* yaml:1177-1185 */
DIOPI_API diopiError_t diopiRsqrt(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input);
/* yaml:781-791 */
DIOPI_API diopiError_t diopiNeg(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input);
/* yaml:1733-1753 */
DIOPI_API diopiError_t diopiSin(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input);
DIOPI_API diopiError_t diopiCos(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input);
/* yaml:1503-1508 */
DIOPI_API diopiError_t diopiExp(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input);
/* input ** exponent (scalar exponent). yaml:1306-1318 */
DIOPI_API diopiError_t diopiPow(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input,
                                const diopiScalar_t* exponent);
/* yaml:28-29 */
DIOPI_API diopiError_t diopiFill(diopiContextHandle_t ctx, diopiTensorHandle_t input, const diopiScalar_t* value);

/* ---- reductions over rows ------------------------------------------------- */
/* softmax along `dim` (any dim, negative allowed), out dtype = in dtype. yaml:1290-1292 */
DIOPI_API diopiError_t diopiSoftmax(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input,
                                    int64_t dim);
/* mean over the listed dims (keepdim decided by out's shape). yaml:830-842 */
DIOPI_API diopiError_t diopiMean(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input,
                                 diopiSize_t dim);

/* ---- data movement -------------------------------------------------------- */
/* dest <- src with broadcasting, arbitrary strides and dtype conversion.
 * yaml:2969-2973 and dipu/torch_dipu/csrc_dipu/aten/ops/DIPUCopy.hpp:633-655 */
DIOPI_API diopiError_t diopiCopyInp(diopiContextHandle_t ctx, diopiConstTensorHandle_t src, diopiTensorHandle_t dest);
/* out = cat(tensors, dim). yaml:1418-1424 */
DIOPI_API diopiError_t diopiCat(diopiContextHandle_t ctx, diopiTensorHandle_t out,
                                const diopiConstTensorHandle_t* tensors, int64_t num_inputs, int64_t dim);
/* input[indices...] = values (or += when accumulate). yaml:2370-2382;
 * this backend implements the dense-prefix form used by KV caches:
 * `indices_counts` integer index tensors addressing the leading dims. */
DIOPI_API diopiError_t diopiIndexPutInp(diopiContextHandle_t ctx, diopiTensorHandle_t input,
                                        diopiConstTensorHandle_t values, diopiConstTensorHandle_t* indices,
                                        int64_t indices_counts, bool accumulate);

/* ---- selection, masks, comparisons, gathers (what a decoder layer written in primitive aten ops needs) ---- */
/* out = condition ? input : other, all three broadcast to out. yaml:1566-1571 */
DIOPI_API diopiError_t diopiWhere(diopiContextHandle_t ctx, diopiTensorHandle_t out,
                                  diopiConstTensorHandle_t condition, diopiConstTensorHandle_t input,
                                  diopiConstTensorHandle_t other);
/* out = mask ? value : input; value is a 0-d device tensor or a Scalar. yaml:1432-1453 */
DIOPI_API diopiError_t diopiMaskedFill(diopiContextHandle_t ctx, diopiTensorHandle_t out,
                                       diopiConstTensorHandle_t input, diopiConstTensorHandle_t mask,
                                       diopiConstTensorHandle_t value);
DIOPI_API diopiError_t diopiMaskedFillInp(diopiContextHandle_t ctx, diopiTensorHandle_t input,
                                          diopiConstTensorHandle_t mask, diopiConstTensorHandle_t value);
DIOPI_API diopiError_t diopiMaskedFillScalar(diopiContextHandle_t ctx, diopiTensorHandle_t out,
                                             diopiConstTensorHandle_t input, diopiConstTensorHandle_t mask,
                                             const diopiScalar_t* value);
DIOPI_API diopiError_t diopiMaskedFillInpScalar(diopiContextHandle_t ctx, diopiTensorHandle_t input,
                                                diopiConstTensorHandle_t mask, const diopiScalar_t* value);
/* lower / upper triangle of the last two dims, zero elsewhere. yaml:1191-1197, 2505-2516 */
DIOPI_API diopiError_t diopiTril(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input,
                                 int64_t diagonal);
DIOPI_API diopiError_t diopiTriu(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input,
                                 int64_t diagonal);
DIOPI_API diopiError_t diopiTriuInp(diopiContextHandle_t ctx, diopiTensorHandle_t input, int64_t diagonal);
/* out[i] = start + i*step for the elements the caller sized out to. yaml:2341-2347 */
DIOPI_API diopiError_t diopiArange(diopiContextHandle_t ctx, diopiTensorHandle_t out, const diopiScalar_t* start,
                                   const diopiScalar_t* end, const diopiScalar_t* step);
/* out = input.index_select(dim, index), index 1-d int32/int64. yaml:1926-1933 */
DIOPI_API diopiError_t diopiIndexSelect(diopiContextHandle_t ctx, diopiTensorHandle_t out,
                                        diopiConstTensorHandle_t input, int64_t dim, diopiConstTensorHandle_t index);
/* out[i][j][k] = input[index[i][j][k]][j][k] (for dim 0), out shaped like index. yaml:1923-1924 */
DIOPI_API diopiError_t diopiGather(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input,
                                   int64_t dim, diopiConstTensorHandle_t index);
/* out (normally bool) = input <cmp> other, broadcasting; Scalar forms take the right operand as a Scalar.
 * yaml:409-420 eq, :443-454 lt, :466-477 ne, :489-500 ge, :512-523 gt, :535-546 le */
DIOPI_API diopiError_t diopiEq(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input,
                               diopiConstTensorHandle_t other);
DIOPI_API diopiError_t diopiEqScalar(diopiContextHandle_t ctx, diopiTensorHandle_t out,
                                     diopiConstTensorHandle_t input, const diopiScalar_t* other);
DIOPI_API diopiError_t diopiNe(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input,
                               diopiConstTensorHandle_t other);
DIOPI_API diopiError_t diopiNeScalar(diopiContextHandle_t ctx, diopiTensorHandle_t out,
                                     diopiConstTensorHandle_t input, const diopiScalar_t* other);
DIOPI_API diopiError_t diopiLt(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input,
                               diopiConstTensorHandle_t other);
DIOPI_API diopiError_t diopiLtScalar(diopiContextHandle_t ctx, diopiTensorHandle_t out,
                                     diopiConstTensorHandle_t input, const diopiScalar_t* other);
DIOPI_API diopiError_t diopiLe(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input,
                               diopiConstTensorHandle_t other);
DIOPI_API diopiError_t diopiLeScalar(diopiContextHandle_t ctx, diopiTensorHandle_t out,
                                     diopiConstTensorHandle_t input, const diopiScalar_t* other);
DIOPI_API diopiError_t diopiGt(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input,
                               diopiConstTensorHandle_t other);
DIOPI_API diopiError_t diopiGtScalar(diopiContextHandle_t ctx, diopiTensorHandle_t out,
                                     diopiConstTensorHandle_t input, const diopiScalar_t* other);
DIOPI_API diopiError_t diopiGe(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input,
                               diopiConstTensorHandle_t other);
DIOPI_API diopiError_t diopiGeScalar(diopiContextHandle_t ctx, diopiTensorHandle_t out,
                                     diopiConstTensorHandle_t input, const diopiScalar_t* other);

/* ---- dense contractions (MFMA for bf16/fp16, fp32 FMA tiles otherwise) ---- */
/* out[M,N] = input[M,K] @ mat2[K,N]. yaml:1829-1837 */
DIOPI_API diopiError_t diopiMm(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input,
                               diopiConstTensorHandle_t mat2);
/* out[B,M,N] = input[B,M,K] @ mat2[B,K,N]. yaml:1755-1765 */
DIOPI_API diopiError_t diopiBmm(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input,
                                diopiConstTensorHandle_t mat2);
/* torch.matmul semantics (1-D/2-D/batched with broadcasting). yaml:1852-1893 */
DIOPI_API diopiError_t diopiMatmul(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input,
                                   diopiConstTensorHandle_t other);
/* out = beta*input + alpha*(mat1 @ mat2). yaml:594-597 */
DIOPI_API diopiError_t diopiAddmm(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input,
                                  diopiConstTensorHandle_t mat1, diopiConstTensorHandle_t mat2,
                                  const diopiScalar_t* beta, const diopiScalar_t* alpha);
/* out = beta*input + alpha*(batch1 @ batch2). yaml:1534-1548 */
DIOPI_API diopiError_t diopiBaddbmm(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input,
                                    diopiConstTensorHandle_t batch1, diopiConstTensorHandle_t batch2, double beta,
                                    double alpha);
/* out[...,N] = input[...,K] @ weight[N,K]^T + bias[N] (bias nullable). yaml:902-909 */
DIOPI_API diopiError_t diopiLinear(diopiContextHandle_t ctx, diopiTensorHandle_t out, diopiConstTensorHandle_t input,
                                   diopiConstTensorHandle_t weight, diopiConstTensorHandle_t bias);

#endif /* DIOPI_FUNCTIONS_H_ */
