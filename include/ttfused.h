/*
 * ttfused — the row-wise inference ops that sit next to attention in a TinyTorch transformer block, for MI355X
 * (gfx950), behind a plain C ABI in the same library as ttsdpa (libttsdpa.so).
 *
 * Each entry point replaces one device op of the reference (its DEFINE_OP slot for {CUDA, dtype}); the binding is the
 * same as for attention: the op implementation passes raw device pointers, sizes and its current stream.
 * All tensors are dense and row-major, as the reference's implementations require (they index dataPtr() directly).
 * Arithmetic is fp32 whatever the element type; results are rounded once to the element type.
 * Every call enqueues on `stream` (a hipStream_t; NULL = the default stream), allocates nothing and does not
 * synchronise.  Return values are ttsdpa_status codes (include/ttsdpa.h); dtype is a ttsdpa_dtype.
 */
#ifndef TTFUSED_H_
#define TTFUSED_H_

#include <stddef.h>
#include <stdint.h>

#include "ttsdpa.h"

#ifdef __cplusplus
extern "C" {
#endif

/* out[r, :] = x[r, :] / sqrt(mean(x[r, :]^2) + eps) * weight  — op::rmsNorm over the last axis (reference
 * src/Operation/OpNNLayer.h:60-61; device kernels src/Operation/OpNNLayerCuda.cuh:253-345, 487-536; CPU
 * src/Operation/OpNNLayerCpu.h:219-233).  x, out: [rows, dim]; weight: [dim] or NULL (no affine).  out may alias x. */
int ttfused_rms_norm(int dtype, const void* x, const void* weight, void* out, int64_t rows, int64_t dim, float eps,
                     void* stream);

/* In place on both tensors — op::fusedAddRmsNorm (reference src/Operation/OpFused.h:16-22; device kernel
 * src/Operation/OpFusedCuda.cuh:104-146; CPU src/Operation/OpFusedCpu.h:44-74):
 *   residual <- input + residual;  input <- residual / sqrt(mean(residual^2) + eps) * weight
 * where the mean uses the unrounded sum and the normalised row is computed from the stored (rounded) residual.
 * input, residual: [rows, dim]; weight: [dim] (required). */
int ttfused_add_rms_norm(int dtype, void* input, void* residual, const void* weight, int64_t rows, int64_t dim,
                         float eps, void* stream);

/* out[r, j] = silu(x[r, j]) * x[r, d + j], silu(a) = a / (1 + exp(-a)) — op::siluMul (reference
 * src/Operation/OpFused.h:14-19; device kernels src/Operation/OpFusedCuda.cuh:16-102; CPU
 * src/Operation/OpFusedCpu.h:16-42).  x: [rows, 2*d] (gate half first, up half second); out: [rows, d]. */
int ttfused_silu_mul(int dtype, const void* x, void* out, int64_t rows, int64_t d, void* stream);

/* softmax (log_form == 0) or logSoftmax (log_form != 0) along the middle axis of x viewed as [outer, dim, inner] —
 * op::softmax / op::logSoftmax over any axis (reference src/Operation/OpNNLayer.h:44-50; device kernels
 * src/Operation/OpNNLayerCuda.cuh:36-145; CPU src/Operation/OpNNLayerCpu.h:16-76, 111-125).  The last axis is
 * inner == 1.  out may alias x. */
int ttfused_softmax(int dtype, const void* x, void* out, int64_t outer, int64_t dim, int64_t inner, int log_form,
                    void* stream);

/* Backward of softmax / logSoftmax over the same [outer, dim, inner] view (reference op::softmaxBackward /
 * op::logSoftmaxBackward, src/Operation/OpNNLayerCpu.h:79-109, 123-150; called by FuncSoftmax / FuncLogSoftmax::backward,
 * src/Function/FuncActivation.h:53-61, 76-84): from the upstream gradient `grad` and the forward's `output`,
 *   softmax:    out_j = output_j * (grad_j - sum_t output_t * grad_t)
 *   logSoftmax: out_j = grad_j - exp(output_j) * sum_t grad_t
 * with the sums in fp32 and one rounding of the result.  out may alias grad. */
int ttfused_softmax_backward(int dtype, const void* grad, const void* output, void* out, int64_t outer, int64_t dim,
                             int64_t inner, int log_form, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TTFUSED_H_ */
