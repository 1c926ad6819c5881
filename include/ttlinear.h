/*
 * ttlinear — the linear layer y = x . w^T + bias for MI355X (gfx950) behind a plain C ABI, in the same library as
 * ttsdpa (libttsdpa.so): the projections on either side of attention (QKV, output, MLP).
 *
 * Replaces, for this call shape, the reference's op::matmul(input, weight, false, true, bias) behind
 * function::linear (reference src/Function/FuncNNLayer.h:14-19, 270-272; host side src/Operation/OpLinalg.cpp:244-276;
 * its device GEMM is a cuBLAS call, src/Operation/OpLinalgCuda.cuh:239-293; CPU loop src/Operation/OpLinalgCpu.h:119-150).
 * The op implementation passes raw device pointers, sizes, leading dimensions and its current stream.
 */
#ifndef TTLINEAR_H_
#define TTLINEAR_H_

#include <stddef.h>
#include <stdint.h>

#include "ttsdpa.h"

#ifdef __cplusplus
extern "C" {
#endif

enum ttlinear_route {
  TTLINEAR_ROUTE_NONE = 0,   /* empty output */
  TTLINEAR_ROUTE_MFMA = 1,   /* K a multiple of 64 (fp16/bf16) or 32 (fp32), 16-byte aligned rows, N a multiple of 4:
                                MFMA kernel, fp32 accumulation (fp32 tensors: full fp32 products) */
  TTLINEAR_ROUTE_GENERAL = 2 /* everything else (other K, unaligned rows): fp32 arithmetic on the vector ALUs */
};

/* out[m, n] = bias[n] + sum_k x[m, k] * w[n, k]   (m < M, n < N, k < K)
 * x: [M, K] with row stride ldx elements; w: [N, K] (the layout of a Linear layer's weight) with row stride ldw;
 * bias: [N] or NULL; out: [M, N] with row stride ldo.  dtype is a ttsdpa_dtype shared by all four tensors.
 * Accumulation is fp32 starting from the bias (the reference writes the bias into C and accumulates onto it), one
 * rounding to the element type at the end.  K == 0 yields the bias (or zeros).
 * Enqueues on `stream` (a hipStream_t; NULL = the default stream); no allocation, no synchronisation.
 * Returns a ttsdpa_status code, or a positive hipError_t. */
int ttlinear_forward(int dtype, const void* x, const void* w, const void* bias, void* out, int64_t M, int64_t N,
                     int64_t K, int64_t ldx, int64_t ldw, int64_t ldo, void* stream);

/* Validate the arguments and report the kernel ttlinear_forward would pick (enum ttlinear_route).  Launches nothing. */
int ttlinear_plan(int dtype, const void* x, const void* w, const void* bias, const void* out, int64_t M, int64_t N,
                  int64_t K, int64_t ldx, int64_t ldw, int64_t ldo, int* route);

/* out[m, n] = bias[n] + sum_k A(m, k) * B(k, n) with the reference's transpose flags — op::matmul(a, b, transA, transB,
 * bias) for 2-D operands (reference src/Operation/OpLinalgCpu.h:119-150: a is [M, K], or [K, M] with transA; b is [K, N], or
 * [N, K] with transB).  (false, true) is ttlinear_forward; FuncLinear::backward (reference
 * src/Function/FuncNNLayer.h:20-33) uses the other two that matter: (false, false) for the input gradient
 * dy[M, N] . w[N, K], and (true, false) for the weight gradient dy^T . x.  lda / ldb / ldo are row strides in elements.
 * fp16 / bf16 operands stored contraction-major are read in place by the matrix-core kernel (K a multiple of 64, N a
 * multiple of 4, 16-byte aligned operands with leading dimensions that are multiples of 8, a contraction-major operand's
 * row count a multiple of 8): no scratch is used then and workspace may be NULL.
 * workspace: ttlinear_matmul_workspace_bytes() bytes of device scratch, 256-byte aligned — for fp32 the MFMA route first
 * makes dense row-major copies of the operands that are stored contraction-major; with less (or NULL), or for shapes the
 * MFMA kernels do not take, the vector-ALU kernel reads the operands in place.  Same return codes as ttlinear_forward. */
size_t ttlinear_matmul_workspace_bytes(int dtype, int64_t M, int64_t N, int64_t K, int trans_a, int trans_b);
int ttlinear_matmul(int dtype, const void* a, const void* b, const void* bias, void* out, int64_t M, int64_t N, int64_t K,
                    int trans_a, int trans_b, int64_t lda, int64_t ldb, int64_t ldo, void* workspace,
                    size_t workspace_bytes, void* stream);

/* op::matmul with batch dimensions (reference src/Operation/OpLinalg.cpp:107-223: leading dimensions of the two
 * operands broadcast against each other; its device path is a strided-batched or pointer-array GEMM, its CPU path a
 * loop over the batch with per-operand offsets, :205-223).  The batch is described as up to TTLINEAR_MAX_BATCH_DIMS
 * dimensions batch_shape[0..nbatch_dims) with element strides a_batch_stride[d] / b_batch_stride[d] (0 broadcasts the
 * operand along d); batch entry i of the output, numbered row-major over batch_shape, starts at out + i * out_batch_stride.
 * Every batch entry is one ttlinear_matmul of the same M, N, K, flags and leading dimensions, enqueued in order on
 * `stream`; the workspace (ttlinear_matmul_workspace_bytes of one entry) is shared by the entries.  bias ([N] or NULL)
 * joins every entry. */
#define TTLINEAR_MAX_BATCH_DIMS 8
int ttlinear_matmul_batched(int dtype, const void* a, const void* b, const void* bias, void* out, int64_t M, int64_t N,
                            int64_t K, int trans_a, int trans_b, int64_t lda, int64_t ldb, int64_t ldo, int nbatch_dims,
                            const int64_t* batch_shape, const int64_t* a_batch_stride, const int64_t* b_batch_stride,
                            int64_t out_batch_stride, void* workspace, size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TTLINEAR_H_ */
