/* TEST INFRASTRUCTURE — the parity checker, never the product.
 *
 * CPU restatement of TinyTorch's scaled-dot-product attention as its CPU path computes it in fp32
 * (reference src/Function/FuncNNLayer.h:231-266 and the CPU ops it calls).  Only tests/, the smoke check and the
 * cpu_baseline leg of bench.py may load this library; the shipped library (include/ttsdpa.h) never does.
 *
 * Pinning status (tests/test_oracle.py):
 *   oracle_sdpa_f32            pinned: reference KATs (test/test_function.cpp:393-419), bit-exact against the compiled
 *                              reference (oracle/_ref) and against fixtures written from it, fp64 closed form,
 *                              invariants (causal row 0 == v[0], rows of P sum to 1, uniform-K running mean).
 *   oracle_sdpa_backward_f32   the reference has no attention (or matmul) backward to compare with: pinned by central
 *                              differences of an independent float64 forward, by closed forms (one key; zero
 *                              queries) and by invariants (columns of dK sum to 0, GQA == repeated K/V summed over
 *                              the group) in tests/test_oracle_backward.py.
 *   oracle_round_bf16 / _f16   pinned: bit-exact against the reference's own casts over a sweep that includes
 *                              ties, subnormals, overflow, inf and NaN; and against numpy float16 casts.
 *   oracle_randn               not a reference function (the harness's own PRNG); pinned by moments and by a
 *                              pure-numpy restatement of the same counter-based construction.
 */
#ifndef SDPA_ORACLE_H
#define SDPA_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { ORACLE_MASK_NONE = 0, ORACLE_MASK_BOOL = 1, ORACLE_MASK_FLOAT = 2 };
enum { ORACLE_F32 = 0, ORACLE_F16 = 1, ORACLE_BF16 = 2 }; /* same numbering as the reference DType enum */

/* fp32 -> 16-bit pattern, round-to-nearest-even. */
uint16_t oracle_f32_to_bf16_bits(float x);
uint16_t oracle_f32_to_f16_bits(float x);
float oracle_bf16_bits_to_f32(uint16_t b);
float oracle_f16_bits_to_f32(uint16_t b);
/* Array forms: round `in` to dtype (ORACLE_F16/ORACLE_BF16; ORACLE_F32 copies); writes the fp32 value of the rounded
 * number to out_f32 (may be NULL) and the bit pattern to out_bits (may be NULL). */
void oracle_round_array(const float* in, float* out_f32, uint16_t* out_bits, int64_t n, int dtype);
void oracle_bits_to_f32_array(const uint16_t* in, float* out, int64_t n, int dtype);

/* Counter-based N(0,1) generator: element i of (seed, stream) never depends on n or on the thread count.
 * out[i] = (float)(mul * z_i). */
void oracle_randn(uint64_t seed, uint64_t stream, int64_t n, float mul, float* out, int nthreads);

/* The reference CPU path, fp32, for q [B,Hq,L,D], k/v [B,Hkv,S,D] (all dense row-major) -> out [B,Hq,L,D].
 * kv head of query head h is h / (Hq/Hkv) (what op::repeatInterleave(k, Hq/Hkv, 1) feeds the reference).
 * causal: top-left aligned lower triangle, key j visible to query i iff j <= i (tril(ones(L,S), 0)).
 * mask: NULL, or [L,S] uint8 (ORACLE_MASK_BOOL: 0 = hidden) or [L,S] float (ORACLE_MASK_FLOAT: added to the scores).
 * nthreads > 1 spreads (batch, head) slices over threads; every slice is computed by the same sequential code, so
 * the result does not depend on nthreads.  Returns 0, or -1 on bad arguments / out of memory. */
int oracle_sdpa_f32(const float* q, const float* k, const float* v, float* out, int64_t B, int64_t Hq, int64_t Hkv,
                    int64_t L, int64_t S, int64_t D, int causal, float scale, int mask_kind, const void* mask,
                    int nthreads);

/* Same arithmetic for a subset of the (batch, head, query-row) triples: rows[3*i..3*i+2] = (b, h, l);
 * out is [nrows, D].  A row's result does not depend on the other rows, so this equals the matching rows of
 * oracle_sdpa_f32 bit for bit. */
int oracle_sdpa_rows_f32(const float* q, const float* k, const float* v, float* out, int64_t B, int64_t Hq,
                         int64_t Hkv, int64_t L, int64_t S, int64_t D, int causal, float scale, const int64_t* rows,
                         int64_t nrows, int nthreads);

/* Gradients of oracle_sdpa_f32's output with respect to q, k, v for an upstream gradient dout [B,Hq,L,D]: the chain
 * rule through scores = scale * Q K^T + bias, P = softmax(scores), out = P V, accumulated in double and rounded to
 * fp32 once.  dq [B,Hq,L,D]; dk, dv [B,Hkv,S,D] sum over the query heads that share a kv head.  Same causal / mask
 * arguments as the forward; D <= 1024.  S == 0 gives dq = 0 and writes nothing to dk / dv. */
int oracle_sdpa_backward_f32(const float* q, const float* k, const float* v, const float* dout, float* dq, float* dk,
                             float* dv, int64_t B, int64_t Hq, int64_t Hkv, int64_t L, int64_t S, int64_t D,
                             int causal, float scale, int mask_kind, const void* mask, int nthreads);

/* Row-wise neighbour ops (fused_oracle.c): rmsNorm, fusedAddRmsNorm (in place), siluMul, softmax / logSoftmax over
 * [outer, dim, inner].  dtype: 0 fp32, 1 fp16, 2 bf16 = the element type the reference would store in. */
void oracle_rms_norm(const float* x, const float* w, float* out, int64_t rows, int64_t dim, float eps, int dtype);
void oracle_fused_add_rms_norm(float* input, float* residual, const float* w, int64_t rows, int64_t dim, float eps,
                               int dtype);
void oracle_silu_mul(const float* x, float* out, int64_t rows, int64_t d, int dtype);
void oracle_softmax(const float* x, float* out, int64_t outer, int64_t dim, int64_t inner, int log_form, int dtype);
/* out[M,N] = bias[N] (or 0) + x[M,K] . w[N,K]^T, the reference's gemm loop order. */
void oracle_linear(const float* x, const float* w, const float* bias, float* out, int64_t M, int64_t N, int64_t K,
                   int dtype);
/* softmax / logSoftmax backward over [outer, dim, inner] from the upstream gradient g and the forward's output y. */
void oracle_softmax_backward(const float* g, const float* y, float* out, int64_t outer, int64_t dim, int64_t inner,
                             int log_form, int dtype);
/* out[M,N] = bias[N] (or 0) + op(a) . op(b): a is [M,K], or [K,M] with trans_a; b is [K,N], or [N,K] with trans_b. */
void oracle_matmul(const float* a, const float* b, const float* bias, float* out, int64_t M, int64_t N, int64_t K,
                   int trans_a, int trans_b, int dtype);

#ifdef __cplusplus
}
#endif
#endif
