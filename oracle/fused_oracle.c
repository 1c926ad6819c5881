/*
 * TEST INFRASTRUCTURE — not part of the product.  Nothing under tinytorch_amd/ may call this.
 *
 * CPU restatement of the row-wise inference ops that sit next to attention in the reference: rmsNorm,
 * fusedAddRmsNorm, siluMul, softmax / logSoftmax, and the linear layer.  All tensors are fp32 arrays here; `dtype` (0 fp32, 1 fp16,
 * 2 bf16) says where the reference rounds to its element type T: inputs are expected to hold T-representable values,
 * intermediate stores to T tensors and the results are rounded with the same casts as the attention oracle.
 * Arithmetic between those points is fp32 — the reference's CPU path for fp32 tensors, and its device kernels
 * (which convert every element to float) for 16-bit tensors.
 *
 * Pinning:
 *   oracle_rms_norm            reference KAT test/test_function.cpp:385-391; oracle/_ref (function::rmsNorm) bit-exact
 *                              in fp32 on random rows
 *   oracle_fused_add_rms_norm  no KAT in the reference; oracle/_ref (op::fusedAddRmsNorm) bit-exact in fp32; the
 *                              identity fusedAddRmsNorm(x, r, w) == rmsNorm(x + r, w) with residual == x + r
 *   oracle_silu_mul            reference KAT for silu test/test_function.cpp:139-143 (up = 1); oracle/_ref
 *                              (op::siluMul) bit-exact in fp32
 *   oracle_linear              reference KAT test/test_function.cpp:234-241; oracle/_ref (function::linear) bit-exact
 *                              in fp32; fp64 closed form
 *   oracle_softmax_backward    oracle/_ref (op::softmaxBackward / op::logSoftmaxBackward, every axis) bit-exact in fp32;
 *                              central differences of the fp64 forward; rows of the softmax gradient sum to 0
 *   oracle_matmul              oracle/_ref (op::matmul with every transpose flag pair, with and without bias) bit-exact in
 *                              fp32; fp64 closed form; (false, true) == oracle_linear
 *   oracle_softmax             reference KATs test/test_function.cpp:147-176; oracle/_ref (function::softmax /
 *                              logSoftmax, every axis) bit-exact in fp32; rows sum to 1
 */
#include <math.h>
#include <stdint.h>

#include "sdpa_oracle.h"

static float round_t(float x, int dtype) {
  if (dtype == 1) return oracle_f16_bits_to_f32(oracle_f32_to_f16_bits(x));
  if (dtype == 2) return oracle_bf16_bits_to_f32(oracle_f32_to_bf16_bits(x));
  return x;
}

/* reference src/Operation/OpNNLayerCpu.h:219-233 (normOpCpuImplDetail, RMSNorm branch): sequential sum of squares,
 * divided by dim, invRms = 1 / sqrt(meanSquare + eps), normed = x * invRms, then *= weight when given.
 * 16-bit: float accumulation and one rounding of the result (device kernel, src/Operation/OpNNLayerCuda.cuh:253-299). */
void oracle_rms_norm(const float* x, const float* w, float* out, int64_t rows, int64_t dim, float eps, int dtype) {
  for (int64_t i = 0; i < rows; i++) {
    const float* src = x + i * dim;
    float* dst = out + i * dim;
    float ms = 0.f;
    for (int64_t j = 0; j < dim; j++) ms += src[j] * src[j];
    ms /= (float)dim;
    const float inv = 1.f / sqrtf(ms + eps);
    for (int64_t j = 0; j < dim; j++) {
      float normed = src[j] * inv;
      if (w) normed *= w[j];
      dst[j] = round_t(normed, dtype);
    }
  }
}

/* reference src/Operation/OpFusedCpu.h:44-74 (fusedAddRmsNormOpCpuImpl), in place on both tensors:
 * r = input + residual in float; residual <- T(r); sumSq += r * r (the unrounded r);
 * invRms = 1 / sqrt(sumSq / dim + eps); input <- T(float(residual) * invRms * float(weight)). */
void oracle_fused_add_rms_norm(float* input, float* residual, const float* w, int64_t rows, int64_t dim, float eps,
                               int dtype) {
  for (int64_t row = 0; row < rows; row++) {
    float* in = input + row * dim;
    float* res = residual + row * dim;
    float sum_sq = 0.f;
    for (int64_t i = 0; i < dim; i++) {
      float r = in[i] + res[i];
      res[i] = round_t(r, dtype);
      sum_sq += r * r;
    }
    const float inv = 1.f / sqrtf(sum_sq / (float)dim + eps);
    for (int64_t i = 0; i < dim; i++) in[i] = round_t(res[i] * inv * w[i], dtype);
  }
}

/* reference src/Operation/OpFusedCpu.h:16-42 (siluMulOpCpuImpl): rows of 2*d elements, gate = first half, up = second
 * half, out = silu(gate) * up with silu(a) = a / (1 + exp(-a)) (src/Operation/OpElemWiseCpu.h:123-128). */
void oracle_silu_mul(const float* x, float* out, int64_t rows, int64_t d, int dtype) {
  for (int64_t i = 0; i < rows; i++)
    for (int64_t j = 0; j < d; j++) {
      const float g = x[i * 2 * d + j], u = x[i * 2 * d + d + j];
      const float s = g / (1.0f + expf(-g));
      out[i * d + j] = round_t(s * u, dtype);
    }
}

/* reference src/Operation/OpNNLayerCpu.h:16-65 (softmaxForwardCpuImpl): for every (outer, inner) column of the axis,
 * maximum from -FLT_MAX, e = exp(x - max) stored and summed in order, then softmax: e * (float)(1.0 / sum);
 * logSoftmax: x - max - log(sum). */
void oracle_softmax(const float* x, float* out, int64_t outer, int64_t dim, int64_t inner, int log_form, int dtype) {
  for (int64_t o = 0; o < outer; o++)
    for (int64_t i = 0; i < inner; i++) {
      const int64_t base = o * dim * inner + i;
      float mx = -3.402823466e+38f;
      for (int64_t d = 0; d < dim; d++) {
        float v = x[base + d * inner];
        if (v > mx) mx = v;
      }
      float sum = 0.f;
      for (int64_t d = 0; d < dim; d++) {
        float e = expf(x[base + d * inner] - mx);
        out[base + d * inner] = e;
        sum += e;
      }
      if (!log_form) {
        const float inv = (float)(1.0 / (double)sum);
        for (int64_t d = 0; d < dim; d++) out[base + d * inner] = round_t(out[base + d * inner] * inv, dtype);
      } else {
        const float ls = logf(sum);
        for (int64_t d = 0; d < dim; d++) out[base + d * inner] = round_t(x[base + d * inner] - mx - ls, dtype);
      }
    }
}

/* reference src/Operation/OpLinalgCpu.h:119-150 (gemmCpuImpl with transA = false, transB = true, as function::linear
 * calls it, src/Function/FuncNNLayer.h:14-19): C starts as the bias broadcast over the rows (or zeros), then
 * c[i][j] += a[i][p] * b[j][p] in i, p, j order, all in fp32; `dtype` rounds the result once (16-bit tensors: fp32
 * accumulation as in the device GEMM).  Pinned by the reference KAT test/test_function.cpp:234-241, bit-exact against
 * oracle/_ref (function::linear) in fp32, and the fp64 closed form. */
/* reference src/Operation/OpNNLayerCpu.h:79-109 (softmax) and 123-150 (logSoftmax): sequential fp32 sum over the axis,
 * then out = y * (g - sum)  /  out = g - expf(y) * sum.  16-bit: float arithmetic on the rounded inputs, one rounding. */
void oracle_softmax_backward(const float* g, const float* y, float* out, int64_t outer, int64_t dim, int64_t inner,
                             int log_form, int dtype) {
  for (int64_t o = 0; o < outer; o++)
    for (int64_t i = 0; i < inner; i++) {
      const int64_t base = o * dim * inner + i;
      float sum = 0.f;
      for (int64_t d = 0; d < dim; d++) sum += log_form ? g[base + d * inner] : y[base + d * inner] * g[base + d * inner];
      for (int64_t d = 0; d < dim; d++) {
        const int64_t at = base + d * inner;
        const float v = log_form ? g[at] - expf(y[at]) * sum : y[at] * (g[at] - sum);
        out[at] = round_t(v, dtype);
      }
    }
}

/* reference src/Operation/OpLinalgCpu.h:119-150 (gemmCpuImpl, the in-tree loop): C = bias rows or zeros, then for i, p, j:
 * c[i][j] += A(i,p) * B(p,j) with A(i,p) = transA ? a[p*m + i] : a[i*k + p], B(p,j) = transB ? b[j*k + p] : b[p*n + j]. */
void oracle_matmul(const float* a, const float* b, const float* bias, float* out, int64_t M, int64_t N, int64_t K,
                   int trans_a, int trans_b, int dtype) {
  for (int64_t i = 0; i < M; i++)
    for (int64_t j = 0; j < N; j++) out[i * N + j] = bias ? bias[j] : 0.f;
  for (int64_t i = 0; i < M; i++)
    for (int64_t p = 0; p < K; p++) {
      const float av = trans_a ? a[p * M + i] : a[i * K + p];
      for (int64_t j = 0; j < N; j++) out[i * N + j] += av * (trans_b ? b[j * K + p] : b[p * N + j]);
    }
  if (dtype != 0)
    for (int64_t e = 0; e < M * N; e++) out[e] = round_t(out[e], dtype);
}

void oracle_linear(const float* x, const float* w, const float* bias, float* out, int64_t M, int64_t N, int64_t K,
                   int dtype) {
  for (int64_t i = 0; i < M; i++)
    for (int64_t j = 0; j < N; j++) out[i * N + j] = bias ? bias[j] : 0.f;
  for (int64_t i = 0; i < M; i++)
    for (int64_t p = 0; p < K; p++) {
      const float av = x[i * K + p];
      for (int64_t j = 0; j < N; j++) out[i * N + j] += av * w[j * K + p];
    }
  if (dtype != 0)
    for (int64_t e = 0; e < M * N; e++) out[e] = round_t(out[e], dtype);
}
