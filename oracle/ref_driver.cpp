// TEST INFRASTRUCTURE — not part of the product.
//
// C-ABI shim over the *real* TinyTorch CPU library (compiled by oracle/Makefile from the sources where they lie
// under /root/reference; nothing of the reference is copied into this repository).  It calls
// tinytorch::function::sdpAttention (reference src/Function/FuncNNLayer.h:298-302) and the row-wise neighbour ops
// (rmsNorm, fusedAddRmsNorm, siluMul, softmax) on CPU fp32 tensors and hands
// the result back through plain pointers, so the tests can pin oracle/sdpa_oracle.c against the reference itself
// and write the golden fixtures under tests/golden/.
//
// Built only where /root/reference exists; the resulting oracle/_ref/libtt_ref.so travels to the GPU box.

#include <cstdint>
#include <cstring>
#include <limits>
#include <vector>

#include "TinyTorch.h"

using namespace tinytorch;

namespace {

Tensor fromF32(const float* p, const std::vector<int64_t>& shape) {
  int64_t n = 1;
  for (auto s : shape) n *= s;
  std::vector<float> buf(p, p + n);
  Tensor t(buf);
  t.reshape_(IntArrayView(shape));
  return t;
}

void ensureCpu() {
  static bool done = false;
  if (!done) {
    setDefaultDevice(DeviceType::CPU);
    done = true;
  }
}

}  // namespace

extern "C" {

// Round-trip fp32 -> {1: Float16, 2: BFloat16} -> fp32 through the reference's own dtype cast
// (Tensor::to, reference src/Tensor/Tensor.cpp:224-233; Half.h:226-257; BFloat16.h:72-85).
int tt_ref_round_trip(const float* in, float* out, int64_t n, int dtype) {
  ensureCpu();
  Tensor t = fromF32(in, {n});
  Tensor r = t.to(dtype == 1 ? DType::Float16 : DType::BFloat16).to(DType::Float32);
  auto v = r.toList<float>();
  std::memcpy(out, v.data(), sizeof(float) * n);
  return 0;
}

// function::sdpAttention on fp32 CPU tensors.
//   q [B,Hq,L,D]; k,v [B,Hkv,S,D]; out [B,Hq,L,D].
//   Hkv != Hq: grouped-query attention through op::repeatInterleave(k, Hq/Hkv, 1)
//   (reference src/Operation/OpTransformCpu.h:399-442), i.e. kv_head = q_head / (Hq/Hkv).
//   mask_kind: 0 none, 1 Bool (uint8 0/1), 2 additive float; the mask has shape mask_dims[0..mask_ndim) (any shape
//   that broadcasts to [B,Hq,L,S]; mask_ndim == 0 means [L,S]).
//   has_scale == 0 -> default 1/sqrt(D).
int tt_ref_sdpa_f32(const float* q, const float* k, const float* v, float* out, int64_t B, int64_t Hq, int64_t Hkv,
                    int64_t L, int64_t S, int64_t D, int causal, int has_scale, float scale, int mask_kind,
                    const void* mask, int mask_ndim, const int64_t* mask_dims) {
  ensureCpu();
  NoGradGuard guard;
  Tensor tq = fromF32(q, {B, Hq, L, D});
  Tensor tk = fromF32(k, {B, Hkv, S, D});
  Tensor tv = fromF32(v, {B, Hkv, S, D});
  if (Hkv != Hq) {
    if (Hq % Hkv != 0) return -1;
    tk = op::repeatInterleave(tk, Hq / Hkv, 1);
    tv = op::repeatInterleave(tv, Hq / Hkv, 1);
  }
  Tensor tm;
  std::vector<int64_t> mshape = {L, S};
  if (mask_ndim > 0) mshape.assign(mask_dims, mask_dims + mask_ndim);
  int64_t mcount = 1;
  for (int64_t d : mshape) mcount *= d;
  if (mask_kind == 1) {
    const auto* m = static_cast<const uint8_t*>(mask);
    std::vector<uint8_t> buf(m, m + mcount);
    tm = Tensor(buf, options::dtype(DType::Bool));
    tm.reshape_(IntArrayView(mshape));
  } else if (mask_kind == 2) {
    tm = fromF32(static_cast<const float*>(mask), mshape);
  }
  std::optional<float> sc = has_scale ? std::optional<float>(scale) : std::nullopt;
  Tensor y = function::sdpAttention(tq, tk, tv, causal != 0, tm, 0.f, sc);
  auto r = y.toList<float>();
  if (static_cast<int64_t>(r.size()) != B * Hq * L * D) return -2;
  std::memcpy(out, r.data(), sizeof(float) * r.size());
  return 0;
}

// Same call through the matmul batch-broadcast form of GQA (5-D q [B,Hkv,G,L,D] x kv [B,Hkv,1,S,D],
// reference src/Operation/OpLinalg.cpp:205-223) — used to check that both GQA spellings agree.
int tt_ref_sdpa_f32_gqa5d(const float* q, const float* k, const float* v, float* out, int64_t B, int64_t Hq,
                          int64_t Hkv, int64_t L, int64_t S, int64_t D, int causal) {
  ensureCpu();
  NoGradGuard guard;
  if (Hq % Hkv != 0) return -1;
  int64_t G = Hq / Hkv;
  Tensor tq = fromF32(q, {B, Hkv, G, L, D});
  Tensor tk = fromF32(k, {B, Hkv, 1, S, D});
  Tensor tv = fromF32(v, {B, Hkv, 1, S, D});
  Tensor y = function::sdpAttention(tq, tk, tv, causal != 0);
  auto r = y.toList<float>();
  if (static_cast<int64_t>(r.size()) != B * Hq * L * D) return -2;
  std::memcpy(out, r.data(), sizeof(float) * r.size());
  return 0;
}

// function::rmsNorm over the last axis of [rows, dim] (reference src/Function/FuncNNLayer.h:294); w may be NULL.
int tt_ref_rms_norm(const float* x, const float* w, float* out, int64_t rows, int64_t dim, float eps) {
  ensureCpu();
  NoGradGuard guard;
  Tensor tx = fromF32(x, {rows, dim});
  Tensor tw;
  if (w) tw = fromF32(w, {dim});
  Tensor y = function::rmsNorm(tx, {dim}, tw, eps);
  auto r = y.toList<float>();
  if (static_cast<int64_t>(r.size()) != rows * dim) return -2;
  std::memcpy(out, r.data(), sizeof(float) * r.size());
  return 0;
}

// function::fusedAddRmsNorm (reference src/Function/FuncFused.h:32), in place: input and residual are overwritten.
int tt_ref_fused_add_rms_norm(float* input, float* residual, const float* w, int64_t rows, int64_t dim, float eps) {
  ensureCpu();
  NoGradGuard guard;
  Tensor ti = fromF32(input, {rows, dim});
  Tensor tr = fromF32(residual, {rows, dim});
  Tensor tw = fromF32(w, {dim});
  function::fusedAddRmsNorm(ti, tr, tw, eps);
  auto a = ti.toList<float>();
  auto b = tr.toList<float>();
  if (static_cast<int64_t>(a.size()) != rows * dim || a.size() != b.size()) return -2;
  std::memcpy(input, a.data(), sizeof(float) * a.size());
  std::memcpy(residual, b.data(), sizeof(float) * b.size());
  return 0;
}

// function::siluMul (reference src/Function/FuncFused.h:30) on [rows, 2*d] -> [rows, d].
int tt_ref_silu_mul(const float* x, float* out, int64_t rows, int64_t d) {
  ensureCpu();
  NoGradGuard guard;
  Tensor y = function::siluMul(fromF32(x, {rows, 2 * d}));
  auto r = y.toList<float>();
  if (static_cast<int64_t>(r.size()) != rows * d) return -2;
  std::memcpy(out, r.data(), sizeof(float) * r.size());
  return 0;
}

// function::softmax / logSoftmax (reference src/Function/FuncActivation.h:91-92) along axis 1 of [outer, dim, inner].
int tt_ref_softmax(const float* x, float* out, int64_t outer, int64_t dim, int64_t inner, int log_form) {
  ensureCpu();
  NoGradGuard guard;
  Tensor tx = fromF32(x, {outer, dim, inner});
  Tensor y = log_form ? function::logSoftmax(tx, 1) : function::softmax(tx, 1);
  auto r = y.toList<float>();
  if (static_cast<int64_t>(r.size()) != outer * dim * inner) return -2;
  std::memcpy(out, r.data(), sizeof(float) * r.size());
  return 0;
}

// op::softmaxBackward / op::logSoftmaxBackward (reference src/Operation/OpNNLayer.h:46-51) over axis 1 of [outer, dim, inner].
int tt_ref_softmax_backward(const float* g, const float* y, float* out, int64_t outer, int64_t dim, int64_t inner,
                            int log_form) {
  ensureCpu();
  NoGradGuard guard;
  Tensor tg = fromF32(g, {outer, dim, inner}), ty = fromF32(y, {outer, dim, inner});
  Tensor r = log_form ? op::logSoftmaxBackward(tg, ty, 1) : op::softmaxBackward(tg, ty, 1);
  auto v = r.toList<float>();
  if (static_cast<int64_t>(v.size()) != outer * dim * inner) return -2;
  std::memcpy(out, v.data(), sizeof(float) * v.size());
  return 0;
}

// function::linear (reference src/Function/FuncNNLayer.h:270-272): x [M,K], w [N,K], bias [N] or NULL -> out [M,N].
int tt_ref_linear(const float* x, const float* w, const float* bias, float* out, int64_t M, int64_t N, int64_t K) {
  ensureCpu();
  NoGradGuard guard;
  Tensor tb;
  if (bias) tb = fromF32(bias, {N});
  Tensor y = function::linear(fromF32(x, {M, K}), fromF32(w, {N, K}), tb);
  auto r = y.toList<float>();
  if (static_cast<int64_t>(r.size()) != M * N) return -2;
  std::memcpy(out, r.data(), sizeof(float) * r.size());
  return 0;
}

int tt_ref_matmul(const float* a, const float* b, const float* bias, float* out, int64_t M, int64_t N, int64_t K,
                  int transA, int transB) {
  ensureCpu();
  NoGradGuard guard;
  Tensor tb;
  if (bias) tb = fromF32(bias, {N});
  Tensor ta = transA ? fromF32(a, {K, M}) : fromF32(a, {M, K});
  Tensor tw = transB ? fromF32(b, {N, K}) : fromF32(b, {K, N});
  Tensor y = op::matmul(ta, tw, transA != 0, transB != 0, tb);
  auto r = y.toList<float>();
  if (static_cast<int64_t>(r.size()) != M * N) return -2;
  std::memcpy(out, r.data(), sizeof(float) * r.size());
  return 0;
}

}  // extern "C"
