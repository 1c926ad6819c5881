// General attention backward: any element type, head_dim <= 256, optional causal / Bool / additive mask, per-batch key
// counts.  fp32 arithmetic on the vector ALUs; the route for fp32 tensors, masks and head sizes the MFMA backward
// kernels do not cover.
//
// The reference has no attention backward (reference src/Function/FuncNNLayer.h:267 is NOT_IMPLEMENTED): this is the
// chain rule through its forward (src/Function/FuncNNLayer.h:237-265), with the softmax step the reference's own
// softmax backward takes (src/Operation/OpNNLayerCpu.h:79-109), written so that no [L,S] matrix is stored:
//   P_ij  = exp(scale * q_i . k_j + bias_ij - lse_i)        lse_i = log sum_j exp(scale * q_i . k_j + bias_ij)
//   dP_ij = dout_i . v_j                                     delta_i = sum_j P_ij dP_ij = dout_i . out_i
//   dS_ij = P_ij (dP_ij - delta_i)
//   dq_i  = scale * sum_j dS_ij k_j      dk_j = scale * sum_i dS_ij q_i      dv_j = sum_i P_ij dout_i
// dk and dv sum over the query heads that share a KV head.
//
// Two kernels, one wavefront per output row, no atomics (a fixed summation order: results are reproducible):
//   1. per query row: lse_i and delta_i (kept in scratch for the second kernel) and dq_i;
//   2. per key: dk_j and dv_j over all query rows and the heads of the group.
// A lane owns a key (kernel 1) or a query row (kernel 2) of a 64-wide block for the dot products, then element
// d = lane, lane + 64, ... of the output row for the weighted sums, the weights passed between lanes by shuffles.
//
// A query row whose keys are all hidden (its forward output is NaN) gets dq = 0 and adds nothing to dk / dv.

#include <float.h>

#include "sdpa_common.h"

namespace ttsdpa {

namespace {

constexpr int kMaxT = 4;  // output elements per lane: head_dim <= 64 * kMaxT

__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o);
  return x;
}
__device__ __forceinline__ float wave_max(float x) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) x = fmaxf(x, __shfl_xor(x, o));
  return x;
}

template <typename T>
__device__ __forceinline__ float dot_rows(const T* x, const T* y, int D) {
  float s = 0.f;
  for (int d = 0; d < D; d++) s = fmaf(load_as_float(x + d), load_as_float(y + d), s);
  return s;
}

// Scaled, biased score of (query row i, key j) given the raw dot product; -inf when the key is hidden.
template <typename T>
__device__ __forceinline__ float biased_score(const KArgs& f, float dot, int i, int j, int coff, long long mrow) {
  float x = dot * f.scale;
  bool hidden = f.causal && j > i + coff;
  if (f.mask_kind == 1) {
    if (((const uint8_t*)f.mask)[mrow + j * f.ms[3]] == 0) hidden = true;
  } else if (f.mask_kind == 2) {
    x += load_as_float((const T*)f.mask + mrow + j * f.ms[3]);
  }
  return hidden ? -INFINITY : x;
}

__device__ __forceinline__ int keys_of_batch(const KArgs& f, int b) {
  int S = f.S;
  if (f.kv_len) {
    int len = f.kv_len[b];
    S = len < 0 ? 0 : (len < S ? len : S);
  }
  return S;
}

template <typename T>
__global__ __launch_bounds__(256) void backward_dq_kernel(BwdArgs a) {
  const KArgs& f = a.f;
  const int lane = threadIdx.x & 63;
  const long long row_id = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);  // (b, h, i) flattened
  if (row_id >= (long long)f.B * f.Hq * f.L) return;
  const int i = (int)(row_id % f.L);
  const int h = (int)((row_id / f.L) % f.Hq);
  const int b = (int)(row_id / ((long long)f.L * f.Hq));
  const int hk = h / f.G;
  const T* qi = (const T*)f.q + b * f.qs[0] + h * f.qs[1] + i * f.qs[2];
  const T* oi = (const T*)f.out + b * f.os[0] + h * f.os[1] + i * f.os[2];
  const T* gi = (const T*)a.dout + b * a.dos[0] + h * a.dos[1] + i * a.dos[2];
  const T* kp = (const T*)f.k + b * f.ks[0] + hk * f.ks[1];
  const T* vp = (const T*)f.v + b * f.vs[0] + hk * f.vs[1];
  const long long mrow = b * f.ms[0] + h * f.ms[1] + i * f.ms[2];
  const int S = keys_of_batch(f, b);
  const int coff = causal_offset(f, S);
  int send = S;
  if (f.causal) send = i + coff + 1 < S ? i + coff + 1 : S;

  float part = 0.f;
  for (int d = lane; d < f.D; d += 64) part = fmaf(load_as_float(gi + d), load_as_float(oi + d), part);
  const float delta = wave_sum(part);

  // log-sum-exp of the row: a running (max, sum) per lane, merged across the lanes
  float m = -FLT_MAX, l = 0.f;
  for (int j0 = 0; j0 < send; j0 += 64) {
    const int j = j0 + lane;
    if (j < send) {
      const float x = biased_score<T>(f, dot_rows(qi, kp + j * f.ks[2], f.D), i, j, coff, mrow);
      const float mn = fmaxf(m, x);
      l = l * __expf(m - mn) + __expf(x - mn);
      m = mn;
    }
  }
  const float mall = wave_max(m);
  const float lall = wave_sum(l * __expf(m - mall));
  const float lse = mall + __logf(lall);  // -inf when every key is hidden
  if (lane == 0) {
    a.stats[2 * row_id] = lse;
    a.stats[2 * row_id + 1] = delta;
  }

  float acc[kMaxT] = {0.f, 0.f, 0.f, 0.f};
  for (int j0 = 0; j0 < send; j0 += 64) {
    const int j = j0 + lane;
    float ds = 0.f;
    if (j < send) {
      const float x = biased_score<T>(f, dot_rows(qi, kp + j * f.ks[2], f.D), i, j, coff, mrow);
      if (x > -INFINITY && lse > -INFINITY) {
        const float p = __expf(x - lse);
        ds = p * (dot_rows(gi, vp + j * f.vs[2], f.D) - delta) * f.scale;
      }
    }
    const int n = send - j0 < 64 ? send - j0 : 64;
    for (int jj = 0; jj < n; jj++) {
      const float w = __shfl(ds, jj);
      const T* kr = kp + (j0 + jj) * f.ks[2];
#pragma unroll
      for (int t = 0; t < kMaxT; t++) {
        const int d = lane + 64 * t;
        if (d < f.D) acc[t] = fmaf(w, load_as_float(kr + d), acc[t]);
      }
    }
  }
  T* dqi = (T*)a.dq + b * a.dqs[0] + h * a.dqs[1] + i * a.dqs[2];
#pragma unroll
  for (int t = 0; t < kMaxT; t++) {
    const int d = lane + 64 * t;
    if (d < f.D) store_from_float(dqi + d, acc[t]);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void backward_dkv_kernel(BwdArgs a) {
  const KArgs& f = a.f;
  const int lane = threadIdx.x & 63;
  const long long key_id = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);  // (b, hk, j) flattened
  if (key_id >= (long long)f.B * f.Hkv * f.S) return;
  const int j = (int)(key_id % f.S);
  const int hk = (int)((key_id / f.S) % f.Hkv);
  const int b = (int)(key_id / ((long long)f.S * f.Hkv));
  const T* kj = (const T*)f.k + b * f.ks[0] + hk * f.ks[1] + j * f.ks[2];
  const T* vj = (const T*)f.v + b * f.vs[0] + hk * f.vs[1] + j * f.vs[2];
  const int S = keys_of_batch(f, b);
  const int coff = causal_offset(f, S);

  float dk[kMaxT] = {0.f, 0.f, 0.f, 0.f}, dv[kMaxT] = {0.f, 0.f, 0.f, 0.f};
  if (j < S) {  // keys past the batch entry's count get zero gradients
    int ifirst = 0;  // first query row that sees key j
    if (f.causal) ifirst = j - coff > 0 ? j - coff : 0;
    for (int g = 0; g < f.G; g++) {
      const int h = hk * f.G + g;
      const T* qp = (const T*)f.q + b * f.qs[0] + h * f.qs[1];
      const T* gp = (const T*)a.dout + b * a.dos[0] + h * a.dos[1];
      const float* st = a.stats + 2 * ((long long)(b * f.Hq + h) * f.L);
      for (int i0 = ifirst & ~63; i0 < f.L; i0 += 64) {
        const int i = i0 + lane;
        float p = 0.f, ds = 0.f;
        if (i < f.L) {
          const long long mrow = b * f.ms[0] + h * f.ms[1] + i * f.ms[2];
          const float x = biased_score<T>(f, dot_rows(qp + i * f.qs[2], kj, f.D), i, j, coff, mrow);
          const float lse = st[2 * i];
          if (x > -INFINITY && lse > -INFINITY) {
            p = __expf(x - lse);
            ds = p * (dot_rows(gp + i * a.dos[2], vj, f.D) - st[2 * i + 1]) * f.scale;
          }
        }
        const int n = f.L - i0 < 64 ? f.L - i0 : 64;
        for (int ii = 0; ii < n; ii++) {
          const float wp = __shfl(p, ii), ws = __shfl(ds, ii);
          const T* gr = gp + (i0 + ii) * a.dos[2];
          const T* qr = qp + (i0 + ii) * f.qs[2];
#pragma unroll
          for (int t = 0; t < kMaxT; t++) {
            const int d = lane + 64 * t;
            if (d < f.D) {
              dv[t] = fmaf(wp, load_as_float(gr + d), dv[t]);
              dk[t] = fmaf(ws, load_as_float(qr + d), dk[t]);
            }
          }
        }
      }
    }
  }
  T* dkj = (T*)a.dk + b * a.dks[0] + hk * a.dks[1] + j * a.dks[2];
  T* dvj = (T*)a.dv + b * a.dvs[0] + hk * a.dvs[1] + j * a.dvs[2];
#pragma unroll
  for (int t = 0; t < kMaxT; t++) {
    const int d = lane + 64 * t;
    if (d < f.D) {
      store_from_float(dkj + d, dk[t]);
      store_from_float(dvj + d, dv[t]);
    }
  }
}

template <typename T>
int launch_t(const BwdArgs& a, hipStream_t stream) {
  const long long rows = (long long)a.f.B * a.f.Hq * a.f.L, keys = (long long)a.f.B * a.f.Hkv * a.f.S;
  if (rows > 0) {
    hipLaunchKernelGGL((backward_dq_kernel<T>), dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, stream, a);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
  }
  if (keys > 0) hipLaunchKernelGGL((backward_dkv_kernel<T>), dim3((unsigned)((keys + 3) / 4)), dim3(256), 0, stream, a);
  return (int)hipGetLastError();
}

}  // namespace

int launch_backward_general(const BwdArgs& a, int dtype, hipStream_t stream) {
  if (dtype == 0) return launch_t<float>(a, stream);
  if (dtype == 1) return launch_t<_Float16>(a, stream);
  return launch_t<__bf16>(a, stream);
}

}  // namespace ttsdpa
