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
// Two kernels per call, no atomics (a fixed summation order: results are reproducible):
//   1. per block of query rows: lse_i and delta_i (kept in scratch for the second kernel) and dq_i, the keys and
//      values streamed through LDS as fp32 tiles, the softmax statistics built online;
//   2. per block of keys: dk_j and dv_j over all query rows and the heads of the group, the query and dout rows
//      streamed the same way.
// A row of the owning side is held by four adjacent lanes (head_dim <= 128; 64 rows per workgroup) or eight
// (head_dim <= 256; 32 rows), each with every fourth / eighth element of it; dot products end in a sum over those lanes.
//
// A query row whose keys are all hidden (its forward output is NaN) gets dq = 0 and adds nothing to dk / dv.

#include <float.h>

#include "sdpa_common.h"

namespace ttsdpa {

namespace {

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

// ---- 64 rows per workgroup with four adjacent lanes per row (head_dim <= 128), 32 rows with eight (<= 256) ----
// The layout of the general forward kernel: lane s of the LPR holds head_dim elements s, s+LPR, s+2*LPR, ... of its
// row's vectors in registers; the other side streams through LDS as fp32 tiles of 32 / 16 rows, read as broadcasts.
// Every (query, key) pair costs 3 (dq kernel) + 4 (dk/dv kernel) passes over head_dim on the vector ALUs.
template <int LPR>
struct Tiled {
  static constexpr int kRows = 256 / LPR;          // rows of the owning side per workgroup
  static constexpr int kTile = LPR == 4 ? 32 : 16;  // rows of the streamed side per LDS tile (two fp32 tiles within 64 KB)
};
constexpr int kChunk = 8;   // streamed rows per online-softmax update (dq kernel)

template <int LPR>  // sum over the LPR adjacent lanes of a row; every one of them gets the result
__device__ __forceinline__ float group_sum(float x) {
  x += __shfl_xor(x, 1);
  x += __shfl_xor(x, 2);
  if (LPR == 8) x += __shfl_xor(x, 4);
  return x;
}

template <typename T, int DQ, int LPR>  // DQ = head_dim elements per lane (head_dim <= LPR*DQ)
__global__ __launch_bounds__(256) void backward_dq_tiled_kernel(BwdArgs a) {
  constexpr int DP = LPR * DQ;
  constexpr int kRows = Tiled<LPR>::kRows, kTile = Tiled<LPR>::kTile;
  __shared__ float Ks[kTile][DP];
  __shared__ float Vs[kTile][DP];
  const KArgs& f = a.f;
  const int tid = threadIdx.x, sub = tid & (LPR - 1);
  // consecutive workgroups (which go to different XCDs) take the same row tile of different (batch, head) pairs, the
  // longest tiles of a causal call first: every XCD gets the same mix
  const int ntile_rows = (f.L + kRows - 1) / kRows;
  const long long npair = (long long)f.B * f.Hq;
  const int blk = (int)(blockIdx.x / npair), pair = (int)(blockIdx.x % npair);
  const int rt = f.causal ? ntile_rows - 1 - blk : blk;
  const int h = pair % f.Hq, b = pair / f.Hq;
  const int hk = h / f.G;
  const int row0 = rt * kRows, row = row0 + (tid / LPR);
  const int rowc = row < f.L ? row : f.L - 1;
  const T* qp = (const T*)f.q + b * f.qs[0] + h * f.qs[1] + rowc * f.qs[2];
  const T* op = (const T*)f.out + b * f.os[0] + h * f.os[1] + rowc * f.os[2];
  const T* gp = (const T*)a.dout + b * a.dos[0] + h * a.dos[1] + rowc * a.dos[2];
  const T* kp = (const T*)f.k + b * f.ks[0] + hk * f.ks[1];
  const T* vp = (const T*)f.v + b * f.vs[0] + hk * f.vs[1];
  const long long mrow = b * f.ms[0] + h * f.ms[1] + rowc * f.ms[2];

  float qreg[DQ], greg[DQ], acc[DQ];
  float dpart = 0.f;
#pragma unroll
  for (int t = 0; t < DQ; t++) {
    const int d = LPR * t + sub;
    qreg[t] = d < f.D ? load_as_float(qp + d) : 0.f;
    greg[t] = d < f.D ? load_as_float(gp + d) : 0.f;
    dpart = fmaf(greg[t], d < f.D ? load_as_float(op + d) : 0.f, dpart);
    acc[t] = 0.f;
  }
  const float delta = group_sum<LPR>(dpart);
  float m = -FLT_MAX, l = 0.f;

  const int S = keys_of_batch(f, b);
  const int coff = causal_offset(f, S);
  int send = S;
  if (f.causal) {
    const int last = (row0 + kRows - 1 < f.L - 1 ? row0 + kRows - 1 : f.L - 1) + coff;
    send = last + 1 < S ? last + 1 : S;
  }
  for (int k0 = 0; k0 < send; k0 += kTile) {
    __syncthreads();
    for (int e = tid; e < kTile * DP; e += 256) {
      const int kk = e / DP, d = e % DP, key = k0 + kk;
      const bool in = key < S && d < f.D;
      Ks[kk][d] = in ? load_as_float(kp + key * f.ks[2] + d) : 0.f;
      Vs[kk][d] = in ? load_as_float(vp + key * f.vs[2] + d) : 0.f;
    }
    __syncthreads();
    for (int c0 = 0; c0 < kTile; c0 += kChunk) {
      if (k0 + c0 >= send) break;
      float x[kChunk], w[kChunk];
      float cmax = -INFINITY;
#pragma unroll
      for (int j = 0; j < kChunk; j++) {
        float ps = 0.f, pd = 0.f;
#pragma unroll
        for (int t = 0; t < DQ; t++) {
          ps = fmaf(qreg[t], Ks[c0 + j][LPR * t + sub], ps);
          pd = fmaf(greg[t], Vs[c0 + j][LPR * t + sub], pd);
        }
        const int key = k0 + c0 + j;
        x[j] = key < S ? biased_score<T>(f, group_sum<LPR>(ps), row, key, coff, mrow) : -INFINITY;
        w[j] = group_sum<LPR>(pd) - delta;
        cmax = fmaxf(cmax, x[j]);
      }
      const float mn = fmaxf(m, cmax);  // stays -FLT_MAX while every key so far is hidden
      const float alpha = __expf(m - mn);
      float psum = 0.f;
#pragma unroll
      for (int j = 0; j < kChunk; j++) {
        const float p = __expf(x[j] - mn);
        psum += p;
        w[j] *= p;  // dS relative to the running maximum; normalised at the end
      }
      l = l * alpha + psum;
      m = mn;
#pragma unroll
      for (int t = 0; t < DQ; t++) {
        float o = acc[t] * alpha;
#pragma unroll
        for (int j = 0; j < kChunk; j++) o = fmaf(w[j], Ks[c0 + j][LPR * t + sub], o);
        acc[t] = o;
      }
    }
  }
  if (row < f.L) {
    const bool seen = l > 0.f;  // a row whose keys are all hidden: dq = 0, and the dk/dv kernel skips it (lse = -inf)
    if (sub == 0) {
      const long long row_id = ((long long)b * f.Hq + h) * f.L + row;
      a.stats[2 * row_id] = seen ? m + __logf(l) : -INFINITY;
      a.stats[2 * row_id + 1] = delta;
    }
    const float wgt = seen ? f.scale / l : 0.f;
    T* dqp = (T*)a.dq + b * a.dqs[0] + h * a.dqs[1] + row * a.dqs[2];
#pragma unroll
    for (int t = 0; t < DQ; t++) {
      const int d = LPR * t + sub;
      if (d < f.D) store_from_float(dqp + d, seen ? acc[t] * wgt : 0.f);
    }
  }
}

template <typename T, int DQ, int LPR>
__global__ __launch_bounds__(256) void backward_dkv_tiled_kernel(BwdArgs a) {
  constexpr int DP = LPR * DQ;
  constexpr int kRows = Tiled<LPR>::kRows, kTile = Tiled<LPR>::kTile;
  __shared__ float Qs[kTile][DP];
  __shared__ float Gs[kTile][DP];
  __shared__ float Ls[kTile], Ds[kTile];
  const KArgs& f = a.f;
  const int tid = threadIdx.x, sub = tid & (LPR - 1);
  const long long npair = (long long)f.B * f.Hkv;  // order as in the dq kernel: the first key blocks are the longest
  const int kb = (int)(blockIdx.x / npair), pair = (int)(blockIdx.x % npair);
  const int hk = pair % f.Hkv, b = pair / f.Hkv;
  const int key0 = kb * kRows, key = key0 + (tid / LPR);
  const int S = keys_of_batch(f, b);
  const int coff = causal_offset(f, S);
  const int keyc = key < f.S ? key : f.S - 1;
  const T* kr = (const T*)f.k + b * f.ks[0] + hk * f.ks[1] + keyc * f.ks[2];
  const T* vr = (const T*)f.v + b * f.vs[0] + hk * f.vs[1] + keyc * f.vs[2];

  float kreg[DQ], vreg[DQ], dk[DQ], dv[DQ];
#pragma unroll
  for (int t = 0; t < DQ; t++) {
    const int d = LPR * t + sub;
    kreg[t] = d < f.D ? load_as_float(kr + d) : 0.f;
    vreg[t] = d < f.D ? load_as_float(vr + d) : 0.f;
    dk[t] = 0.f, dv[t] = 0.f;
  }
  int ifirst = 0;  // first query row that sees a key of this workgroup
  if (f.causal) ifirst = key0 - coff > 0 ? key0 - coff : 0;
  if (key0 < S) {  // else: no query row attends to these keys; zeros
    for (int g = 0; g < f.G; g++) {
      const int h = hk * f.G + g;
      const T* qp = (const T*)f.q + b * f.qs[0] + h * f.qs[1];
      const T* gp = (const T*)a.dout + b * a.dos[0] + h * a.dos[1];
      const float* st = a.stats + 2 * (((long long)b * f.Hq + h) * f.L);
      for (int i0 = ifirst & ~(kTile - 1); i0 < f.L; i0 += kTile) {
        __syncthreads();
        for (int e = tid; e < kTile * DP; e += 256) {
          const int ii = e / DP, d = e % DP, i = i0 + ii;
          const bool in = i < f.L && d < f.D;
          Qs[ii][d] = in ? load_as_float(qp + i * f.qs[2] + d) : 0.f;
          Gs[ii][d] = in ? load_as_float(gp + i * a.dos[2] + d) : 0.f;
        }
        if (tid < kTile) {
          const int i = i0 + tid;
          Ls[tid] = i < f.L ? st[2 * i] : -INFINITY;  // rows past the end weigh nothing
          Ds[tid] = i < f.L ? st[2 * i + 1] : 0.f;
        }
        __syncthreads();
        for (int ii = 0; ii < kTile; ii++) {
          const int i = i0 + ii;
          if (i >= f.L) break;
          float ps = 0.f, pd = 0.f;
#pragma unroll
          for (int t = 0; t < DQ; t++) {
            ps = fmaf(Qs[ii][LPR * t + sub], kreg[t], ps);
            pd = fmaf(Gs[ii][LPR * t + sub], vreg[t], pd);
          }
          const float sdot = group_sum<LPR>(ps), ddot = group_sum<LPR>(pd);
          const float lse = Ls[ii];
          float p = 0.f, ds = 0.f;
          if (key < S && lse > -INFINITY) {
            const long long mrow = b * f.ms[0] + h * f.ms[1] + i * f.ms[2];
            const float x = biased_score<T>(f, sdot, i, key, coff, mrow);
            if (x > -INFINITY) {
              p = __expf(x - lse);
              ds = p * (ddot - Ds[ii]) * f.scale;
            }
          }
#pragma unroll
          for (int t = 0; t < DQ; t++) {
            dv[t] = fmaf(p, Gs[ii][LPR * t + sub], dv[t]);
            dk[t] = fmaf(ds, Qs[ii][LPR * t + sub], dk[t]);
          }
        }
      }
    }
  }
  if (key < f.S) {
    T* dkp = (T*)a.dk + b * a.dks[0] + hk * a.dks[1] + key * a.dks[2];
    T* dvp = (T*)a.dv + b * a.dvs[0] + hk * a.dvs[1] + key * a.dvs[2];
#pragma unroll
    for (int t = 0; t < DQ; t++) {
      const int d = LPR * t + sub;
      if (d < f.D) {
        store_from_float(dkp + d, dk[t]);
        store_from_float(dvp + d, dv[t]);
      }
    }
  }
}

template <typename T, int DQ, int LPR>
int launch_tiled(const BwdArgs& a, hipStream_t stream) {
  constexpr int kRows = Tiled<LPR>::kRows;
  const long long g1 = (long long)a.f.B * a.f.Hq * ((a.f.L + kRows - 1) / kRows);
  const long long g2 = (long long)a.f.B * a.f.Hkv * ((a.f.S + kRows - 1) / kRows);
  if (g1 > 0) {
    hipLaunchKernelGGL((backward_dq_tiled_kernel<T, DQ, LPR>), dim3((unsigned)g1), dim3(256), 0, stream, a);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
  }
  if (g2 > 0) hipLaunchKernelGGL((backward_dkv_tiled_kernel<T, DQ, LPR>), dim3((unsigned)g2), dim3(256), 0, stream, a);
  return (int)hipGetLastError();
}

template <typename T>
int launch_t(const BwdArgs& a, hipStream_t stream) {
  if (a.f.D <= 32) return launch_tiled<T, 8, 4>(a, stream);
  if (a.f.D <= 64) return launch_tiled<T, 16, 4>(a, stream);
  if (a.f.D <= 128) return launch_tiled<T, 32, 4>(a, stream);
  if (a.f.D <= 256) return launch_tiled<T, 32, 8>(a, stream);
  return (int)hipErrorInvalidValue;  // head_dim > 256 is refused before any launch
}

}  // namespace

int launch_backward_general(const BwdArgs& a, int dtype, hipStream_t stream) {
  if (dtype == 0) return launch_t<float>(a, stream);
  if (dtype == 1) return launch_t<_Float16>(a, stream);
  return launch_t<__bf16>(a, stream);
}

}  // namespace ttsdpa
