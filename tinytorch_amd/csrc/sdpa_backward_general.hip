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
// Two kernels per call, no atomics (a fixed summation order: results are reproducible).  Head sizes up to 128 take the
// tiled forms further down; larger ones the per-row forms, one wavefront per output row:
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

// ---- tiled forms for head_dim <= 128: 64 rows per workgroup, four adjacent lanes per row ------------------------------------
// The layout of the general forward kernel: lane s of the four holds head_dim elements s, s+4, s+8, ... of its row's
// vectors in registers; the other side streams through LDS as fp32 tiles of 32 rows, read as broadcasts.  Every
// (query, key) pair then costs 3 (dq kernel) + 4 (dk/dv kernel) passes over head_dim on the vector ALUs, against the
// per-row kernels' uncoalesced dot products.
constexpr int kRows = 64;   // rows of the owning side per workgroup
constexpr int kTile = 32;   // rows of the streamed side per LDS tile
constexpr int kChunk = 8;   // streamed rows per online-softmax update (dq kernel)

__device__ __forceinline__ float quad_sum(float x) {
  x += __shfl_xor(x, 1);
  x += __shfl_xor(x, 2);
  return x;
}

template <typename T, int DQ>  // DQ = head_dim elements per lane (head_dim <= 4*DQ)
__global__ __launch_bounds__(256) void backward_dq_tiled_kernel(BwdArgs a) {
  constexpr int DP = 4 * DQ;
  __shared__ float Ks[kTile][DP];
  __shared__ float Vs[kTile][DP];
  const KArgs& f = a.f;
  const int tid = threadIdx.x, sub = tid & 3;
  // consecutive workgroups (which go to different XCDs) take the same row tile of different (batch, head) pairs, the
  // longest tiles of a causal call first: every XCD gets the same mix
  const int ntile_rows = (f.L + kRows - 1) / kRows;
  const long long npair = (long long)f.B * f.Hq;
  const int blk = (int)(blockIdx.x / npair), pair = (int)(blockIdx.x % npair);
  const int rt = f.causal ? ntile_rows - 1 - blk : blk;
  const int h = pair % f.Hq, b = pair / f.Hq;
  const int hk = h / f.G;
  const int row0 = rt * kRows, row = row0 + (tid >> 2);
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
    const int d = 4 * t + sub;
    qreg[t] = d < f.D ? load_as_float(qp + d) : 0.f;
    greg[t] = d < f.D ? load_as_float(gp + d) : 0.f;
    dpart = fmaf(greg[t], d < f.D ? load_as_float(op + d) : 0.f, dpart);
    acc[t] = 0.f;
  }
  const float delta = quad_sum(dpart);
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
          ps = fmaf(qreg[t], Ks[c0 + j][4 * t + sub], ps);
          pd = fmaf(greg[t], Vs[c0 + j][4 * t + sub], pd);
        }
        const int key = k0 + c0 + j;
        x[j] = key < S ? biased_score<T>(f, quad_sum(ps), row, key, coff, mrow) : -INFINITY;
        w[j] = quad_sum(pd) - delta;
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
        for (int j = 0; j < kChunk; j++) o = fmaf(w[j], Ks[c0 + j][4 * t + sub], o);
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
      const int d = 4 * t + sub;
      if (d < f.D) store_from_float(dqp + d, seen ? acc[t] * wgt : 0.f);
    }
  }
}

template <typename T, int DQ>
__global__ __launch_bounds__(256) void backward_dkv_tiled_kernel(BwdArgs a) {
  constexpr int DP = 4 * DQ;
  __shared__ float Qs[kTile][DP];
  __shared__ float Gs[kTile][DP];
  __shared__ float Ls[kTile], Ds[kTile];
  const KArgs& f = a.f;
  const int tid = threadIdx.x, sub = tid & 3;
  const long long npair = (long long)f.B * f.Hkv;  // order as in the dq kernel: the first key blocks are the longest
  const int kb = (int)(blockIdx.x / npair), pair = (int)(blockIdx.x % npair);
  const int hk = pair % f.Hkv, b = pair / f.Hkv;
  const int key0 = kb * kRows, key = key0 + (tid >> 2);
  const int S = keys_of_batch(f, b);
  const int coff = causal_offset(f, S);
  const int keyc = key < f.S ? key : f.S - 1;
  const T* kr = (const T*)f.k + b * f.ks[0] + hk * f.ks[1] + keyc * f.ks[2];
  const T* vr = (const T*)f.v + b * f.vs[0] + hk * f.vs[1] + keyc * f.vs[2];

  float kreg[DQ], vreg[DQ], dk[DQ], dv[DQ];
#pragma unroll
  for (int t = 0; t < DQ; t++) {
    const int d = 4 * t + sub;
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
            ps = fmaf(Qs[ii][4 * t + sub], kreg[t], ps);
            pd = fmaf(Gs[ii][4 * t + sub], vreg[t], pd);
          }
          const float sdot = quad_sum(ps), ddot = quad_sum(pd);
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
            dv[t] = fmaf(p, Gs[ii][4 * t + sub], dv[t]);
            dk[t] = fmaf(ds, Qs[ii][4 * t + sub], dk[t]);
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
      const int d = 4 * t + sub;
      if (d < f.D) {
        store_from_float(dkp + d, dk[t]);
        store_from_float(dvp + d, dv[t]);
      }
    }
  }
}

template <typename T, int DQ>
int launch_tiled(const BwdArgs& a, hipStream_t stream) {
  const long long g1 = (long long)a.f.B * a.f.Hq * ((a.f.L + kRows - 1) / kRows);
  const long long g2 = (long long)a.f.B * a.f.Hkv * ((a.f.S + kRows - 1) / kRows);
  if (g1 > 0) {
    hipLaunchKernelGGL((backward_dq_tiled_kernel<T, DQ>), dim3((unsigned)g1), dim3(256), 0, stream, a);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
  }
  if (g2 > 0) hipLaunchKernelGGL((backward_dkv_tiled_kernel<T, DQ>), dim3((unsigned)g2), dim3(256), 0, stream, a);
  return (int)hipGetLastError();
}

template <typename T>
int launch_t(const BwdArgs& a, hipStream_t stream) {
  if (a.f.D <= 32) return launch_tiled<T, 8>(a, stream);
  if (a.f.D <= 64) return launch_tiled<T, 16>(a, stream);
  if (a.f.D <= 128) return launch_tiled<T, 32>(a, stream);
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
