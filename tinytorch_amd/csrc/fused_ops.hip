// Row-wise inference ops next to attention — rmsNorm, fusedAddRmsNorm, siluMul, softmax / logSoftmax — for gfx950.
// They replace the reference's device kernels src/Operation/OpFusedCuda.cuh:16-146 and
// src/Operation/OpNNLayerCuda.cuh:36-145, 253-345.  All are bound by HBM traffic: every element is read once with
// 16-byte nontemporal loads (the data is not needed again by this kernel), rows stay in registers between the
// reduction and the write, and the arithmetic is fp32 with one rounding to the element type.
//
// Row kernels: a workgroup of 256 lanes serves 256/LPR rows, LPR lanes per row (8 .. 256, chosen so that a lane holds
// one or two 16-byte vectors for common row lengths).  A lane keeps up to CACHE vectors of its row in registers; longer
// rows re-read the part that does not fit.  Rows that cannot be read as 16-byte vectors use the same kernels with
// one element per access.

#include "sdpa_common.h"
#include "../../include/ttfused.h"

namespace ttsdpa {
namespace {

constexpr int CACHE = 8;  // 16-byte vectors a lane keeps of its row

template <typename T, int VEC>
struct Pack {
  typedef T type __attribute__((ext_vector_type(VEC)));
};
template <typename T>
struct Pack<T, 1> {
  struct type {
    T x;
    __device__ __forceinline__ T& operator[](int) { return x; }
    __device__ __forceinline__ const T& operator[](int) const { return x; }
  };
};

template <typename T, int VEC>
__device__ __forceinline__ typename Pack<T, VEC>::type load_stream(const T* p) {
  typedef typename Pack<T, VEC>::type V;
  if constexpr (VEC == 1) {
    V v;
    v.x = __builtin_nontemporal_load(p);
    return v;
  } else {
    return __builtin_nontemporal_load((const V*)p);
  }
}
template <typename T, int VEC>
__device__ __forceinline__ typename Pack<T, VEC>::type load_plain(const T* p) {
  typedef typename Pack<T, VEC>::type V;
  if constexpr (VEC == 1) {
    V v;
    v.x = *p;
    return v;
  } else {
    return *(const V*)p;
  }
}
template <typename T, int VEC>
__device__ __forceinline__ void store_pack(T* p, const typename Pack<T, VEC>::type& v) {
  typedef typename Pack<T, VEC>::type V;
  // written once, not read again here: keep it from displacing the cached input
  if constexpr (VEC == 1) {
    __builtin_nontemporal_store(v.x, p);
  } else {
    __builtin_nontemporal_store(v, (V*)p);
  }
}

struct SumOp {
  static __device__ __forceinline__ float apply(float a, float b) { return a + b; }
};
struct MaxOp {
  static __device__ __forceinline__ float apply(float a, float b) { return fmaxf(a, b); }
};

// Reduction over the LPR lanes of a row; every lane of the row gets the result.  LPR <= 64: butterfly inside the
// wavefront.  LPR == 256 or 1024: the workgroup is one row; wavefront totals cross through LDS (`slot` tells successive
// reductions of one kernel apart, so one barrier per reduction suffices; lds holds 2 slots x LPR/64 floats).
template <int LPR, typename Op>
__device__ __forceinline__ float row_reduce(float v, float* lds, int slot) {
  constexpr int W = LPR < 64 ? LPR : 64;
#pragma unroll
  for (int o = W / 2; o >= 1; o >>= 1) v = Op::apply(v, __shfl_xor(v, o));
  if constexpr (LPR == 256) {
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) lds[4 * slot + wave] = v;
    __syncthreads();
    v = Op::apply(Op::apply(lds[4 * slot], lds[4 * slot + 1]), Op::apply(lds[4 * slot + 2], lds[4 * slot + 3]));
  } else if constexpr (LPR > 256) {
    constexpr int NW = LPR / 64;
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) lds[NW * slot + wave] = v;
    __syncthreads();
    v = lds[NW * slot];
#pragma unroll
    for (int w = 1; w < NW; w++) v = Op::apply(v, lds[NW * slot + w]);  // the same order in every lane
  }
  return v;
}

// Walk the part of a row that a lane does not keep in registers (vectors lr + CACHE*LPR, + LPR, ...), four loads in
// flight: `load(i)` fetches vector i, `use(i, v)` consumes it.
template <int LPR, typename Load, typename Use, int KEPT = CACHE>
__device__ __forceinline__ void walk_rest(int lr, int nvec, Load load, Use use) {
  for (int i0 = lr + KEPT * LPR; i0 < nvec; i0 += 4 * LPR) {
    decltype(load(0)) v[4];
#pragma unroll
    for (int u = 0; u < 4; u++)
      if (i0 + u * LPR < nvec) v[u] = load(i0 + u * LPR);
#pragma unroll
    for (int u = 0; u < 4; u++)
      if (i0 + u * LPR < nvec) use(i0 + u * LPR, v[u]);
  }
}

// ---- rmsNorm and fusedAddRmsNorm ---------------------------------------------------------------------------------
// FUSED: r = input + residual, residual <- T(r), sum of squares over the unrounded r, input <- T(float(T(r)) * inv * w).
// else:  out <- T(x * inv [* w]).
template <typename T, int VEC, int LPR, bool FUSED>
__global__ __launch_bounds__(256) void rms_norm_kernel(const T* x, T* res, const T* __restrict__ w, T* out,  // out may be x
                                                       long long rows, int dim, float eps) {
  typedef typename Pack<T, VEC>::type V;
  __shared__ float lds[8];
  constexpr int RPB = 256 / LPR;
  const int lr = threadIdx.x % LPR;
  const long long row = (long long)blockIdx.x * RPB + threadIdx.x / LPR;
  const bool live = row < rows;
  const int nvec = dim / VEC;
  const T* xr = x + row * dim;
  T* rr = FUSED ? res + row * dim : nullptr;
  T* orow = out + row * dim;

  V keep[CACHE];
  float ss = 0.f;
  // input vector i (FUSED: both operands, packed side by side)
  struct In {
    V a, b;
  };
  auto fetch = [&](int i) __attribute__((always_inline)) {
    In v;
    v.a = load_stream<T, VEC>(xr + (long long)i * VEC);
    if constexpr (FUSED) v.b = load_stream<T, VEC>(rr + (long long)i * VEC);
    return v;
  };
  // -> the vector the second phase normalises; adds its squares to ss
  auto absorb = [&](int i, const In& v) __attribute__((always_inline)) {
    V a = v.a;
    if constexpr (FUSED) {
#pragma unroll
      for (int e = 0; e < VEC; e++) {
        float r = (float)v.a[e] + (float)v.b[e];
        a[e] = (T)r;
        ss = fmaf(r, r, ss);
      }
      store_pack<T, VEC>(rr + (long long)i * VEC, a);
    } else {
#pragma unroll
      for (int e = 0; e < VEC; e++) ss = fmaf((float)a[e], (float)a[e], ss);
    }
    return a;
  };
  if (live) {
    In first[CACHE];
#pragma unroll
    for (int c = 0; c < CACHE; c++)
      if (lr + c * LPR < nvec) first[c] = fetch(lr + c * LPR);
#pragma unroll
    for (int c = 0; c < CACHE; c++)
      if (lr + c * LPR < nvec) keep[c] = absorb(lr + c * LPR, first[c]);
    walk_rest<LPR>(lr, nvec, fetch, [&](int i, const In& v) __attribute__((always_inline)) { absorb(i, v); });
  }
  ss = row_reduce<LPR, SumOp>(ss, lds, 0);
  const float inv = 1.f / sqrtf(ss / (float)dim + eps);
  if (!live) return;
  auto give = [&](int i, const V& a) __attribute__((always_inline)) {
    V o;
    if (w) {
      V wv = load_plain<T, VEC>(w + (long long)i * VEC);
#pragma unroll
      for (int e = 0; e < VEC; e++) o[e] = (T)((float)a[e] * inv * (float)wv[e]);
    } else {
#pragma unroll
      for (int e = 0; e < VEC; e++) o[e] = (T)((float)a[e] * inv);
    }
    store_pack<T, VEC>(orow + (long long)i * VEC, o);
  };
#pragma unroll
  for (int c = 0; c < CACHE; c++)
    if (lr + c * LPR < nvec) give(lr + c * LPR, keep[c]);
  // the part of a very long row that was not kept is read again (FUSED: the residual just stored)
  walk_rest<LPR>(
      lr, nvec, [&](int i) __attribute__((always_inline)) { return load_plain<T, VEC>((FUSED ? rr : xr) + (long long)i * VEC); },
      give);
}

// ---- softmax / logSoftmax over the last axis ---------------------------------------------------------------------------
// One reading pass: every lane keeps a running maximum and the sum of exponentials relative to it (rescaled when the
// maximum grows), the lanes' pairs are merged after the row maximum is known, then the row is written from the
// registers (and from a second read for the part of a very long row that was not kept).
// KEEP: vectors of its row a lane holds in registers between the statistics and the write (16 for rows of one workgroup
// that would otherwise be read twice: up to 32768 16-bit elements are then read once).
// LPR == 1024 (a few very long rows: the softmax over a vocabulary for a batch of sequences): a workgroup of 16
// wavefronts per row.  With 256 lanes such a launch has one small workgroup per row on a quarter of the CUs and four
// loads per lane in flight: latency-bound (64 rows of 128256 bf16 elements: 30 us, 1.1 TB/s; 19 us with 1024 lanes, of
// which a third is the row's exponentials on one CU.  Keeping 16 vectors per lane instead of 8 measured the same: a
// wavefront of such a workgroup has 128 registers, too few to hold a longer row's exponentials as fp32).
template <typename T, int VEC, int LPR, bool LOG, int KEEP>
__global__ __launch_bounds__(LPR > 256 ? LPR : 256) void softmax_rows_kernel(const T* x, T* out, long long rows, int dim) {  // out may be x
  typedef typename Pack<T, VEC>::type V;
  constexpr int BLK = LPR > 256 ? LPR : 256;
  __shared__ float lds[LPR > 256 ? 2 * (LPR / 64) : 8];
  constexpr int RPB = BLK / LPR;
  const int lr = threadIdx.x % LPR;
  const long long row = (long long)blockIdx.x * RPB + threadIdx.x / LPR;
  const bool live = row < rows;
  const int nvec = dim / VEC;
  const T* xr = x + row * dim;
  T* orow = out + row * dim;

  V keep[KEEP];
  float mx = -3.402823466e+38f;  // the reference starts from the lowest finite float
  float sum = 0.f;
  auto absorb = [&](int, const V& a) __attribute__((always_inline)) {
    float vm = (float)a[0];
#pragma unroll
    for (int e = 1; e < VEC; e++) vm = fmaxf(vm, (float)a[e]);
    const float mn = fmaxf(mx, vm);
    sum *= __expf(mx - mn);
#pragma unroll
    for (int e = 0; e < VEC; e++) sum += __expf((float)a[e] - mn);
    mx = mn;
  };
  auto reload = [&](int i) __attribute__((always_inline)) { return load_plain<T, VEC>(xr + (long long)i * VEC); };
  if (!LOG && nvec <= KEEP * LPR) {
    // The whole row sits in the lanes' registers: the reference's own three steps (maximum, exponentials and their
    // sum, scaling: reference src/Operation/OpNNLayerCpu.h:27-54) with one exponential per element — they are kept
    // as fp32 between the sum and the write.  (The running form below spends two per element: one for the statistics
    // and one for the result.)
    if (live) {
#pragma unroll
      for (int c = 0; c < KEEP; c++)
        if (lr + c * LPR < nvec) keep[c] = load_stream<T, VEC>(xr + (long long)(lr + c * LPR) * VEC);
#pragma unroll
      for (int c = 0; c < KEEP; c++)
        if (lr + c * LPR < nvec) {
#pragma unroll
          for (int e = 0; e < VEC; e++) mx = fmaxf(mx, (float)keep[c][e]);
        }
    }
    const float rmax = row_reduce<LPR, MaxOp>(mx, lds, 0);
    float ex[KEEP][VEC];
    if (live) {
#pragma unroll
      for (int c = 0; c < KEEP; c++)
        if (lr + c * LPR < nvec) {
#pragma unroll
          for (int e = 0; e < VEC; e++) {
            ex[c][e] = __expf((float)keep[c][e] - rmax);
            sum += ex[c][e];
          }
        }
    }
    sum = row_reduce<LPR, SumOp>(sum, lds, 1);
    if (!live) return;
    const float inv = 1.f / sum;
#pragma unroll
    for (int c = 0; c < KEEP; c++)
      if (lr + c * LPR < nvec) {
        V o;
#pragma unroll
        for (int e = 0; e < VEC; e++) o[e] = (T)(ex[c][e] * inv);
        store_pack<T, VEC>(orow + (long long)(lr + c * LPR) * VEC, o);
      }
    return;
  }
  if (live) {
#pragma unroll
    for (int c = 0; c < KEEP; c++)
      if (lr + c * LPR < nvec) keep[c] = load_stream<T, VEC>(xr + (long long)(lr + c * LPR) * VEC);
#pragma unroll
    for (int c = 0; c < KEEP; c++)
      if (lr + c * LPR < nvec) absorb(0, keep[c]);
    walk_rest<LPR, decltype(reload), decltype(absorb), KEEP>(lr, nvec, reload, absorb);
  }
  const float rmax = row_reduce<LPR, MaxOp>(mx, lds, 0);
  sum = row_reduce<LPR, SumOp>(sum * __expf(mx - rmax), lds, 1);
  if (!live) return;
  const float inv = 1.f / sum;
  const float lsum = LOG ? __logf(sum) : 0.f;
  auto give = [&](int i, const V& a) __attribute__((always_inline)) {
    V o;
#pragma unroll
    for (int e = 0; e < VEC; e++) {
      float v = (float)a[e] - rmax;
      o[e] = (T)(LOG ? v - lsum : __expf(v) * inv);
    }
    store_pack<T, VEC>(orow + (long long)i * VEC, o);
  };
#pragma unroll
  for (int c = 0; c < KEEP; c++)
    if (lr + c * LPR < nvec) give(lr + c * LPR, keep[c]);
  walk_rest<LPR, decltype(reload), decltype(give), KEEP>(lr, nvec, reload, give);
}

// ---- softmax / logSoftmax over an inner axis: a lane owns VEC neighbouring (outer, inner) columns, lanes run along the
// contiguous axis, four steps of the softmax axis are in flight ----------------------------------------------------------------
template <typename T, int VEC, bool LOG>
__global__ __launch_bounds__(256) void softmax_strided_kernel(const T* x, T* out, long long outer, int dim,  // out may be x
                                                              long long inner) {
  typedef typename Pack<T, VEC>::type V;
  const long long ivec = inner / VEC;  // column groups per outer index
  const long long cg = (long long)blockIdx.x * 256 + threadIdx.x;
  if (cg >= outer * ivec) return;
  const long long base = (cg / ivec) * dim * inner + (cg % ivec) * VEC;
  float mx[VEC], sum[VEC];
#pragma unroll
  for (int e = 0; e < VEC; e++) mx[e] = -3.402823466e+38f, sum[e] = 0.f;
  for (int d0 = 0; d0 < dim; d0 += 4) {  // running maximum and rescaled sum per column
    V v[4];
#pragma unroll
    for (int u = 0; u < 4; u++)
      if (d0 + u < dim) v[u] = load_plain<T, VEC>(x + base + (d0 + u) * inner);
#pragma unroll
    for (int e = 0; e < VEC; e++) {
      float mn = mx[e];
#pragma unroll
      for (int u = 0; u < 4; u++)
        if (d0 + u < dim) mn = fmaxf(mn, (float)v[u][e]);
      float acc = sum[e] * __expf(mx[e] - mn);
#pragma unroll
      for (int u = 0; u < 4; u++)
        if (d0 + u < dim) acc += __expf((float)v[u][e] - mn);
      sum[e] = acc, mx[e] = mn;
    }
  }
  float inv[VEC], lsum[VEC];
#pragma unroll
  for (int e = 0; e < VEC; e++) inv[e] = 1.f / sum[e], lsum[e] = LOG ? __logf(sum[e]) : 0.f;
  for (int d0 = 0; d0 < dim; d0 += 4) {
    V v[4];
#pragma unroll
    for (int u = 0; u < 4; u++)
      if (d0 + u < dim) v[u] = load_plain<T, VEC>(x + base + (d0 + u) * inner);
#pragma unroll
    for (int u = 0; u < 4; u++)
      if (d0 + u < dim) {
        V o;
#pragma unroll
        for (int e = 0; e < VEC; e++) {
          float t = (float)v[u][e] - mx[e];
          o[e] = (T)(LOG ? t - lsum[e] : __expf(t) * inv[e]);
        }
        store_pack<T, VEC>(out + base + (d0 + u) * inner, o);
      }
  }
}

// ---- siluMul --------------------------------------------------------------------------------------------------------------
// A workgroup is 2^txshift lanes along the row by 256 >> txshift rows and takes UNR consecutive row groups of one
// column chunk; workgroups are numbered with the chunk running fastest, so the launch walks memory front to back and
// no lane divides.
constexpr int kSiluUnroll = 4;

template <typename T, int VEC>
__global__ __launch_bounds__(256) void silu_mul_kernel(const T* __restrict__ x, T* __restrict__ out, long long rows, int d,
                                                       int txshift, unsigned nchunk) {
  typedef typename Pack<T, VEC>::type V;
  constexpr int UNR = kSiluUnroll;
  const int vpr = d / VEC;  // vectors per output row
  const int tx = threadIdx.x & ((1 << txshift) - 1), ty = threadIdx.x >> txshift;
  const unsigned chunk = blockIdx.x % nchunk, group = blockIdx.x / nchunk;
  const int col = (int)(chunk << txshift) + tx;
  if (col >= vpr) return;
  const int rpb = 256 >> txshift;
  const long long row0 = (long long)group * UNR * rpb + ty;
  V gv[UNR], uv[UNR];
#pragma unroll
  for (int u = 0; u < UNR; u++) {
    const long long row = row0 + u * rpb;
    if (row < rows) {
      const T* g = x + row * 2 * d + (long long)col * VEC;
      gv[u] = load_stream<T, VEC>(g);
      uv[u] = load_stream<T, VEC>(g + d);
    }
  }
#pragma unroll
  for (int u = 0; u < UNR; u++) {
    const long long row = row0 + u * rpb;
    if (row < rows) {
      V o;
#pragma unroll
      for (int e = 0; e < VEC; e++) {
        float gf = (float)gv[u][e];
        o[e] = (T)(gf / (1.f + __expf(-gf)) * (float)uv[u][e]);
      }
      store_pack<T, VEC>(out + row * d + (long long)col * VEC, o);
    }
  }
}

// ---- host side ---------------------------------------------------------------------------------------------------------------
bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

// lanes per row: the smallest of 8, 16, 32, 64 that leaves a lane at most two vectors, else the whole workgroup
// (128 lanes per row would need a reduction shape of its own)
int pick_lpr(long long nvec) {
  for (int lpr = 8; lpr <= 64; lpr *= 2)
    if (nvec <= 2LL * lpr) return lpr;
  return 256;
}

template <typename T, int VEC, bool FUSED>
int launch_rms(const void* x, void* res, const void* w, void* out, long long rows, int dim, float eps, hipStream_t s) {
  const int lpr = pick_lpr(dim / VEC);
  const long long rpb = 256 / lpr;
  const unsigned grid = (unsigned)((rows + rpb - 1) / rpb);
#define TT_RMS(LPR)                                                                                              \
  hipLaunchKernelGGL((rms_norm_kernel<T, VEC, LPR, FUSED>), dim3(grid), dim3(256), 0, s, (const T*)x, (T*)res, \
                     (const T*)w, (T*)out, rows, dim, eps)
  switch (lpr) {
    case 8: TT_RMS(8); break;
    case 16: TT_RMS(16); break;
    case 32: TT_RMS(32); break;
    case 64: TT_RMS(64); break;
    default: TT_RMS(256); break;
  }
#undef TT_RMS
  return (int)hipGetLastError();
}

template <typename T, int VEC, bool LOG>
int launch_softmax_rows(const void* x, void* out, long long rows, int dim, hipStream_t s) {
  const int lpr = pick_lpr(dim / VEC);
  const long long rpb = 256 / lpr;
  const unsigned grid = (unsigned)((rows + rpb - 1) / rpb);
#define TT_SM(LPR) \
  hipLaunchKernelGGL((softmax_rows_kernel<T, VEC, LPR, LOG, CACHE>), dim3(grid), dim3(256), 0, s, (const T*)x, (T*)out, rows, dim)
  switch (lpr) {
    case 8: TT_SM(8); break;
    case 16: TT_SM(16); break;
    case 32: TT_SM(32); break;
    case 64: TT_SM(64); break;
    default:
      if (dim / VEC > CACHE * 256 && dim / VEC <= 2 * CACHE * 256)  // a row of 8 to 16 vectors per lane: keep all of it
        hipLaunchKernelGGL((softmax_rows_kernel<T, VEC, 256, LOG, 2 * CACHE>), dim3(grid), dim3(256), 0, s, (const T*)x, (T*)out, rows, dim);
      else if (dim / VEC > 2 * CACHE * 256 && rows <= 2048)  // few rows, longer than 256 lanes keep: 1024 lanes per row
        hipLaunchKernelGGL((softmax_rows_kernel<T, VEC, 1024, LOG, CACHE>), dim3((unsigned)rows), dim3(1024), 0, s, (const T*)x, (T*)out, rows, dim);
      else
        TT_SM(256);
      break;
  }
#undef TT_SM
  return (int)hipGetLastError();
}

// ---- softmax / logSoftmax backward (reference src/Operation/OpNNLayerCpu.h:79-109, 123-150) -----------------------------
// softmax:    dx_j = y_j * (g_j - sum_t y_t g_t)        logSoftmax: dx_j = g_j - exp(y_j) * sum_t g_t
// over [outer, dim, inner]; inner == 1 is the last axis.  One workgroup lane group walks a row twice: the sum, then the
// result (the second read of a row comes from L2).  Lanes run along the contiguous axis in both layouts.
template <typename T, int VEC, int LPR, bool LOG>
__global__ __launch_bounds__(256) void softmax_backward_rows_kernel(const T* g, const T* y, T* out, long long rows, int dim) {
  typedef typename Pack<T, VEC>::type V;
  __shared__ float lds[4];
  constexpr int RPB = 256 / LPR;
  const int lr = threadIdx.x % LPR;
  const long long row = (long long)blockIdx.x * RPB + threadIdx.x / LPR;
  const bool live = row < rows;
  const int nvec = dim / VEC;
  const T* gr = g + row * dim;
  const T* yr = y + row * dim;
  float part = 0.f;
  if (live) {
    for (int i = lr; i < nvec; i += LPR) {
      const V a = load_plain<T, VEC>(gr + (long long)i * VEC);
      if (LOG) {
#pragma unroll
        for (int e = 0; e < VEC; e++) part += (float)a[e];
      } else {
        const V b = load_plain<T, VEC>(yr + (long long)i * VEC);
#pragma unroll
        for (int e = 0; e < VEC; e++) part = fmaf((float)a[e], (float)b[e], part);
      }
    }
  }
  const float sum = row_reduce<LPR, SumOp>(part, lds, 0);
  if (!live) return;
  for (int i = lr; i < nvec; i += LPR) {
    const V a = load_plain<T, VEC>(gr + (long long)i * VEC);
    const V b = load_stream<T, VEC>(yr + (long long)i * VEC);
    V o;
#pragma unroll
    for (int e = 0; e < VEC; e++) o[e] = (T)(LOG ? (float)a[e] - __expf((float)b[e]) * sum : (float)b[e] * ((float)a[e] - sum));
    store_pack<T, VEC>(out + row * dim + (long long)i * VEC, o);
  }
}

template <typename T, int VEC, bool LOG>
__global__ __launch_bounds__(256) void softmax_backward_strided_kernel(const T* g, const T* y, T* out, long long outer, int dim,
                                                                       long long inner) {
  typedef typename Pack<T, VEC>::type V;
  const long long ivec = inner / VEC;
  const long long cg = (long long)blockIdx.x * 256 + threadIdx.x;
  if (cg >= outer * ivec) return;
  const long long base = (cg / ivec) * dim * inner + (cg % ivec) * VEC;
  float sum[VEC];
#pragma unroll
  for (int e = 0; e < VEC; e++) sum[e] = 0.f;
  for (int d = 0; d < dim; d++) {
    const V a = load_plain<T, VEC>(g + base + d * inner);
    if (LOG) {
#pragma unroll
      for (int e = 0; e < VEC; e++) sum[e] += (float)a[e];
    } else {
      const V b = load_plain<T, VEC>(y + base + d * inner);
#pragma unroll
      for (int e = 0; e < VEC; e++) sum[e] = fmaf((float)a[e], (float)b[e], sum[e]);
    }
  }
  for (int d = 0; d < dim; d++) {
    const V a = load_plain<T, VEC>(g + base + d * inner);
    const V b = load_plain<T, VEC>(y + base + d * inner);
    V o;
#pragma unroll
    for (int e = 0; e < VEC; e++) o[e] = (T)(LOG ? (float)a[e] - __expf((float)b[e]) * sum[e] : (float)b[e] * ((float)a[e] - sum[e]));
    store_pack<T, VEC>(out + base + d * inner, o);
  }
}

template <typename T>
int softmax_backward_dispatch(const void* g, const void* y, void* out, long long outer, int dim, long long inner, bool log_form,
                              hipStream_t s) {
  constexpr int VEC = 16 / (int)sizeof(T);
  if (inner == 1) {
    const bool vec = dim % VEC == 0 && aligned16(g) && aligned16(y) && aligned16(out);
    const int lpr = pick_lpr(vec ? dim / VEC : dim);
    const long long rpb = 256 / lpr;
    const unsigned grid = (unsigned)((outer + rpb - 1) / rpb);
#define TT_SMB(V_, LPR_, LOG_) \
  hipLaunchKernelGGL((softmax_backward_rows_kernel<T, V_, LPR_, LOG_>), dim3(grid), dim3(256), 0, s, (const T*)g, (const T*)y, (T*)out, outer, dim)
#define TT_SMB_L(V_, LOG_)                  \
  switch (lpr) {                            \
    case 8: TT_SMB(V_, 8, LOG_); break;     \
    case 16: TT_SMB(V_, 16, LOG_); break;   \
    case 32: TT_SMB(V_, 32, LOG_); break;   \
    case 64: TT_SMB(V_, 64, LOG_); break;   \
    default: TT_SMB(V_, 256, LOG_); break;  \
  }
    if (vec) {
      if (log_form) { TT_SMB_L(VEC, true) } else { TT_SMB_L(VEC, false) }
    } else {
      if (log_form) { TT_SMB_L(1, true) } else { TT_SMB_L(1, false) }
    }
#undef TT_SMB_L
#undef TT_SMB
    return (int)hipGetLastError();
  }
  const bool vec = inner % VEC == 0 && aligned16(g) && aligned16(y) && aligned16(out);
  const long long groups = outer * (vec ? inner / VEC : inner);
  const unsigned grid = (unsigned)((groups + 255) / 256);
#define TT_SMBS(V_, LOG_) \
  hipLaunchKernelGGL((softmax_backward_strided_kernel<T, V_, LOG_>), dim3(grid), dim3(256), 0, s, (const T*)g, (const T*)y, (T*)out, outer, dim, inner)
  if (vec) {
    if (log_form) TT_SMBS(VEC, true); else TT_SMBS(VEC, false);
  } else {
    if (log_form) TT_SMBS(1, true); else TT_SMBS(1, false);
  }
#undef TT_SMBS
  return (int)hipGetLastError();
}

int check_common(int dtype, long long rows, long long dim) {
  if (dtype != TTSDPA_F32 && dtype != TTSDPA_F16 && dtype != TTSDPA_BF16) return TTSDPA_ERR_DTYPE;
  if (rows < 0 || dim < 0 || dim > 0x7fffffffLL) return TTSDPA_ERR_SHAPE;
  return TTSDPA_OK;
}

bool grid_ok(long long blocks) { return blocks <= 0x7fffffffLL; }

template <typename T>
int rms_dispatch(bool fused, const void* x, void* res, const void* w, void* out, long long rows, int dim, float eps,
                 hipStream_t s) {
  constexpr int VEC = 16 / (int)sizeof(T);
  const bool vec = dim % VEC == 0 && aligned16(x) && aligned16(out) && (!w || aligned16(w)) && (!fused || aligned16(res));
  if (fused) return vec ? launch_rms<T, VEC, true>(x, res, w, out, rows, dim, eps, s) : launch_rms<T, 1, true>(x, res, w, out, rows, dim, eps, s);
  return vec ? launch_rms<T, VEC, false>(x, res, w, out, rows, dim, eps, s) : launch_rms<T, 1, false>(x, res, w, out, rows, dim, eps, s);
}

template <typename T>
int softmax_dispatch(const void* x, void* out, long long outer, int dim, long long inner, bool log_form, hipStream_t s) {
  if (inner == 1) {
    constexpr int VEC = 16 / (int)sizeof(T);
    const bool vec = dim % VEC == 0 && aligned16(x) && aligned16(out);
    if (log_form) return vec ? launch_softmax_rows<T, VEC, true>(x, out, outer, dim, s) : launch_softmax_rows<T, 1, true>(x, out, outer, dim, s);
    return vec ? launch_softmax_rows<T, VEC, false>(x, out, outer, dim, s) : launch_softmax_rows<T, 1, false>(x, out, outer, dim, s);
  }
  constexpr int VEC = 16 / (int)sizeof(T);
  const bool vec = inner % VEC == 0 && aligned16(x) && aligned16(out);
  const long long groups = outer * (vec ? inner / VEC : inner);
  const unsigned grid = (unsigned)((groups + 255) / 256);
#define TT_SMS(V_, LOG_) \
  hipLaunchKernelGGL((softmax_strided_kernel<T, V_, LOG_>), dim3(grid), dim3(256), 0, s, (const T*)x, (T*)out, outer, dim, inner)
  if (vec) {
    if (log_form) TT_SMS(VEC, true); else TT_SMS(VEC, false);
  } else {
    if (log_form) TT_SMS(1, true); else TT_SMS(1, false);
  }
#undef TT_SMS
  return (int)hipGetLastError();
}

template <typename T>
int silu_dispatch(const void* x, void* out, long long rows, int d, hipStream_t s) {
  constexpr int VEC = 16 / (int)sizeof(T);
  const bool vec = d % VEC == 0 && aligned16(x) && aligned16(out);
  const int vpr = vec ? d / VEC : d;
  int txshift = 0;
  while (txshift < 8 && (1 << txshift) < vpr) txshift++;
  const long long rows_per_wg = (long long)(256 >> txshift) * kSiluUnroll;
  const unsigned nchunk = (unsigned)((vpr + (1 << txshift) - 1) >> txshift);
  const long long blocks = (rows + rows_per_wg - 1) / rows_per_wg * nchunk;
  if (!grid_ok(blocks)) return TTSDPA_ERR_SHAPE;
  if (vec)
    hipLaunchKernelGGL((silu_mul_kernel<T, VEC>), dim3((unsigned)blocks), dim3(256), 0, s, (const T*)x, (T*)out, rows, d, txshift, nchunk);
  else
    hipLaunchKernelGGL((silu_mul_kernel<T, 1>), dim3((unsigned)blocks), dim3(256), 0, s, (const T*)x, (T*)out, rows, d, txshift, nchunk);
  return (int)hipGetLastError();
}

}  // namespace
}  // namespace ttsdpa

using namespace ttsdpa;

extern "C" {

int ttfused_rms_norm(int dtype, const void* x, const void* weight, void* out, int64_t rows, int64_t dim, float eps,
                     void* stream) {
  int rc = check_common(dtype, rows, dim);
  if (rc != TTSDPA_OK) return rc;
  if (rows == 0 || dim == 0) return TTSDPA_OK;
  if (!x || !out) return TTSDPA_ERR_NULL;
  if (!grid_ok(rows)) return TTSDPA_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case TTSDPA_F32: return rms_dispatch<float>(false, x, nullptr, weight, out, rows, (int)dim, eps, s);
    case TTSDPA_F16: return rms_dispatch<_Float16>(false, x, nullptr, weight, out, rows, (int)dim, eps, s);
    default: return rms_dispatch<__bf16>(false, x, nullptr, weight, out, rows, (int)dim, eps, s);
  }
}

int ttfused_add_rms_norm(int dtype, void* input, void* residual, const void* weight, int64_t rows, int64_t dim,
                         float eps, void* stream) {
  int rc = check_common(dtype, rows, dim);
  if (rc != TTSDPA_OK) return rc;
  if (rows == 0 || dim == 0) return TTSDPA_OK;
  if (!input || !residual || !weight) return TTSDPA_ERR_NULL;
  if (!grid_ok(rows)) return TTSDPA_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case TTSDPA_F32: return rms_dispatch<float>(true, input, residual, weight, input, rows, (int)dim, eps, s);
    case TTSDPA_F16: return rms_dispatch<_Float16>(true, input, residual, weight, input, rows, (int)dim, eps, s);
    default: return rms_dispatch<__bf16>(true, input, residual, weight, input, rows, (int)dim, eps, s);
  }
}

int ttfused_silu_mul(int dtype, const void* x, void* out, int64_t rows, int64_t d, void* stream) {
  int rc = check_common(dtype, rows, d);
  if (rc != TTSDPA_OK) return rc;
  if (d > 0x3fffffffLL) return TTSDPA_ERR_SHAPE;
  if (rows == 0 || d == 0) return TTSDPA_OK;
  if (!x || !out) return TTSDPA_ERR_NULL;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case TTSDPA_F32: return silu_dispatch<float>(x, out, rows, (int)d, s);
    case TTSDPA_F16: return silu_dispatch<_Float16>(x, out, rows, (int)d, s);
    default: return silu_dispatch<__bf16>(x, out, rows, (int)d, s);
  }
}

int ttfused_softmax(int dtype, const void* x, void* out, int64_t outer, int64_t dim, int64_t inner, int log_form,
                    void* stream) {
  int rc = check_common(dtype, outer, dim);
  if (rc != TTSDPA_OK) return rc;
  if (inner < 0) return TTSDPA_ERR_SHAPE;
  if (outer == 0 || dim == 0 || inner == 0) return TTSDPA_OK;
  if (!x || !out) return TTSDPA_ERR_NULL;
  if (inner > 0x7fffffffLL || !grid_ok(outer) || outer > (0x7fffffffLL * 256) / inner) return TTSDPA_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case TTSDPA_F32: return softmax_dispatch<float>(x, out, outer, (int)dim, inner, log_form != 0, s);
    case TTSDPA_F16: return softmax_dispatch<_Float16>(x, out, outer, (int)dim, inner, log_form != 0, s);
    default: return softmax_dispatch<__bf16>(x, out, outer, (int)dim, inner, log_form != 0, s);
  }
}

int ttfused_softmax_backward(int dtype, const void* grad, const void* output, void* out, int64_t outer, int64_t dim,
                             int64_t inner, int log_form, void* stream) {
  int rc = check_common(dtype, outer, dim);
  if (rc != TTSDPA_OK) return rc;
  if (inner < 0) return TTSDPA_ERR_SHAPE;
  if (outer == 0 || dim == 0 || inner == 0) return TTSDPA_OK;
  if (!grad || !output || !out) return TTSDPA_ERR_NULL;
  if (inner > 0x7fffffffLL || !grid_ok(outer) || outer > (0x7fffffffLL * 256) / inner) return TTSDPA_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case TTSDPA_F32: return softmax_backward_dispatch<float>(grad, output, out, outer, (int)dim, inner, log_form != 0, s);
    case TTSDPA_F16: return softmax_backward_dispatch<_Float16>(grad, output, out, outer, (int)dim, inner, log_form != 0, s);
    default: return softmax_backward_dispatch<__bf16>(grad, output, out, outer, (int)dim, inner, log_form != 0, s);
  }
}

}  // extern "C"
