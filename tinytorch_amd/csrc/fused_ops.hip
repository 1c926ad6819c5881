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
  if constexpr (VEC == 1) {
    *p = v.x;
  } else {
    *(V*)p = v;
  }
}

struct SumOp {
  static __device__ __forceinline__ float apply(float a, float b) { return a + b; }
};
struct MaxOp {
  static __device__ __forceinline__ float apply(float a, float b) { return fmaxf(a, b); }
};

// Reduction over the LPR lanes of a row; every lane of the row gets the result.  LPR <= 64: butterfly inside the
// wavefront.  LPR == 256: the workgroup is one row; wavefront totals cross through LDS (`slot` tells successive
// reductions of one kernel apart, so one barrier per reduction suffices).
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
  }
  return v;
}

// ---- rmsNorm and fusedAddRmsNorm ---------------------------------------------------------------------------------
// FUSED: r = input + residual, residual <- T(r), sum of squares over the unrounded r, input <- T(float(T(r)) * inv * w).
// else:  out <- T(x * inv [* w]).
template <typename T, int VEC, int LPR, bool FUSED>
__global__ __launch_bounds__(256) void rms_norm_kernel(const T* x, T* res, const T* __restrict__ w, T* out,  // out may be x
                                                       long long rows,
                                                       int dim, float eps) {
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
  auto take = [&](int i) __attribute__((always_inline)) {
    V a = load_stream<T, VEC>(xr + (long long)i * VEC);
    if constexpr (FUSED) {
      V b = load_stream<T, VEC>(rr + (long long)i * VEC);
#pragma unroll
      for (int e = 0; e < VEC; e++) {
        float r = (float)a[e] + (float)b[e];
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
#pragma unroll
    for (int c = 0; c < CACHE; c++) {
      int i = lr + c * LPR;
      if (i < nvec) keep[c] = take(i);
    }
    for (int i = lr + CACHE * LPR; i < nvec; i += LPR) take(i);
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
  for (int c = 0; c < CACHE; c++) {
    int i = lr + c * LPR;
    if (i < nvec) give(i, keep[c]);
  }
  for (int i = lr + CACHE * LPR; i < nvec; i += LPR)  // the part of a very long row that was not kept
    give(i, load_plain<T, VEC>((FUSED ? rr : xr) + (long long)i * VEC));
}

// ---- softmax / logSoftmax over the last axis ---------------------------------------------------------------------------
template <typename T, int VEC, int LPR, bool LOG>
__global__ __launch_bounds__(256) void softmax_rows_kernel(const T* x, T* out, long long rows, int dim) {  // out may be x
  typedef typename Pack<T, VEC>::type V;
  __shared__ float lds[8];
  constexpr int RPB = 256 / LPR;
  const int lr = threadIdx.x % LPR;
  const long long row = (long long)blockIdx.x * RPB + threadIdx.x / LPR;
  const bool live = row < rows;
  const int nvec = dim / VEC;
  const T* xr = x + row * dim;
  T* orow = out + row * dim;

  V keep[CACHE];
  float mx = -3.402823466e+38f;  // the reference starts from the lowest finite float
  if (live) {
#pragma unroll
    for (int c = 0; c < CACHE; c++) {
      int i = lr + c * LPR;
      if (i < nvec) {
        keep[c] = load_stream<T, VEC>(xr + (long long)i * VEC);
#pragma unroll
        for (int e = 0; e < VEC; e++) mx = fmaxf(mx, (float)keep[c][e]);
      }
    }
    for (int i = lr + CACHE * LPR; i < nvec; i += LPR) {
      V a = load_plain<T, VEC>(xr + (long long)i * VEC);
#pragma unroll
      for (int e = 0; e < VEC; e++) mx = fmaxf(mx, (float)a[e]);
    }
  }
  mx = row_reduce<LPR, MaxOp>(mx, lds, 0);
  float sum = 0.f;
  if (live) {
#pragma unroll
    for (int c = 0; c < CACHE; c++) {
      int i = lr + c * LPR;
      if (i < nvec) {
#pragma unroll
        for (int e = 0; e < VEC; e++) sum += __expf((float)keep[c][e] - mx);
      }
    }
    for (int i = lr + CACHE * LPR; i < nvec; i += LPR) {
      V a = load_plain<T, VEC>(xr + (long long)i * VEC);
#pragma unroll
      for (int e = 0; e < VEC; e++) sum += __expf((float)a[e] - mx);
    }
  }
  sum = row_reduce<LPR, SumOp>(sum, lds, 1);
  if (!live) return;
  const float inv = 1.f / sum;
  const float lsum = LOG ? __logf(sum) : 0.f;
  auto give = [&](int i, const V& a) __attribute__((always_inline)) {
    V o;
#pragma unroll
    for (int e = 0; e < VEC; e++) {
      float v = (float)a[e] - mx;
      o[e] = (T)(LOG ? v - lsum : __expf(v) * inv);
    }
    store_pack<T, VEC>(orow + (long long)i * VEC, o);
  };
#pragma unroll
  for (int c = 0; c < CACHE; c++) {
    int i = lr + c * LPR;
    if (i < nvec) give(i, keep[c]);
  }
  for (int i = lr + CACHE * LPR; i < nvec; i += LPR) give(i, load_plain<T, VEC>(xr + (long long)i * VEC));
}

// ---- softmax / logSoftmax over an inner axis: one lane per (outer, inner) column, lanes along the contiguous axis --------
template <typename T, bool LOG>
__global__ __launch_bounds__(256) void softmax_strided_kernel(const T* x, T* out, long long outer, int dim,  // out may be x
                                                              long long inner) {
  const long long col = (long long)blockIdx.x * 256 + threadIdx.x;
  if (col >= outer * inner) return;
  const long long base = (col / inner) * dim * inner + col % inner;
  float mx = -3.402823466e+38f, sum = 0.f;
  for (int d = 0; d < dim; d++) {  // one pass: running maximum and rescaled sum
    float v = (float)x[base + d * inner];
    float mn = fmaxf(mx, v);
    sum = sum * __expf(mx - mn) + __expf(v - mn);
    mx = mn;
  }
  const float inv = 1.f / sum;
  const float lsum = LOG ? __logf(sum) : 0.f;
  for (int d = 0; d < dim; d++) {
    float v = (float)x[base + d * inner] - mx;
    out[base + d * inner] = (T)(LOG ? v - lsum : __expf(v) * inv);
  }
}

// ---- siluMul --------------------------------------------------------------------------------------------------------------
template <typename T, int VEC>
__global__ __launch_bounds__(256) void silu_mul_kernel(const T* __restrict__ x, T* __restrict__ out, long long rows, int d) {
  typedef typename Pack<T, VEC>::type V;
  const int vpr = d / VEC;  // vectors per output row
  const long long total = rows * vpr;
  for (long long idx = (long long)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (long long)gridDim.x * 256) {
    const long long row = idx / vpr;
    const int col = (int)(idx % vpr) * VEC;
    const T* g = x + row * 2 * d + col;
    V gv = load_stream<T, VEC>(g);
    V uv = load_stream<T, VEC>(g + d);
    V o;
#pragma unroll
    for (int e = 0; e < VEC; e++) {
      float gf = (float)gv[e];
      o[e] = (T)(gf / (1.f + __expf(-gf)) * (float)uv[e]);
    }
    store_pack<T, VEC>(out + row * d + col, o);
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
  hipLaunchKernelGGL((softmax_rows_kernel<T, VEC, LPR, LOG>), dim3(grid), dim3(256), 0, s, (const T*)x, (T*)out, rows, dim)
  switch (lpr) {
    case 8: TT_SM(8); break;
    case 16: TT_SM(16); break;
    case 32: TT_SM(32); break;
    case 64: TT_SM(64); break;
    default: TT_SM(256); break;
  }
#undef TT_SM
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
  const long long cols = outer * inner;
  const unsigned grid = (unsigned)((cols + 255) / 256);
  if (log_form)
    hipLaunchKernelGGL((softmax_strided_kernel<T, true>), dim3(grid), dim3(256), 0, s, (const T*)x, (T*)out, outer, dim, inner);
  else
    hipLaunchKernelGGL((softmax_strided_kernel<T, false>), dim3(grid), dim3(256), 0, s, (const T*)x, (T*)out, outer, dim, inner);
  return (int)hipGetLastError();
}

template <typename T>
int silu_dispatch(const void* x, void* out, long long rows, int d, hipStream_t s) {
  constexpr int VEC = 16 / (int)sizeof(T);
  const bool vec = d % VEC == 0 && aligned16(x) && aligned16(out);
  const long long total = rows * (vec ? d / VEC : d);
  long long blocks = (total + 255) / 256;
  const long long cap = 256LL * 32;  // grid-stride beyond 32 workgroups per CU
  if (blocks > cap) blocks = cap;
  if (vec)
    hipLaunchKernelGGL((silu_mul_kernel<T, VEC>), dim3((unsigned)blocks), dim3(256), 0, s, (const T*)x, (T*)out, rows, d);
  else
    hipLaunchKernelGGL((silu_mul_kernel<T, 1>), dim3((unsigned)blocks), dim3(256), 0, s, (const T*)x, (T*)out, rows, d);
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

}  // extern "C"
