// General attention forward: any element type, any head_dim <= 256, optional causal / Bool / additive mask.
//
// One pass over the keys with a running (max, sum, accumulator) per query row — the result the reference's
// matmul -> scale -> bias -> softmax -> matmul chain produces (reference src/Function/FuncNNLayer.h:237-265),
// without materialising the [L,S] score matrix.  Arithmetic is fp32 on the vector ALUs; this is the route for
// fp32 tensors, attention masks and head sizes the MFMA kernels do not cover.
//
// Work split: a workgroup of 256 lanes owns 64 consecutive query rows of one (batch, head); four adjacent lanes
// share a row, lane s of the four holding head_dim elements s, s+4, s+8, ...  Keys and values are staged through
// LDS as fp32 tiles of 32 keys and read as broadcasts (all 16 rows of a wavefront read the same key).
//
// A row whose keys are all hidden keeps max = -FLT_MAX and sum = 0 and comes out as 0/0 = NaN, which is what the
// reference's softmax yields for such a row (reference src/Operation/OpNNLayerCpu.h:29-53).

#include <float.h>

#include "sdpa_common.h"

namespace ttsdpa {

namespace {

constexpr int kRows = 64;    // query rows per workgroup
constexpr int kTileK = 32;   // keys per LDS tile
constexpr int kChunk = 8;    // keys per online-softmax update

template <typename T, int DQ>  // DQ = head_dim elements per lane (head_dim <= 4*DQ)
__global__ __launch_bounds__(256) void general_kernel(KArgs a) {
  constexpr int DP = 4 * DQ;
  __shared__ float Ks[kTileK][DP];
  __shared__ float Vs[kTileK][DP];

  const int tid = threadIdx.x;
  const int sub = tid & 3;
  const int ntile_rows = (a.L + kRows - 1) / kRows;
  long long wg = blockIdx.x;
  const int rt = (int)(wg % ntile_rows);
  wg /= ntile_rows;
  const int h = (int)(wg % a.Hq);
  const int b = (int)(wg / a.Hq);
  const int hk = h / a.G;
  const int row0 = rt * kRows;
  const int row = row0 + (tid >> 2);
  const int rowc = row < a.L ? row : a.L - 1;

  const T* qp = (const T*)a.q + b * a.qs[0] + h * a.qs[1] + rowc * a.qs[2];
  const T* kp = (const T*)a.k + b * a.ks[0] + hk * a.ks[1];
  const T* vp = (const T*)a.v + b * a.vs[0] + hk * a.vs[1];
  const long long mrow = b * a.ms[0] + h * a.ms[1] + rowc * a.ms[2];  // a stride of 0 broadcasts that axis

  float qreg[DQ], acc[DQ];
#pragma unroll
  for (int t = 0; t < DQ; t++) {
    int d = 4 * t + sub;
    qreg[t] = d < a.D ? load_as_float(qp + d) : 0.f;
    acc[t] = 0.f;
  }
  float m = -FLT_MAX, l = 0.f;

  int S = a.S;  // keys of this batch entry: all of them, or the filled prefix of a cache
  if (a.kv_len) {
    int len = a.kv_len[b];
    S = len < 0 ? 0 : (len < S ? len : S);
  }
  int send = S;
  const int coff = causal_offset(a, S);
  if (a.causal) {
    int last = (row0 + kRows - 1 < a.L - 1 ? row0 + kRows - 1 : a.L - 1) + coff;
    send = last + 1 < S ? last + 1 : S;
  }

  for (int k0 = 0; k0 < send; k0 += kTileK) {
    __syncthreads();
    for (int e = tid; e < kTileK * DP; e += 256) {
      int kk = e / DP, d = e % DP;
      int key = k0 + kk;
      float kv = 0.f, vv = 0.f;
      if (key < S && d < a.D) {
        if (a.block_table) {  // paged cache: page pools [pages, Hkv, page_size, D]
          const long long page = a.block_table[(long long)b * a.bt_stride + (key >> a.page_shift)];
          const int row = key & ((1 << a.page_shift) - 1);
          kv = load_as_float((const T*)a.k + page * a.ks[0] + hk * a.ks[1] + row * a.ks[2] + d);
          vv = load_as_float((const T*)a.v + page * a.vs[0] + hk * a.vs[1] + row * a.vs[2] + d);
        } else {
          kv = load_as_float(kp + key * a.ks[2] + d);
          vv = load_as_float(vp + key * a.vs[2] + d);
        }
      }
      Ks[kk][d] = kv;
      Vs[kk][d] = vv;
    }
    __syncthreads();

    for (int c0 = 0; c0 < kTileK; c0 += kChunk) {
      if (k0 + c0 >= send) break;
      float s[kChunk];
      float cmax = -INFINITY;
#pragma unroll
      for (int j = 0; j < kChunk; j++) {
        float part = 0.f;
#pragma unroll
        for (int t = 0; t < DQ; t++) part = fmaf(qreg[t], Ks[c0 + j][4 * t + sub], part);
        part += __shfl_xor(part, 1);
        part += __shfl_xor(part, 2);
        float x = part * a.scale;
        int key = k0 + c0 + j;
        bool hidden = key >= S || (a.causal && key > row + coff);
        if (a.mask_kind == 1) {
          if (key < S && ((const uint8_t*)a.mask)[mrow + key * a.ms[3]] == 0) hidden = true;
        } else if (a.mask_kind == 2) {
          if (key < S) x += load_as_float((const T*)a.mask + mrow + key * a.ms[3]);
        }
        if (hidden) x = -INFINITY;
        s[j] = x;
        cmax = fmaxf(cmax, x);
      }
      float mn = fmaxf(m, cmax);  // stays -FLT_MAX while every key so far is hidden
      float alpha = __expf(m - mn);
      float psum = 0.f;
#pragma unroll
      for (int j = 0; j < kChunk; j++) {
        s[j] = __expf(s[j] - mn);
        psum += s[j];
      }
      l = l * alpha + psum;
      m = mn;
#pragma unroll
      for (int t = 0; t < DQ; t++) {
        float o = acc[t] * alpha;
#pragma unroll
        for (int j = 0; j < kChunk; j++) o = fmaf(s[j], Vs[c0 + j][4 * t + sub], o);
        acc[t] = o;
      }
    }
  }

  if (row < a.L) {
    T* op = (T*)a.out + b * a.os[0] + h * a.os[1] + row * a.os[2];
    float inv = S == 0 ? 0.f : 1.f / l;  // no keys: zeros (the reference's empty contraction); hidden rows: NaN
#pragma unroll
    for (int t = 0; t < DQ; t++) {
      int d = 4 * t + sub;
      if (d < a.D) store_from_float(op + d, acc[t] * inv);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void zero_kernel(KArgs a) {
  long long n = (long long)a.B * a.Hq * a.L * a.D;
  long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  int d = (int)(i % a.D);
  long long r = i / a.D;
  int row = (int)(r % a.L);
  r /= a.L;
  int h = (int)(r % a.Hq);
  int b = (int)(r / a.Hq);
  store_from_float((T*)a.out + b * a.os[0] + h * a.os[1] + row * a.os[2] + d, 0.f);
}

template <typename T>
int launch_general_t(const KArgs& a, hipStream_t stream) {
  long long nwg = (long long)a.B * a.Hq * ((a.L + kRows - 1) / kRows);
  dim3 grid((unsigned)nwg), block(256);
  if (a.D <= 32) {
    hipLaunchKernelGGL((general_kernel<T, 8>), grid, block, 0, stream, a);
  } else if (a.D <= 64) {
    hipLaunchKernelGGL((general_kernel<T, 16>), grid, block, 0, stream, a);
  } else if (a.D <= 128) {
    hipLaunchKernelGGL((general_kernel<T, 32>), grid, block, 0, stream, a);
  } else {
    hipLaunchKernelGGL((general_kernel<T, 64>), grid, block, 0, stream, a);
  }
  return (int)hipGetLastError();
}

}  // namespace

int launch_general(const KArgs& a, int dtype, hipStream_t stream) {
  switch (dtype) {
    case 0: return launch_general_t<float>(a, stream);
    case 1: return launch_general_t<_Float16>(a, stream);
    default: return launch_general_t<__bf16>(a, stream);
  }
}

int launch_zero(const KArgs& a, int dtype, hipStream_t stream) {
  long long n = (long long)a.B * a.Hq * a.L * a.D;
  dim3 grid((unsigned)((n + 255) / 256)), block(256);
  switch (dtype) {
    case 0: hipLaunchKernelGGL((zero_kernel<float>), grid, block, 0, stream, a); break;
    case 1: hipLaunchKernelGGL((zero_kernel<_Float16>), grid, block, 0, stream, a); break;
    default: hipLaunchKernelGGL((zero_kernel<__bf16>), grid, block, 0, stream, a); break;
  }
  return (int)hipGetLastError();
}

}  // namespace ttsdpa
