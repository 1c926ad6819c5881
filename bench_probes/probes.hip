// Measurement probes: what this GPU sustains on the two resources the attention kernels are bound by.  Bench tooling, built
// into a shared object of its own (libttbench_probes.so) that only bench.py and its test load; the product library does
// not contain it.  A roofline fraction can then also be read against the rate the hardware actually delivers (the matrix
// pipe under its power limit, HBM for a streaming read).
//   mfma_probe_kernel   register-only loop of v_mfma_f32_32x32x16_bf16, two accumulators per wavefront, eight wavefronts
//                       per workgroup (two per SIMD): 32768 flop per MFMA, no memory traffic.  RANDOM: the operands are
//                       random bf16 values (sign, mantissa, exponents 2^-3 .. 2^0) instead of small constants: the chip's
//                       power management lowers the clock under such operands, so this is the rate the matrix pipe
//                       sustains on data like the attention kernels'.
//   read_probe_kernel   every workgroup streams a contiguous chunk of a buffer with 16-byte loads, plain or nontemporal.
//
//   int ttbench_probe(int kind, void* buffer, size_t bytes, int iters, void* stream, double* work)
//     kind 0: matrix pipe, constant operands; 1: streaming read; 2: nontemporal streaming read; 3: matrix pipe, random
//     operands.  buffer: device memory, 16-byte aligned (64 bytes suffice for kinds 0 and 3).  *work = flop or bytes of
//     the enqueued launch.  Returns 0, or -1 for bad arguments, or a hipError_t.

#include <hip/hip_runtime.h>
#include <cstddef>
#include <cstdint>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

namespace {

__device__ unsigned probe_mix(unsigned x) { x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16; return x; }

template <bool RANDOM>
__global__ __launch_bounds__(512) void mfma_probe_kernel(float* out, int iters) {
  bf16x8 x, y;
#pragma unroll
  for (int i = 0; i < 8; i++) {
    x[i] = (__bf16)(0.001f * (float)(threadIdx.x & 63) + (float)i);
    y[i] = (__bf16)(0.5f * (float)i);
  }
  if (RANDOM) {
    u32x4 xr, yr;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const unsigned h = probe_mix((blockIdx.x * 512u + threadIdx.x) * 8u + i), g = probe_mix(h);
      xr[i] = ((h & 0x80ffu) | ((124u + ((h >> 8) & 3u)) << 7)) | (((h >> 16) & 0x80ffu) | ((124u + ((h >> 24) & 3u)) << 7)) << 16;
      yr[i] = ((g & 0x80ffu) | ((124u + ((g >> 8) & 3u)) << 7)) | (((g >> 16) & 0x80ffu) | ((124u + ((g >> 24) & 3u)) << 7)) << 16;
    }
    x = __builtin_bit_cast(bf16x8, xr);
    y = __builtin_bit_cast(bf16x8, yr);
  }
  f32x16 acc0, acc1;
#pragma unroll
  for (int r = 0; r < 16; r++) acc0[r] = 0.f, acc1[r] = 0.f;
  for (int it = 0; it < iters; it++) {
    acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x, y, acc0, 0, 0, 0);
    acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(y, x, acc1, 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int r = 0; r < 16; r++) s += acc0[r] + acc1[r];
  if (s == 12345.678f) out[0] = s;  // keeps the loop alive; practically never true
}

template <bool NT>
__global__ __launch_bounds__(256) void read_probe_kernel(const u32x4* __restrict__ p, long long n_per_wg, float* out) {
  const u32x4* base = p + (long long)blockIdx.x * n_per_wg;
  uint32_t acc = 0;
  for (long long i = threadIdx.x; i + 7 * 256 < n_per_wg; i += 8 * 256) {
    u32x4 v[8];
#pragma unroll
    for (int u = 0; u < 8; u++) v[u] = NT ? __builtin_nontemporal_load(base + i + u * 256) : base[i + u * 256];
#pragma unroll
    for (int u = 0; u < 8; u++) acc += v[u][0] ^ v[u][1] ^ v[u][2] ^ v[u][3];
  }
  if (acc == 0x12345679u) out[0] = 1.f;
}

}  // namespace

extern "C" int ttbench_probe(int kind, void* buffer, size_t bytes, int iters, void* stream_, double* work) {
  hipStream_t stream = (hipStream_t)stream_;
  if (!buffer || !work || kind < 0 || kind > 3 || iters < 1 || ((uintptr_t)buffer & 15) != 0) return -1;
  if (kind == 0 || kind == 3) {  // matrix pipe
    if (bytes < 64) return -1;
    if (kind == 0) hipLaunchKernelGGL(mfma_probe_kernel<false>, dim3(256), dim3(512), 0, stream, (float*)buffer, iters);
    else hipLaunchKernelGGL(mfma_probe_kernel<true>, dim3(256), dim3(512), 0, stream, (float*)buffer, iters);
    *work = 256.0 * 8.0 * (double)iters * 2.0 * 32768.0;  // flop
    return (int)hipGetLastError();
  }
  const int wgs = 2048;
  long long n_per_wg = (long long)(bytes / 16 / wgs) / 2048 * 2048;  // whole passes of 8 x 256 loads
  if (n_per_wg < 2048) return -1;
  if (kind == 1) hipLaunchKernelGGL(read_probe_kernel<false>, dim3(wgs), dim3(256), 0, stream, (const u32x4*)buffer, n_per_wg, (float*)buffer);
  else hipLaunchKernelGGL(read_probe_kernel<true>, dim3(wgs), dim3(256), 0, stream, (const u32x4*)buffer, n_per_wg, (float*)buffer);
  *work = (double)n_per_wg * 16.0 * wgs;  // bytes read
  return (int)hipGetLastError();
}
