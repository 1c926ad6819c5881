// Shared device-side definitions for the gfx950 attention kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ttsdpa {

// Kernel argument block: the validated contents of ttsdpa_params plus derived values.
struct KArgs {
  const void* q;
  const void* k;
  const void* v;
  void* out;
  const void* mask;
  const int* kv_len;  // per-batch valid key count (device), or nullptr
  const int* block_table;  // paged cache: page of key j of batch b = block_table[b * bt_stride + (j >> page_shift)], or nullptr
  int page_shift, bt_stride;
  int B, Hq, Hkv, L, S, D;
  int G;  // Hq / Hkv: query heads per KV head
  int causal;     // key j is visible to query i iff j <= i + offset
  int causal_br;  // offset: 0 (top-left aligned, the reference's mask) or max(0, keys of the batch entry - L) (bottom-right)
  int mask_kind;
  float scale;
  long long qs[3], ks[3], vs[3], os[3];  // element strides: batch, head, sequence
  long long ms[4];                       // mask element strides: batch, head, query row, key (0 = broadcast)
  // Packed query heads (4-wavefront prefill kernel only): the G query heads of a KV head are presented as one head of
  // G * pack_L rows (dense q / out make that a plain reshape); row x is query position x % pack_L.  0 = not packed.
  int pack_L;
  // Split keys (4-wavefront prefill kernel, one query head per KV head after packing): workgroup (.., split) covers keys
  // split * kv_chunk .. + kv_chunk - 1 and writes a (acc[D], max, sum) record per row to ws instead of the output;
  // the decode path's merge kernel combines them.  kv_splits <= 1: no split.
  int kv_splits, kv_chunk;
  float* ws;
  int mask_vec4;  // keys are contiguous in the mask and groups of 4 keys starting at a multiple of 4 are naturally aligned
  // Pipelined prefill kernels under a causal mask: 0 = a workgroup takes a row tile and its mirror (equal work for all),
  // 1 = one row tile per workgroup, longest first (launches whose pairs would leave CUs without a workgroup).
  int single_tiles;
};

// Offset of the causal diagonal in key coordinates for a batch entry with S keys.
__device__ __forceinline__ int causal_offset(const KArgs& a, int S) {
  const int d = S - (a.pack_L ? a.pack_L : a.L);
  return (a.causal_br && d > 0) ? d : 0;
}

// Element offset of key tile kv0 (a multiple of the tile length, which divides the page size) from the K or V pointer
// of a (batch, kv head): `table` is the batch entry's row of the block table, or nullptr for a contiguous cache.  For
// paged caches the (batch, kv head) pointer carries the head offset only: pstride is the pool's page stride.
__device__ __forceinline__ long long kv_tile_offset(const KArgs& a, const int* table, int kv0, long long rstride, long long pstride) {
  if (!table) return (long long)kv0 * rstride;
  const int page = __builtin_amdgcn_readfirstlane(table[kv0 >> a.page_shift]);
  return (long long)page * pstride + (long long)(kv0 & ((1 << a.page_shift) - 1)) * rstride;
}

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr float kLog2e = 1.4426950408889634f;

// Kernels that use more than 64 KiB of dynamic LDS need that granted per kernel and per device.  Done on the first
// launch on a device (the device is the current one of the calling thread) and remembered; safe from several host
// threads (the worst case is granting twice).
constexpr int kMaxDevices = 64;
constexpr int kCusPerXcd = 32;  // MI355X: 256 compute units in 8 XCDs, each XCD with an L2 of its own
inline hipError_t grant_dynamic_lds(const void* kernel, int bytes, hipError_t (&state)[kMaxDevices], bool (&done)[kMaxDevices]) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= kMaxDevices) return hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (!__atomic_load_n(&done[dev], __ATOMIC_ACQUIRE)) {
    state[dev] = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    __atomic_store_n(&done[dev], true, __ATOMIC_RELEASE);
  }
  return state[dev];
}

// Element-type traits: storage is 16-bit (or fp32 for the general kernel), arithmetic is fp32.
struct BF16 {
  typedef __bf16 elem;
  typedef bf16x8 vec8;
  typedef bf16x4 vec4;
  static __device__ __forceinline__ f32x16 mfma32(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 mfma16(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  // fp32 value of the low / high 16-bit half of a packed pair
  static __device__ __forceinline__ float lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
  static __device__ __forceinline__ float hi(uint32_t w) { return __builtin_bit_cast(float, w & 0xffff0000u); }
};

struct F16 {
  typedef _Float16 elem;
  typedef f16x8 vec8;
  typedef f16x4 vec4;
  static __device__ __forceinline__ f32x16 mfma32(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 mfma16(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ float lo(uint32_t w) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)(w & 0xffffu));
  }
  static __device__ __forceinline__ float hi(uint32_t w) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)(w >> 16));
  }
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ float load_as_float(const float* p) { return *p; }
__device__ __forceinline__ float load_as_float(const __bf16* p) { return (float)*p; }
__device__ __forceinline__ float load_as_float(const _Float16* p) { return (float)*p; }
__device__ __forceinline__ void store_from_float(float* p, float x) { *p = x; }
__device__ __forceinline__ void store_from_float(__bf16* p, float x) { *p = (__bf16)x; }
__device__ __forceinline__ void store_from_float(_Float16* p, float x) { *p = (_Float16)x; }

// attnMask applied to the 32 x 32 score block of an MFMA accumulator (reference src/Function/FuncNNLayer.h:249-260):
// a lane holds one query row (mask row offset `mrow`, in elements) and, in register group rg, the four consecutive
// keys kv0 + 8*rg + 4*lh .. +3.  Bool: hidden keys get -inf; additive: the bias joins the scaled score, i.e.
// bias * inv_scale the raw score held here.  Element strides of 0 broadcast an axis.  Keys at or beyond S are left
// alone (masked by the caller).  With a.mask_vec4 a group of four keys is one load.  VEC_ONLY: the caller guarantees
// a.mask_vec4 and S % 4 == 0, and the element-wise path (and its registers) is left out.
template <typename T, bool VEC_ONLY>
__device__ __forceinline__ void apply_attn_mask(const KArgs& a, f32x16& s, long long mrow, int kv0, int lh, int S,
                                                float inv_scale) {
#pragma unroll
  for (int rg = 0; rg < 4; rg++) {
    const int key0 = kv0 + 8 * rg + 4 * lh;
    if (VEC_ONLY && key0 >= S) continue;
    if (VEC_ONLY || (a.mask_vec4 && key0 + 3 < S)) {
      const long long at = mrow + key0;
      if (a.mask_kind == 1) {
        const uint32_t w = *(const uint32_t*)((const uint8_t*)a.mask + at);
#pragma unroll
        for (int e = 0; e < 4; e++)
          if (((w >> (8 * e)) & 0xffu) == 0) s[4 * rg + e] = -INFINITY;
      } else {
        typedef T vec4t __attribute__((ext_vector_type(4)));
        const vec4t w = *(const vec4t*)((const T*)a.mask + at);
#pragma unroll
        for (int e = 0; e < 4; e++) s[4 * rg + e] += (float)w[e] * inv_scale;
      }
    } else {
#pragma unroll
      for (int e = 0; e < 4; e++) {
        const int key = key0 + e;
        if (key < S) {
          const long long at = mrow + key * a.ms[3];
          if (a.mask_kind == 1) {
            if (((const uint8_t*)a.mask)[at] == 0) s[4 * rg + e] = -INFINITY;
          } else {
            s[4 * rg + e] += (float)((const T*)a.mask)[at] * inv_scale;
          }
        }
      }
    }
  }
}

// Backward call: the forward's arguments (f.out holds the forward's result, an input here) plus the upstream gradient
// and the three gradients to write.  stats is scratch [B,Hq,L,2] floats: per query row the log of the sum of
// exponentials of its scaled, biased scores (natural log in the vector-ALU kernels, log2 in the MFMA kernels: the two
// kernels of a call are always of one family), and delta = dout . out.
struct BwdArgs {
  KArgs f;
  const void* dout;
  void* dq;
  void* dk;
  void* dv;
  long long dos[3], dqs[3], dks[3], dvs[3];  // element strides: batch, head, sequence
  float* stats;
  // matrix-core pairs only: with dkv_splits > 1 the query stream of every key block is dealt out to that many
  // workgroups, which leave partial dk / dv in `partial` ([split][dk | dv][B][Hkv][S][D] floats) for a third kernel to add.
  float* partial;
  int dkv_splits;
  // matrix-core pairs only: with dq_splits > 1 the key range of every 128-row query block is dealt out to that many
  // workgroups of the dq kernel, which leave their unnormalised fp32 sums in `dq_partial` ([split][B][Hq][L][D] floats,
  // then [split][B][Hq][L] pairs (maximum in log2 units, sum of exponentials)) for backward_dq_merge_kernel.
  float* dq_partial;
  int dq_splits;
  // dk/dv kernels under a causal mask: workgroups of an XCD that run together (CUs per XCD x workgroups per CU), or 0.
  // The workgroups of every second such round walk their query tiles upwards (dkv_walks_up).
  int dkv_round;
};

// Workgroups that share a key block in the matrix-core dk/dv kernels (1: none, the kernel writes dk / dv itself).
// A dk/dv workgroup owns 128 keys and about one runs per CU at a time; under a causal mask its length varies
// 1 : (number of key blocks), and below about four workgroups per CU the longest ones set the time.  Without a causal
// mask all are equally long and splitting only serves to give every CU one (splitting 256 equal workgroups further
// measured 1 % slower, 13-20 % with an attnMask).  A split must still get a few tiles.  `groups`: wavefront groups
// that already share a key block inside a workgroup (2 in the 16-bit head_dim-128 kernel, where splitting 512
// workgroups of a causal call further measured 4 % slower, 256 of them 7-21 % faster).
// `per_cu`: workgroups of the kernel that fit a CU (2 at head_dim 64 without an attnMask, else 1): head_dim 64, 256 equal
// workgroups without a causal mask: two splits +28 %; causal with 512: four splits instead of two -2 to -5 %.
inline int backward_dkv_splits(int B, int Hkv, int Hq, int L, int S, bool causal, int groups, int per_cu) {
  const long long wgs = (long long)B * Hkv * ((S + 127) / 128) * groups;
  const long long tiles = (long long)(Hq / Hkv) * ((L + 31) / 32) / groups;  // the longest query stream, in 32-row tiles
  // causal: two rounds of the workgroups a CU holds at a time (one for the 8-wavefront head_dim-128 kernel, whose two
  // groups make `wgs` count double, and for the fp32 head_dim-128 kernel; two at head_dim 64).  fp32 head_dim 128, 512
  // workgroups (B2 32q/8kv 4096 x 4096): splitting them in two measured the same time, 60 % more bytes read and a
  // third kernel for the partial sums; 256 of them (2048 x 2048) two splits 76.5, four 74.1 TFLOP/s.
  const long long enough = causal ? 512LL * per_cu * groups : 256 * per_cu;
  int n = 1;
  while (n < 4 && wgs * n < enough && tiles >= 16 * n) n *= 2;
  return n;
}

// Workgroups that share a 128-row query block in the matrix-core dq kernels (1: none, the kernel writes dq itself).
// Two of its workgroups fit a CU (512 at a time on the chip).  A launch of fewer is split: that gives every slot a
// workgroup, and under a causal mask, where their lengths vary 1 : (number of row blocks) and they start longest first,
// a second round to end evenly
// (bf16 head_dim 128, one batch entry: 8 heads 4096 x 4096 causal +26 %, 32 heads 512 x 8192 +46 %, 8 heads 2048 x 2048
// without a mask +22 %; 512 causal workgroups split in two measured 5 % slower: the partial records cost more than the
// uneven end).  A split must still get a few hundred keys.
// `slots`: workgroups of the kernel the chip holds at a time (512; 256 for the fp32 kernel at head_dim 128).
inline int backward_dq_splits(int B, int Hq, int L, int S, bool causal, int slots) {
  const long long wgs = (long long)B * Hq * ((L + 127) / 128);
  const long long tiles = (S + 31) / 32;  // the longest key range, in 32-key tiles
  if (wgs >= slots) return 1;
  const long long enough = causal ? 2 * slots : slots;
  int n = 1;
  while (n < 8 && wgs * n < enough && tiles >= 16 * n) n *= 2;
  return n;
}

// Workgroup id of a dk/dv launch with split query streams -> (key-block workgroup n, split).  The hardware hands
// workgroup id to XCD id % 8 and map_workgroup places n by n % 8: the splits of eight consecutive n follow each other in
// groups of eight, so that n % 8 == id % 8 and the order (longest key blocks first) is kept.
__device__ __forceinline__ void split_of_workgroup(int id, int nsplit, int npair, int* n, int* split) {
  if ((npair & 7) == 0) {
    const int r = id % (8 * nsplit);
    *split = r >> 3;
    *n = (id / (8 * nsplit)) * 8 + (r & 7);
  } else {
    *split = id % nsplit;
    *n = id / nsplit;
  }
}

// dk / dv = sum of the partials, split 0 first (a fixed order), converted to the tensors' element type.
template <typename T>
__global__ __launch_bounds__(256) void backward_dkv_sum_kernel(BwdArgs a, long long nvec) {
  typedef T vec4t __attribute__((ext_vector_type(4)));
  const KArgs& f = a.f;
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;  // one group of four elements of dk and of dv
  if (i >= nvec) return;
  const int dvec = f.D / 4;
  const int d = 4 * (int)(i % dvec);
  long long row = i / dvec;
  const int key = (int)(row % f.S);
  row /= f.S;
  const int hk = (int)(row % f.Hkv), b = (int)(row / f.Hkv);
  const long long plane = (long long)f.B * f.Hkv * f.S * f.D;
  const float* p = a.partial + 4 * i;
  f32x4 x = *(const f32x4*)p, y = *(const f32x4*)(p + plane);
  for (int s = 1; s < a.dkv_splits; s++) {
    x += *(const f32x4*)(p + 2 * s * plane);
    y += *(const f32x4*)(p + (2 * s + 1) * plane);
  }
  *(vec4t*)((T*)a.dk + b * a.dks[0] + hk * a.dks[1] + key * a.dks[2] + d) = __builtin_convertvector(x, vec4t);
  *(vec4t*)((T*)a.dv + b * a.dvs[0] + hk * a.dvs[1] + key * a.dvs[2] + d) = __builtin_convertvector(y, vec4t);
}
template <typename T>
int launch_backward_dkv_sum(const BwdArgs& a, hipStream_t stream) {
  const long long nvec = (long long)a.f.B * a.f.Hkv * a.f.S * (a.f.D / 4);
  hipLaunchKernelGGL(backward_dkv_sum_kernel<T>, dim3((unsigned)((nvec + 255) / 256)), dim3(256), 0, stream, a, nvec);
  return (int)hipGetLastError();
}
// A lane's share of a query row's unnormalised dq sums (accumulator layout of the 32 x 32 matrix instructions: registers 4rg .. 4rg+3 of block db are
// elements 32db + 8rg + 4lh .. +3) and the row's (maximum in log2
// units, sum of exponentials) as this split's partial record; split 0 also leaves delta for the dk/dv kernel.
template <int D>
__device__ __forceinline__ void store_dq_partial(const BwdArgs& a, int piece, long long row_id, int lh, const f32x16 (&dqacc)[D / 32],
                                                 float mc, float l_tot, float delta) {
  const long long rows = (long long)a.f.B * a.f.Hq * a.f.L;
  float* dst = a.dq_partial + (piece * rows + row_id) * D;
#pragma unroll
  for (int db = 0; db < D / 32; db++)
#pragma unroll
    for (int rg = 0; rg < 4; rg++) {
      f32x4 x;
#pragma unroll
      for (int i = 0; i < 4; i++) x[i] = dqacc[db][4 * rg + i];
      *(f32x4*)(dst + 32 * db + 8 * rg + 4 * lh) = x;
    }
  if (lh == 0) {
    float* ml = a.dq_partial + a.dq_splits * rows * D;
    *(float2*)(ml + 2 * (piece * rows + row_id)) = make_float2(mc, l_tot);
    if (piece == 0) a.stats[2 * row_id + 1] = delta;
  }
}

// dq of a call whose key ranges were split: the splits' sums brought to the common maximum, added in a fixed order (split
// 0 first) and normalised; the row statistic for the dk/dv kernel.  One thread per four elements of a row.
template <typename T>
__global__ __launch_bounds__(256) void backward_dq_merge_kernel(BwdArgs a, long long nvec) {
  typedef T vec4t __attribute__((ext_vector_type(4)));
  const KArgs& f = a.f;
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= nvec) return;
  const int dvec = f.D / 4;
  const int d = 4 * (int)(i % dvec);
  const long long row_id = i / dvec;  // (b * Hq + h) * L + qi
  const int qi = (int)(row_id % f.L);
  const long long bh = row_id / f.L;
  const int h = (int)(bh % f.Hq), b = (int)(bh / f.Hq);
  const long long rows = (long long)f.B * f.Hq * f.L;
  const float* ml = a.dq_partial + (long long)a.dq_splits * rows * f.D;
  vec4t* out = (vec4t*)((T*)a.dq + b * a.dqs[0] + h * a.dqs[1] + qi * a.dqs[2] + d);
  f32x4 x = {0.f, 0.f, 0.f, 0.f};
  int S = f.S;
  if (f.kv_len) {
    const int len = f.kv_len[b];
    S = len < 0 ? 0 : (len < S ? len : S);
  }
  if (S == 0) {  // no keys: the dq kernel's workgroups returned at once
    *out = __builtin_convertvector(x, vec4t);
    return;
  }
  float m = -INFINITY;
  for (int s = 0; s < a.dq_splits; s++) m = fmaxf(m, ml[2 * (s * rows + row_id)]);
  float l = 0.f;
  for (int s = 0; s < a.dq_splits; s++) {
    const float2 st = *(const float2*)(ml + 2 * (s * rows + row_id));
    const float w = fast_exp2(st.x - m);
    l += st.y * w;
    x += *(const f32x4*)(a.dq_partial + (s * rows + row_id) * f.D + d) * w;
  }
  // a row whose keys are all hidden: dq = 0, and a statistic that gives it weight 0 in the dk/dv kernel
  const bool seen = l > 0.f;
  const float w = seen ? f.scale / l : 0.f;
#pragma unroll
  for (int e = 0; e < 4; e++) x[e] = seen ? x[e] * w : 0.f;
  *out = __builtin_convertvector(x, vec4t);
  if (d == 0) a.stats[2 * row_id] = seen ? m + __log2f(l) : 1e30f;
}
template <typename T>
int launch_backward_dq_merge(const BwdArgs& a, hipStream_t stream) {
  const long long nvec = (long long)a.f.B * a.f.Hq * a.f.L * (a.f.D / 4);
  hipLaunchKernelGGL(backward_dq_merge_kernel<T>, dim3((unsigned)((nvec + 255) / 256)), dim3(256), 0, stream, a, nvec);
  return (int)hipGetLastError();
}
int launch_backward_general(const BwdArgs& a, int dtype, hipStream_t stream);
int launch_backward_mfma(const BwdArgs& a, int dtype, hipStream_t stream);  // fp16/bf16, head_dim 64 or 128
int launch_backward_f32(const BwdArgs& a, hipStream_t stream);              // fp32 on the fp32 matrix cores, head_dim 64 or 128

// Workgroup n -> (pair, block) for npair (batch, head) pairs of nblk blocks each, block 0 the longest under a causal
// mask.  Workgroups are handed to the 8 XCDs round-robin (n % 8) and start in order: every XCD gets whole pairs (a
// contiguous range, so the heads of a group share its L2) and takes their blocks longest first across all its pairs,
// which keeps the XCDs evenly loaded and the short blocks for the end.  Without a multiple of 8 pairs: longest first
// over all pairs.
__device__ __forceinline__ void map_workgroup(int n, int npair, int nblk, int* pair, int* blk) {
  if ((npair & 7) == 0) {
    const int xcd = n & 7, slot = n >> 3, ppx = npair >> 3;
    *blk = slot / ppx;
    *pair = xcd * ppx + slot % ppx;
  } else {
    *blk = n / npair;
    *pair = n % npair;
  }
}

// head_dim 128 needs more than 256 registers per lane: one wavefront per SIMD, the gradient accumulators in the
// accumulation registers.  Pinning them there at the end of every iteration keeps the loop-carried values in that
// register class, so the matrix instructions accumulate in place instead of being fed through copies (128 moves each
// way per tile otherwise).
template <bool PIN>
__device__ __forceinline__ void pin_accumulator(f32x16& acc) {
  if constexpr (PIN) asm volatile("" : "+a"(acc));
}

// Direction in which a dk/dv workgroup walks the query tiles it0 .. ntq-1 that see its key block.  The workgroups of an XCD
// start longest first (map_workgroup), `dkv_round` of them at a time.  Those of the first round start together at the last
// tile and walk down in step (the tile one fetches is in the XCD's L2 for the others); the workgroup of key block kb ends
// after ntq - it0(kb) tiles, and the CU it frees takes the longest block left, which has as many tiles as the first had
// few.  Walking UP from its first tile, that workgroup is at the same tile at the same time as every other one of the
// second round (all arrive at the last tile together); walking down, each would be alone with its position and fetch
// its tiles from memory itself.  The third round starts together again: rounds alternate.  (bf16 head_dim 128, B2 32q/8kv
// 4096 x 4096: 458 -> 240 MB read per launch of the dk/dv kernel.)
__device__ __forceinline__ bool dkv_walks_up(const BwdArgs& a, bool causal) {
  return causal && a.dkv_round > 0 && ((a.f.B * a.f.Hkv) & 7) == 0 && (((int)(blockIdx.x >> 3) / a.dkv_round) & 1) != 0;
}

// Workgroups of `kernel` that fit one CU, times the CUs of an XCD: the dkv_round of a launch (looked up once per device).
inline int dkv_round_of(const void* kernel, int threads, int lds_bytes, int (&cache)[kMaxDevices]) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 0;
  if (cache[dev] == 0) {
    int n = 0;
    cache[dev] = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, threads, (size_t)lds_bytes) == hipSuccess && n > 0 ? n * kCusPerXcd : -1;
  }
  return cache[dev] > 0 ? cache[dev] : 0;
}

// A Bool attnMask the pipelined prefill kernels' streams can apply: four keys per aligned dword, row offsets of a
// (batch, head) within 32 bits, no causal flag, per-batch key counts, pages or key splits beside it.
inline bool bool_mask_streams_ok(const KArgs& a) {
  return !a.causal && a.mask_kind == 1 && a.mask_vec4 && (a.S % 4) == 0 && !a.kv_len && !a.block_table && a.kv_splits <= 1 &&
         (long long)(a.L - 1) * a.ms[2] + 8 < (1ll << 32);
}

// Keys of batch entry b: all S of them, or the filled prefix of a cache / the unpadded length (kv_len).
__device__ __forceinline__ int keys_of_batch(const KArgs& f, int b) {
  int S = f.S;
  if (f.kv_len) {
    const int len = __builtin_amdgcn_readfirstlane(f.kv_len[b]);
    S = len < 0 ? 0 : (len < S ? len : S);
  }
  return S;
}

// Host-side launchers (one per kernel family); each returns a hipError_t as int.
int launch_general(const KArgs& a, int dtype, hipStream_t stream);
int launch_prefill(const KArgs& a, int dtype, hipStream_t stream);       // 128-row workgroups; head_dim 64 or 128
int launch_prefill_d128(const KArgs& a, int dtype, hipStream_t stream);  // 256-row workgroups, pipelined; head_dim 128
int launch_prefill_d64(const KArgs& a, int dtype, hipStream_t stream);   // the same at head_dim 64 (no attnMask, no pages)
int launch_prefill_f32(const KArgs& a, hipStream_t stream);              // fp32 tensors on the fp32 matrix cores; head_dim 64 or 128
int launch_decode(const KArgs& a, int dtype, void* workspace, hipStream_t stream);
// combines per-split records [pair][split][row][D + 2] (pair = batch * Hkv + kv head, row = l * G + g) into a.out
int launch_merge(const KArgs& a, int dtype, int splits, const float* ws, hipStream_t stream);

// The records of a split launch of a pipelined prefill kernel -> out.  One thread per four elements of a row (eight rows per workgroup): the row's
// splits up to its last visible key (a split wholly beyond the keys of a row tile wrote nothing), brought to their
// common maximum, added in split order, normalised.  Rows of a batch entry without keys: zeros.
template <typename T, int D>
__global__ __launch_bounds__(256) void prefill_split_merge_kernel(KArgs a, long long nvec) {
  typedef T vec4t __attribute__((ext_vector_type(4)));
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= nvec) return;
  const int d = 4 * (int)(i % (D / 4));
  const long long row_id = i / (D / 4);  // (b * Hq + h) * L + qi
  const int qi = (int)(row_id % a.L);
  const long long bh = row_id / a.L;
  const int h = (int)(bh % a.Hq), b = (int)(bh / a.Hq);
  int S = a.S;
  if (a.kv_len) {
    const int len = a.kv_len[b];
    S = len < 0 ? 0 : (len < S ? len : S);
  }
  int last = S - 1;
  if (a.causal) {
    const int v = qi + causal_offset(a, S);
    last = v < last ? v : last;
  }
  int n = last < 0 ? 0 : last / a.kv_chunk + 1;
  n = n < a.kv_splits ? n : a.kv_splits;
  const float c = a.scale * kLog2e;
  const long long step = (long long)a.L * (D + 2);
  const float* rec = a.ws + (bh * a.kv_splits * a.L + qi) * (D + 2);
  float m = -1e30f;
  for (int s = 0; s < n; s++) m = fmaxf(m, rec[s * step + D]);
  float l = 0.f;
  f32x4 x = {0.f, 0.f, 0.f, 0.f};
  for (int s = 0; s < n; s++) {
    const float w = fast_exp2((rec[s * step + D] - m) * c);
    l = fmaf(w, rec[s * step + D + 1], l);
    const float2 lo = *(const float2*)(rec + s * step + d), hi = *(const float2*)(rec + s * step + d + 2);
    x[0] = fmaf(w, lo.x, x[0]), x[1] = fmaf(w, lo.y, x[1]), x[2] = fmaf(w, hi.x, x[2]), x[3] = fmaf(w, hi.y, x[3]);
  }
  const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
  for (int e = 0; e < 4; e++) x[e] *= inv;
  *(vec4t*)((T*)a.out + b * a.os[0] + h * a.os[1] + qi * a.os[2] + d) = __builtin_convertvector(x, vec4t);
}

template <int D>
int launch_prefill_split_merge(const KArgs& a, int dtype, hipStream_t stream) {
  const long long nvec = (long long)a.B * a.Hq * a.L * (D / 4);
  const dim3 grid((unsigned)((nvec + 255) / 256));
  if (dtype == 1) hipLaunchKernelGGL((prefill_split_merge_kernel<_Float16, D>), grid, dim3(256), 0, stream, a, nvec);
  else hipLaunchKernelGGL((prefill_split_merge_kernel<__bf16, D>), grid, dim3(256), 0, stream, a, nvec);
  return (int)hipGetLastError();
}


int launch_zero(const KArgs& a, int dtype, hipStream_t stream);
struct KvAppendArgs {
  void* kc;
  void* vc;
  const void* kn;
  const void* vn;
  const int* positions;
  const int* block_table;  // paged caches, as in KArgs
  int page_shift, bt_stride;
  int B, Hkv, Smax, Lnew, D, position, esz;
  long long kcs[3], vcs[3], kns[3], vns[3];
};
int launch_kv_append(const KvAppendArgs& a, hipStream_t stream);

// Decode tiling, shared by the workspace-size query and the launcher.
struct DecodePlan {
  int splits;      // KV splits per (batch, kv head)
  int chunk;       // keys per split (multiple of the per-wave key block)
  int rows;        // query rows handled together per KV head: L * G
  size_t ws_bytes; // workspace: per (batch, kv head, split): rows * (D + 2) floats
};
DecodePlan plan_decode(const KArgs& a);

constexpr int kDecodeMaxRows = 16;  // L * (Hq/Hkv) handled by one MFMA row block

}  // namespace ttsdpa
