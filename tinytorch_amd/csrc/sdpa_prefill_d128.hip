// Flash-attention forward for fp16 / bf16, head_dim 128, on gfx950 matrix cores: the prefill / training-shape path.
//
// Replaces, in one kernel, the reference's device chain transpose -> batched GEMM -> scale -> causal bias ->
// softmax -> batched GEMM (reference src/Function/FuncNNLayer.h:237-265; device ops at
// src/Operation/OpLinalgCuda.cuh:239-293 and src/Operation/OpNNLayerCuda.cuh:36-145): the [L,S] score matrix
// never leaves registers.
//
// Work split.  A workgroup of 8 wavefronts owns 256 query rows of one (batch, query head), 32 rows per wavefront,
// two wavefronts per SIMD.  Keys/values are consumed in tiles of 64 rows shared by the 8 wavefronts.
//
// LDS.  Four K stages and four V stages of 16 KiB, filled by direct global->LDS loads (global_load_lds_dwordx4: no
// staging registers, no ds_write).  Such a load deposits the 64 lanes' 16-byte pieces contiguously, so rows cannot
// be padded; instead the 16-byte chunk c of tile row r is stored at chunk slot c ^ f(r), f(r) = (r%4)*4 + (r/4)%4,
// which makes both access patterns below bank-conflict free.  The swizzle is applied on the global side (a lane
// fetches the chunk that belongs in its slot).
//
// Per wavefront and half tile of 32 keys, with v_mfma_f32_32x32x16 (A: 32 rows x 16, B: 16 x 32 cols, lane l supplies
// row/col l%32 and the 8 contraction elements of half l/32; C: lane l holds column l%32 and rows
// 8*(r/4) + 4*(l/32) + r%4):
//   S^T[32 keys x 32 queries] = K_half . Q^T      A = K rows (ds_read_b128), B = Q rows held in registers
//   P^T = exp2((S^T - m) * scale*log2e)           a query is one lane column: its keys sit in that lane's registers
//                                                 and in lane l^32, so a row reduction is one cross-lane step
//   O^T[128 x 32 queries] += V_half^T . P^T       A = V^T, read from the row-major V tile with the LDS transpose
//                                                 load ds_read_b64_tr_b16; B = P^T straight from the S^T
//                                                 accumulator registers (same permutation of the contraction
//                                                 index on both sides)
// Software pipeline: the S^T MFMAs of half h+1 are issued in the same straight-line block as the exponentials of
// half h, and the row maximum of half h+1 is taken while the P.V MFMAs of half h run, so the matrix pipe works under
// the vector work.  K and V tiles are requested three tiles before use (four stages each); one barrier per 64-key
// tile.
// The running maximum m is raised only when a half's maximum exceeds it by more than 2^8 in the exponent (the
// probabilities stay <= 256), so the accumulator rescale is rare.
// Causal masking (key j visible to query i iff j <= i, reference src/Operation/OpTransformCpu.h:202-209) skips
// halves above the diagonal and applies the predicate only on halves that straddle it.
// Grouped-query attention: kv head = query head / (Hq/Hkv), resolved in the kernel; the workgroup order puts the
// query heads and row tiles that share a KV head on the same XCD so its L2 holds that K/V once.

#include "sdpa_common.h"

namespace ttsdpa {

namespace {

constexpr int D = 128;
constexpr int NW = 8;    // wavefronts per workgroup
constexpr int WM = 32;   // query rows per wavefront
constexpr int BM = NW * WM;  // query rows per workgroup
constexpr int BN = 64;   // keys per tile
constexpr int ROW_BYTES = D * 2;
constexpr int STAGE_BYTES = BN * ROW_BYTES;  // 16 KiB
constexpr int KSTAGES = 4, VSTAGES = 4;     // K and V tiles are requested three tiles before use
constexpr int LDS_BYTES = (KSTAGES + VSTAGES) * STAGE_BYTES;
constexpr float kLazyExp = 8.f;

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
typedef __attribute__((address_space(3))) void lds_void;
typedef __attribute__((address_space(1))) const void gbl_void;

__device__ __forceinline__ int swz(int row) { return ((row & 3) << 2) | ((row >> 2) & 3); }

template <typename TR, bool CAUSAL>
__global__ __launch_bounds__(NW * 64, 2) void prefill128_kernel(KArgs a) {
  typedef typename TR::elem T;
  typedef typename TR::vec8 vec8;

  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lq = lane & 31;
  const int lh = lane >> 5;

  // ---- workgroup -> (batch, kv head, query head in group, row tile) -------------------------------------------
  // Under a causal mask a workgroup takes row tile t and then its mirror ntile-1-t: every workgroup sees the same
  // number of KV tiles, so the launch has no long tail behind the heavy tiles.
  const int ntile = (a.L + BM - 1) / BM;
  const int nslot = CAUSAL ? (ntile + 1) / 2 : ntile;
  const int inner = a.G * nslot;
  const int npair = a.B * a.Hkv;
  int pair, in;
  {
    int n = blockIdx.x;
    if ((npair & 7) == 0) {  // workgroup n runs on XCD n % 8: keep a (batch, kv head) on one XCD
      int xcd = n & 7, slot = n >> 3;
      pair = (slot / inner) * 8 + xcd;
      in = slot % inner;
    } else {
      pair = n / inner;
      in = n % inner;
    }
  }
  const int b = pair / a.Hkv, hk = pair % a.Hkv;
  const int g = in % a.G;
  const int slot_rt = in / a.G;
  const int h = hk * a.G + g;

  const T* qp = (const T*)a.q + b * a.qs[0] + h * a.qs[1];
  const T* kp = (const T*)a.k + b * a.ks[0] + hk * a.ks[1];
  const T* vp = (const T*)a.v + b * a.vs[0] + hk * a.vs[1];

  for (int part = 0; part < (CAUSAL ? 2 : 1); part++) {
  const int rt = (CAUSAL && part == 0) ? ntile - 1 - slot_rt : slot_rt;  // the long tile first
  if (part == 1 && slot_rt >= ntile - 1 - slot_rt) break;                  // odd count: the middle tile has no mirror
  const int q0 = rt * BM;
  const int qw0 = q0 + wave * WM;

  int ntiles_kv = (a.S + BN - 1) / BN;
  if (CAUSAL) {
    int last = q0 + BM - 1 < a.L - 1 ? q0 + BM - 1 : a.L - 1;
    int lastkv = last < a.S - 1 ? last : a.S - 1;
    ntiles_kv = lastkv / BN + 1;
  }
  // 32-key halves this wavefront computes on: under a causal mask those that start at or before its last row
  int my_halves = 2 * ntiles_kv;
  // tiles whose both halves need no mask for this wavefront and whose successor half exists: the fast path
  int nfast = a.S / BN;
  if (CAUSAL) {
    int t = (qw0 + WM - 1) / 32 + 1;
    my_halves = t < my_halves ? t : my_halves;
    int f = (qw0 + 1) / BN;  // tiles with 64j + 63 <= qw0
    nfast = f < nfast ? f : nfast;
  }
  if (nfast > ntiles_kv - 1) nfast = ntiles_kv - 1;
  if (2 * nfast > my_halves - 2) nfast = (my_halves - 2) / 2;  // half 2j+2 must be one of ours
  if (nfast < 0) nfast = 0;

  // ---- global -> LDS: wavefront w moves rows 8w .. 8w+7 of a tile, 4 rows (1 KiB) per instruction --------------
  // lane l fills slot (row 4i + l/16, chunk slot l%16) and therefore fetches chunk (l%16) ^ f(row)
  unsigned ld_koff[2], ld_voff[2];
#pragma unroll
  for (int i = 0; i < 2; i++) {
    int row = 8 * wave + 4 * i + (lane >> 4);
    int chunk = (lane & 15) ^ swz(row);
    ld_koff[i] = (unsigned)(row * a.ks[2] + 8 * chunk) * 2u;
    ld_voff[i] = (unsigned)(row * a.vs[2] + 8 * chunk) * 2u;
  }
  auto dma_tile = [&](const T* base, long long rstride, const unsigned (&off)[2], int kv0, char* stage) __attribute__((always_inline)) {
    const char* src = (const char*)(base + kv0 * rstride);
    if (kv0 + BN <= a.S) {
#pragma unroll
      for (int i = 0; i < 2; i++)
        __builtin_amdgcn_global_load_lds((gbl_void*)(src + off[i]), (lds_void*)(stage + (8 * wave + 4 * i) * ROW_BYTES),
                                         16, 0, 0);
    } else {  // ragged last tile: rows past the end re-read the last valid row (their scores are masked)
#pragma unroll
      for (int i = 0; i < 2; i++) {
        int row = 8 * wave + 4 * i + (lane >> 4);
        int key = kv0 + row;
        key = key < a.S ? key : a.S - 1;
        int chunk = (lane & 15) ^ swz(row);
        __builtin_amdgcn_global_load_lds((gbl_void*)(base + key * rstride + 8 * chunk),
                                         (lds_void*)(stage + (8 * wave + 4 * i) * ROW_BYTES), 16, 0, 0);
      }
    }
  };
  auto dma_k = [&](int tile, int stage) __attribute__((always_inline)) { dma_tile(kp, a.ks[2], ld_koff, tile * BN, smem + stage * STAGE_BYTES); };
  auto dma_v = [&](int tile, int stage) __attribute__((always_inline)) { dma_tile(vp, a.vs[2], ld_voff, tile * BN, smem + (KSTAGES + stage) * STAGE_BYTES); };
  // Wait until at most `keep` of this wavefront's global->LDS loads are still in flight (they complete in issue
  // order), then meet the other wavefronts: what was issued before the newest `keep` loads is visible to all.
  auto dma_wait_and_sync = [&](int keep) __attribute__((always_inline)) {
    if (keep >= 4) {
      asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
    } else if (keep >= 2) {
      asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
    } else {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    __syncthreads();
  };

  // ---- LDS operand addresses (bytes), loop-invariant ---------------------------------------------------------------
  // K operand (half, ks): row 32*half + lq, chunk 2*ks + lh  ->  row*256 + 16*((2ks + lh) ^ f(row))
  unsigned k_addr[8];
  {
    unsigned base = (unsigned)(lq * ROW_BYTES + 16 * (lh ^ swz(lq)));  // f(32*half + lq) == f(lq)
#pragma unroll
    for (int ks = 0; ks < 8; ks++) k_addr[ks] = base ^ (unsigned)(32 * ks);
  }
  // V operand part (db, ld) of k-step t via the transpose load: this lane points at row 16t + 8ld + 4lh + s/4,
  // elements 32db + 16*dhalf + 4*(s%4) .. +3 (s = lane%16, dhalf = (lane/16)%2) and receives
  // V[16t + 8ld + 4lh + 0..3][32db + lq]
  unsigned v_addr[4][2];
  {
    const int s = lane & 15, dhalf = (lane >> 4) & 1;
#pragma unroll
    for (int ld = 0; ld < 2; ld++) {
      int row = 8 * ld + 4 * lh + (s >> 2);  // + 16t later: f(row) does not depend on t
#pragma unroll
      for (int db = 0; db < 4; db++) {
        int chunk = 4 * db + 2 * dhalf + ((s & 3) >> 1);
        // the V region's base is folded in here so that stage and k-step offsets fit the 16-bit ds_read immediate
        v_addr[db][ld] = (unsigned)(KSTAGES * STAGE_BYTES + row * ROW_BYTES + 16 * (chunk ^ swz(row)) + 8 * (s & 1));
      }
    }
  }

  // ---- prologue: first tiles on their way, Q into registers ---------------------------------------------------------
  dma_k(0, 0);
  dma_v(0, 0);
  if (ntiles_kv > 1) dma_k(1, 1);
  if (ntiles_kv > 1) dma_v(1, 1);
  if (ntiles_kv > 2) dma_k(2, 2);
  if (ntiles_kv > 2) dma_v(2, 2);

  vec8 qreg[8];
  {
    int row = qw0 + lq;
    row = row < a.L ? row : a.L - 1;
    const T* qr = qp + row * a.qs[2] + 8 * lh;
#pragma unroll
    for (int ks = 0; ks < 8; ks++) qreg[ks] = *(const vec8*)(qr + 16 * ks);
  }

  f32x16 oacc[4];
#pragma unroll
  for (int db = 0; db < 4; db++)
#pragma unroll
    for (int r = 0; r < 16; r++) oacc[db][r] = 0.f;
  const float c = a.scale * kLog2e;
  const float lazy = kLazyExp / c;
  float m_use = -1e30f;  // maximum the exponentials are taken against (raw scores)
  float mc = -1e30f * c;
  float l_run = 0.f;

  // S^T of one half tile (32 keys); kh = LDS address of the half's first K row
  auto qk_half = [&](f32x16& s, const char* kh) __attribute__((always_inline)) {
#pragma unroll
    for (int r = 0; r < 16; r++) s[r] = 0.f;
#pragma unroll
    for (int ks = 0; ks < 8; ks++) {
      vec8 ka = *(const vec8*)(kh + k_addr[ks]);
      s = TR::mfma32(ka, qreg[ks], s);
    }
  };

  auto mask_half = [&](f32x16& s, int kv0) __attribute__((always_inline)) {
    const int qi = qw0 + lq;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      int key = kv0 + 8 * (r >> 2) + 4 * lh + (r & 3);
      bool hidden = key >= a.S || (CAUSAL && key > qi);
      if (hidden) s[r] = -INFINITY;
    }
  };

  auto row_max = [&](const f32x16& s) __attribute__((always_inline)) {
    float m = s[0];
#pragma unroll
    for (int r = 1; r < 16; r++) m = fmaxf(m, s[r]);
    // The other 16 keys of this query sit in lane l^32.  v_permlane32_swap exchanges the upper 32 lanes of its
    // first operand with the lower 32 lanes of its second, so two copies of m become (lower half, lower half) and
    // (upper half, upper half).  Written as asm: the compiler folds the two results of the builtin into one.
    unsigned lo = __builtin_bit_cast(unsigned, m), hi = lo;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(lo), "+v"(hi));
    return fmaxf(__builtin_bit_cast(float, lo), __builtin_bit_cast(float, hi));
  };

  // raise the running maximum when some row needs it (rare), rescaling sum and accumulator
  auto raise_max = [&](float mx) __attribute__((always_inline)) {
    if (__builtin_amdgcn_ballot_w64(mx > m_use + lazy) != 0) {
      const float m_new = fmaxf(m_use, mx);
      const float alpha = fast_exp2((m_use - m_new) * c);
      m_use = m_new;
      mc = m_new * c;
      l_run *= alpha;
#pragma unroll
      for (int db = 0; db < 4; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) oacc[db][r] *= alpha;
    }
  };

  // exponentials of one half -> P^T as MFMA B operands pb[k-step of 16 keys]
  auto exp_half = [&](f32x16& s, vec8 (&pb)[2]) __attribute__((always_inline)) {
    float psum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      float p = fast_exp2(fmaf(s[r], c, -mc));
      s[r] = p;
      psum += p;
    }
    l_run += psum;
#pragma unroll
    for (int t = 0; t < 2; t++) {
      f32x8 x;
#pragma unroll
      for (int i = 0; i < 8; i++) x[i] = s[8 * t + i];
      pb[t] = __builtin_convertvector(x, vec8);
    }
  };

  // O^T += V_half^T . P^T; vh = LDS address of the half's first V row
  auto pv_half = [&](const vec8 (&pb)[2], const char* vh) __attribute__((always_inline)) {
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
      for (int db = 0; db < 4; db++) {
        s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(vh + v_addr[db][0] + 16 * t * ROW_BYTES));
        s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(vh + v_addr[db][1] + 16 * t * ROW_BYTES));
        vec8 va = __builtin_bit_cast(vec8, (s16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
        oacc[db] = TR::mfma32(va, pb[t], oacc[db]);
      }
  };

  // Pipeline step, fast form: half hb needs no mask and half hb+1 is wanted.
  auto fast_step = [&](f32x16& cur, float& mcur, f32x16& nxt, float& mnxt, const char* kn, const char* vc) __attribute__((always_inline)) {
    raise_max(mcur);
    vec8 pb[2];
    qk_half(nxt, kn);
    exp_half(cur, pb);
    pv_half(pb, vc);
    mnxt = row_max(nxt);
  };
  // General form: half hb may be unwanted / masked, half hb+1 may be unwanted.
  auto slow_step = [&](f32x16& cur, float& mcur, f32x16& nxt, float& mnxt, int hb, const char* kn, const char* vc,
                       bool do_nxt) __attribute__((always_inline)) {
    const int kv0 = 32 * hb;
    if (do_nxt) qk_half(nxt, kn);
    if (hb < my_halves) {
      if ((CAUSAL && kv0 + 31 > qw0) || kv0 + 32 > a.S) {  // the half straddles the diagonal or the end of the keys
        mask_half(cur, kv0);
        mcur = row_max(cur);
      }
      raise_max(mcur);
      vec8 pb[2];
      exp_half(cur, pb);
      pv_half(pb, vc);
    }
    if (do_nxt) mnxt = row_max(nxt);
  };

  f32x16 sP, sN;
  float mP, mN = 0.f;
  dma_wait_and_sync(0);
  qk_half(sP, smem);
  mP = row_max(sP);
  // Tile t lives in stage t % 4 (K and V alike).  Iteration j reads K(j) (second half), K(j+1) (first half) and
  // V(j), and sends for K(j+3) and V(j+3), whose stage was last read in iteration j-1.  Its closing barrier publishes
  // tile j+2, requested one iteration earlier: only this iteration's own loads may still be in flight.
  // The stage index is a compile-time constant in the unrolled fast loop, so every LDS address there is
  // lane address + immediate.
  auto tile_iter = [&](int j, const int st, const bool fast) __attribute__((always_inline)) {
    int keep = 0;
    if (j + 3 < ntiles_kv) {
      dma_k(j + 3, (st + 3) & 3);
      dma_v(j + 3, (st + 3) & 3);
      keep = 4;
    }
    const char* kc1 = smem + st * STAGE_BYTES + 32 * ROW_BYTES;
    const char* kn0 = smem + ((st + 1) & 3) * STAGE_BYTES;
    const char* vc = smem + st * STAGE_BYTES;  // v_addr carries the V region's base
    if (fast) {
      fast_step(sP, mP, sN, mN, kc1, vc);
      fast_step(sN, mN, sP, mP, kn0, vc + 32 * ROW_BYTES);
    } else {
      slow_step(sP, mP, sN, mN, 2 * j, kc1, vc, 2 * j + 1 < my_halves);
      slow_step(sN, mN, sP, mP, 2 * j + 1, kn0, vc + 32 * ROW_BYTES, j + 1 < ntiles_kv && 2 * j + 2 < my_halves);
    }
    dma_wait_and_sync(keep);
  };
  int j = 0;
  for (; j + 4 <= nfast; j += 4) {  // tiles that need no mask and whose successor half is wanted
    tile_iter(j, 0, true);
    tile_iter(j + 1, 1, true);
    tile_iter(j + 2, 2, true);
    tile_iter(j + 3, 3, true);
  }
  for (; j < ntiles_kv; j++)  // the rest: diagonal tiles, the ragged end of the keys, tiles this wavefront skips
    tile_iter(j, j & 3, false);

  // ---- normalise and store ----------------------------------------------------------------------------------------------
  {
    float l_tot = l_run + __shfl_xor(l_run, 32);
    const float inv = 1.f / l_tot;
    const int qi = qw0 + lq;
    if (qi < a.L) {
      T* op = (T*)a.out + b * a.os[0] + h * a.os[1] + qi * a.os[2];
#pragma unroll
      for (int db = 0; db < 4; db++)
#pragma unroll
        for (int rg = 0; rg < 4; rg++) {
          f32x4 x;
#pragma unroll
          for (int i = 0; i < 4; i++) x[i] = oacc[db][4 * rg + i] * inv;
          typename TR::vec4 y = __builtin_convertvector(x, typename TR::vec4);
          *(typename TR::vec4*)(op + 32 * db + 8 * rg + 4 * lh) = y;
        }
    }
  }
  }  // part
}

template <typename TR, bool CAUSAL>
int launch_k(const KArgs& a, dim3 grid, hipStream_t stream) {
  static const hipError_t granted = hipFuncSetAttribute((const void*)prefill128_kernel<TR, CAUSAL>,
                                                        hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
  if (granted != hipSuccess) return (int)granted;
  hipLaunchKernelGGL((prefill128_kernel<TR, CAUSAL>), grid, dim3(NW * 64), LDS_BYTES, stream, a);
  return (int)hipGetLastError();
}

}  // namespace

int launch_prefill_d128(const KArgs& a, int dtype, hipStream_t stream) {
  const int ntile = (a.L + BM - 1) / BM;
  long long nwg = (long long)a.B * a.Hq * (a.causal ? (ntile + 1) / 2 : ntile);
  dim3 grid((unsigned)nwg);
  if (dtype == 1) return a.causal ? launch_k<F16, true>(a, grid, stream) : launch_k<F16, false>(a, grid, stream);
  return a.causal ? launch_k<BF16, true>(a, grid, stream) : launch_k<BF16, false>(a, grid, stream);
}

}  // namespace ttsdpa
