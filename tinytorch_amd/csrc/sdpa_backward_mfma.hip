// Attention backward for fp16 / bf16 on gfx950 matrix cores, head_dim 64 or 128, optional causal mask (either
// alignment), grouped heads.  The reference has no attention backward (reference src/Function/FuncNNLayer.h:267 is
// NOT_IMPLEMENTED); this is the chain rule through its forward chain matmul -> scale -> bias -> softmax -> matmul
// (src/Function/FuncNNLayer.h:237-265, softmax step as src/Operation/OpNNLayerCpu.h:79-109) without ever storing an
// [L,S] matrix:
//   P_ij = exp(scale * q_i.k_j - lse_i)    dP_ij = dout_i.v_j    delta_i = dout_i.out_i    dS_ij = P_ij (dP_ij - delta_i)
//   dq_i = scale * sum_j dS_ij k_j         dk_j = scale * sum_i dS_ij q_i                  dv_j = sum_i P_ij dout_i
//
// Two kernels, no atomics (fixed summation order, reproducible results):
//   1. backward_dq_mfma_kernel — a workgroup owns 128 query rows of one (batch, query head), a wavefront 32 of them,
//      and streams the keys in tiles of 64 (32 at head_dim 128) like the forward kernel: S^T = K.Q^T, an online softmax with a lazily
//      raised maximum (so lse_i needs no pass of its own), dP^T = V.dout^T, dS^T, dq^T += K^T.dS^T.  At the end
//      dq = scale/l * accumulator, and (lse_i, delta_i) go to scratch for the second kernel.
//   2. backward_dkv_mfma_kernel (head_dim 64) / backward_dkv128_kernel (head_dim 128) — a workgroup owns 128 keys of
//      one (batch, kv head), a wavefront 32 of them, and streams the query rows of every head of the group in tiles
//      of 32: S = Q.K^T, P from lse, dP = dout.V^T, dS, dv^T += dout^T.P, dk^T += Q^T.dS.
// Both compute 32 x 32 score blocks with v_mfma_f32_32x32x16 whose accumulator layout (lane = column, registers = rows)
// is the B operand of the following product, so P and dS go from registers to the matrix cores without touching LDS;
// the register-staged tiles are kept in LDS twice where both a row-major operand and a transposed one
// (ds_read_b64_tr_b16) are read from them, each copy with the row pitch that makes its reads conflict-free; the
// head_dim-128 dk/dv kernel keeps one swizzled copy instead (see there).
// Seven matrix products in all, against five in the textbook count (the scores are computed in both kernels).
// When a call has too few key blocks to fill and balance the chip, the query stream of a key block is dealt out to 2-4
// workgroups of kernel 2, which leave fp32 partial sums in scratch, and backward_dkv_sum_kernel (sdpa_common.h) adds
// them in a fixed order.  Likewise kernel 1: with fewer than 512 query blocks the key range of a block is dealt out to
// 2-8 workgroups, whose unnormalised fp32 sums and (maximum, sum of exponentials) backward_dq_merge_kernel combines.

#include "sdpa_common.h"

namespace ttsdpa {

namespace {

constexpr int BM = 128;  // rows of the owning side per workgroup (queries in kernel 1, keys in kernel 2)
constexpr int BQ = 32;   // query rows per streamed tile, kernel 2
constexpr float kLazyExp = 8.f;

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));

template <int D>
struct BwdLds {
  static constexpr int RP = D + 8;    // row pitch (elements) of a tile read as a row-major operand (ds_read_b128)
  static constexpr int TP = D + 32;   // row pitch of a tile read as a transposed operand (ds_read_b64_tr_b16)
  static constexpr int KV_STAGE = BQ * (2 * RP + 2 * TP);   // Q and dout, each in both layouts
  static constexpr int KV_STATS = 2 * BQ;                   // floats per stage: (lse, delta) per query row
  static constexpr int KV_BYTES = 2 * KV_STAGE * 2 + 2 * KV_STATS * 4;
};

// Key tile of the dq kernel: keys per tile, elements per LDS stage (K row-major, V row-major, K for transposed reads).
template <int D>
struct DqTile {
  static constexpr int BN = D > 64 ? 32 : 64;
  static constexpr int STAGE = BN * (2 * BwdLds<D>::RP + BwdLds<D>::TP);
  static constexpr int BYTES = 2 * STAGE * 2;
};

// One MFMA A operand of X^T from a row-major tile X with pitch TP: lane l (column d = d0 + l%32, half h = l/32)
// receives the 8 rows base + {4h + 0..3, 8 + 4h + 0..3} — the order in which a 32x32 accumulator's registers 8t..8t+7
// hold rows, so the other operand can be taken straight from such registers.
template <typename vec8>
__device__ __forceinline__ vec8 transposed_operand(const void* lane_base, int byte_off_lo, int byte_off_hi) {
  typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
  s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)((const char*)lane_base + byte_off_lo));
  s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)((const char*)lane_base + byte_off_hi));
  s16x8 r = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(vec8, r);
}

// A lane's share of the dk / dv rows of key `key` (accumulator layout: registers 4rg .. 4rg+3 of block db are elements
// 32db + 8rg + 4lh .. +3) goes to the gradient tensors, or — when the key block's query stream is split over several
// workgroups — as fp32 to this split's partial sums, dense [split][dk | dv][B][Hkv][S][D].
// PAD: the tensors' head_dim a.f.D is a multiple of 8 below D; only its columns are written (no splits then).
template <typename TR, int D, bool PAD = false>
__device__ __forceinline__ void store_key_grads(const BwdArgs& a, int split, int b, int hk, int key, int lh,
                                                const f32x16 (&dkacc)[D / 32], const f32x16 (&dvacc)[D / 32], float scale) {
  typedef typename TR::elem T;
  if (key >= a.f.S) return;
  if (a.dkv_splits > 1) {
    const long long plane = (long long)a.f.B * a.f.Hkv * a.f.S * D;
    float* dkp = a.partial + 2 * split * plane + (((long long)b * a.f.Hkv + hk) * a.f.S + key) * D;
#pragma unroll
    for (int db = 0; db < D / 32; db++)
#pragma unroll
      for (int rg = 0; rg < 4; rg++) {
        f32x4 x, y;
#pragma unroll
        for (int i = 0; i < 4; i++) x[i] = dkacc[db][4 * rg + i] * scale, y[i] = dvacc[db][4 * rg + i];
        *(f32x4*)(dkp + 32 * db + 8 * rg + 4 * lh) = x;
        *(f32x4*)(dkp + plane + 32 * db + 8 * rg + 4 * lh) = y;
      }
    return;
  }
  T* dkp = (T*)a.dk + b * a.dks[0] + hk * a.dks[1] + key * a.dks[2];
  T* dvp = (T*)a.dv + b * a.dvs[0] + hk * a.dvs[1] + key * a.dvs[2];
#pragma unroll
  for (int db = 0; db < D / 32; db++)
#pragma unroll
    for (int rg = 0; rg < 4; rg++) {
      f32x4 x, y;
#pragma unroll
      for (int i = 0; i < 4; i++) x[i] = dkacc[db][4 * rg + i] * scale, y[i] = dvacc[db][4 * rg + i];
      if (PAD && 32 * db + 8 * rg + 4 * lh >= a.f.D) continue;
      *(typename TR::vec4*)(dkp + 32 * db + 8 * rg + 4 * lh) = __builtin_convertvector(x, typename TR::vec4);
      *(typename TR::vec4*)(dvp + 32 * db + 8 * rg + 4 * lh) = __builtin_convertvector(y, typename TR::vec4);
    }
}

// dk and dv rows of a key no query row attends to (at or beyond the batch entry's key count): zeros.
template <typename TR, int D, bool PAD = false>
__device__ __forceinline__ void zero_key_rows(const BwdArgs& a, int split, int b, int hk, int key, int lh) {
  f32x16 zero[D / 32];
#pragma unroll
  for (int i = 0; i < D / 32; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) zero[i][r] = 0.f;
  store_key_grads<TR, D, PAD>(a, split, b, hk, key, lh, zero, zero, 0.f);
}

template <typename vec8>
__device__ __forceinline__ vec8 regs_to_operand(const f32x16& acc, int t) {
  f32x8 x;
#pragma unroll
  for (int i = 0; i < 8; i++) x[i] = acc[8 * t + i];
  return __builtin_convertvector(x, vec8);
}

// ---- kernel 1: dq, lse, delta ----------------------------------------------------------------------------------------
// BN: keys per streamed tile.  64 for head_dim 64; 32 for head_dim 128, which keeps a wavefront under 256 registers:
// two wavefronts per SIMD (one's vector work overlaps the other's matrix work), accumulators in ordinary registers.
// MASKED: an attnMask (exclusive with CAUSAL) whose keys can be read four at a time, as in the forward kernels.
// PAD (both register-staged kernels): the tensors' head_dim f.D is a multiple of 8 below D.  The 16-byte chunks of a row
// beyond it are taken as zeros (q, k: nothing added to a score; dout, v: nothing added to dP or delta; the gradients'
// columns beyond f.D are not stored); everything else is the kernel for head_dim D.  No splits (their records are laid
// out for D).
template <typename TR, int D, bool CAUSAL, bool MASKED, bool PAD>
__global__ __launch_bounds__(256, 2) void backward_dq_mfma_kernel(BwdArgs a) {
  constexpr int BN = DqTile<D>::BN;
  typedef typename TR::elem T;
  typedef typename TR::vec8 vec8;
  typedef BwdLds<D> Lds;
  constexpr int RP = Lds::RP, TP = Lds::TP;
  constexpr int NBLK = BN / 32;            // 32-key blocks per tile
  constexpr int KSTEPS = D / 16, DBLK = D / 32;
  constexpr int NLD = (BN * D / 8) / 256;
  const KArgs& f = a.f;

  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  T* smem = (T*)smem_raw;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lq = lane & 31, lh = lane >> 5;

  const int ntile = (f.L + BM - 1) / BM;
  int pair, in, piece;  // piece: this workgroup's share of the row block's key range (dq_splits > 1)
  {
    int n;
    split_of_workgroup(blockIdx.x, a.dq_splits, f.B * f.Hq, &n, &piece);
    map_workgroup(n, f.B * f.Hq, ntile, &pair, &in);
  }
  const int h = pair % f.Hq, b = pair / f.Hq;
  const int hk = h / f.G;
  const int rt = CAUSAL ? ntile - 1 - in : in;  // longest rows first
  const int q0 = rt * BM, qw0 = q0 + wave * 32;
  const bool wave_live = qw0 < f.L;

  const T* kp = (const T*)f.k + b * f.ks[0] + hk * f.ks[1];
  const T* vp = (const T*)f.v + b * f.vs[0] + hk * f.vs[1];

  // ---- this lane's query row: q and dout as B operands, delta = dout . out ------------------------------------------------
  vec8 qreg[KSTEPS], greg[KSTEPS];
  float delta;
  {
    int row = qw0 + lq;
    row = row < f.L ? row : f.L - 1;
    const T* qr = (const T*)f.q + b * f.qs[0] + h * f.qs[1] + row * f.qs[2] + 8 * lh;
    const T* gr = (const T*)a.dout + b * a.dos[0] + h * a.dos[1] + row * a.dos[2] + 8 * lh;
    const T* orow = (const T*)f.out + b * f.os[0] + h * f.os[1] + row * f.os[2] + 8 * lh;
    float part = 0.f;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) {
      if (PAD && 16 * ks + 8 * lh >= f.D) {
#pragma unroll
        for (int i = 0; i < 8; i++) qreg[ks][i] = (T)0.f, greg[ks][i] = (T)0.f;
        continue;
      }
      qreg[ks] = *(const vec8*)(qr + 16 * ks);
      greg[ks] = *(const vec8*)(gr + 16 * ks);
      const vec8 o = *(const vec8*)(orow + 16 * ks);
#pragma unroll
      for (int i = 0; i < 8; i++) part = fmaf((float)o[i], (float)greg[ks][i], part);
    }
    delta = part + __shfl_xor(part, 32);
  }

  f32x16 dqacc[DBLK];
#pragma unroll
  for (int i = 0; i < DBLK; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) dqacc[i][r] = 0.f;
  const float c = f.scale * kLog2e;
  const float lazy = kLazyExp / c;
  float m_use = -1e30f, mc = m_use * c, l_run = 0.f;

  const int S = keys_of_batch(f, b);
  if (S == 0) {  // no keys (an empty cache entry): the output did not depend on q
    if (a.dq_splits > 1) return;  // the merge kernel writes the zeros
    const int qi = qw0 + lq;
    if (qi < f.L) {
      T* dqp = (T*)a.dq + b * a.dqs[0] + h * a.dqs[1] + qi * a.dqs[2];
      typename TR::vec4 zero;
#pragma unroll
      for (int i = 0; i < 4; i++) zero[i] = (T)0.f;
      for (int d = 4 * lh; d < (PAD ? f.D : D); d += 8) *(typename TR::vec4*)(dqp + d) = zero;
    }
    return;
  }
  const int coff = CAUSAL ? causal_offset(f, S) : 0;
  int ntiles_kv = (S + BN - 1) / BN;
  if (CAUSAL) {
    const int last = (q0 + BM - 1 < f.L - 1 ? q0 + BM - 1 : f.L - 1) + coff;  // last key any row of the workgroup sees
    const int lastkv = last < S - 1 ? last : S - 1;
    ntiles_kv = lastkv / BN + 1;
  }
  // this workgroup's tiles: all of them, or piece `piece` of dq_splits nearly equal ones (possibly none)
  const int t0 = (int)((long long)ntiles_kv * piece / a.dq_splits), t1 = (int)((long long)ntiles_kv * (piece + 1) / a.dq_splits);

  // ---- global -> register -> LDS staging of one K/V tile (thread t moves 16-byte chunks t, t+256, ...) ----------------------
  u32x4 kst[NLD], vst[NLD];
  int lrow[NLD], lcol[NLD], gcol[NLD];
  bool cval[NLD];  // PAD: the chunk lies inside the tensors' rows; the others are loaded from the row's first chunk instead
                   // (the loads stay unconditional) and reach LDS as zeros
#pragma unroll
  for (int i = 0; i < NLD; i++) {
    const int cidx = tid + 256 * i;
    lrow[i] = cidx / (D / 8);
    lcol[i] = cidx % (D / 8);
    cval[i] = !PAD || 8 * lcol[i] < f.D;
    gcol[i] = cval[i] ? lcol[i] : 0;
  }
  const u32x4 zero4 = {0u, 0u, 0u, 0u};
  auto load_tile = [&](int kv0) {
#pragma unroll
    for (int i = 0; i < NLD; i++) {
      int key = kv0 + lrow[i];
      key = key < S ? key : S - 1;  // rows past the end re-read the last valid row (hidden below)
      kst[i] = *(const u32x4*)(kp + key * f.ks[2] + 8 * gcol[i]);
      vst[i] = *(const u32x4*)(vp + key * f.vs[2] + 8 * gcol[i]);
    }
  };
  auto store_tile = [&](int stage) {
    T* Kr = smem + stage * DqTile<D>::STAGE;
    T* Vr = Kr + BN * RP;
    T* Kt = Vr + BN * RP;
#pragma unroll
    for (int i = 0; i < NLD; i++) {
      *(u32x4*)(Kr + lrow[i] * RP + 8 * lcol[i]) = cval[i] ? kst[i] : zero4;
      *(u32x4*)(Kt + lrow[i] * TP + 8 * lcol[i]) = cval[i] ? kst[i] : zero4;
      *(u32x4*)(Vr + lrow[i] * RP + 8 * lcol[i]) = cval[i] ? vst[i] : zero4;
    }
  };
  const int r_lane = lq * RP + 8 * lh;
  const int t_lane = (4 * lh + ((lane & 15) >> 2)) * TP + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

  if (t0 < t1) {
    load_tile(t0 * BN);
    store_tile(0);
    if (t0 + 1 < t1) load_tile((t0 + 1) * BN);
  }
  __syncthreads();

  for (int jt = t0; jt < t1; jt++) {
    const int kv0 = jt * BN;
    const int cur = (jt - t0) & 1;
    if (jt + 1 < t1) {
      store_tile(cur ^ 1);
      if (jt + 2 < t1) load_tile(kv0 + 2 * BN);
    }
    if (wave_live && (!CAUSAL || kv0 <= qw0 + 31 + coff)) {
      const T* Kr = smem + cur * DqTile<D>::STAGE;
      const T* Vr = Kr + BN * RP;
      const T* Kt = Vr + BN * RP;

      f32x16 sacc[NBLK];
#pragma unroll
      for (int blk = 0; blk < NBLK; blk++) {
#pragma unroll
        for (int r = 0; r < 16; r++) sacc[blk][r] = 0.f;
        const T* krow = Kr + r_lane + 32 * blk * RP;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ks++) sacc[blk] = TR::mfma32(*(const vec8*)(krow + 16 * ks), qreg[ks], sacc[blk]);
      }
      if ((CAUSAL && kv0 + BN - 1 > qw0 + coff) || kv0 + BN > S) {
        const int qi = qw0 + lq + coff;
#pragma unroll
        for (int blk = 0; blk < NBLK; blk++)
#pragma unroll
          for (int r = 0; r < 16; r++) {
            const int key = kv0 + 32 * blk + 8 * (r >> 2) + 4 * lh + (r & 3);
            if (key >= S || (CAUSAL && key > qi)) sacc[blk][r] = -INFINITY;
          }
      }
      if (MASKED) {
        int qi = qw0 + lq;
        qi = qi < f.L ? qi : f.L - 1;
        const long long mrow = b * f.ms[0] + h * f.ms[1] + qi * f.ms[2];
#pragma unroll
        for (int blk = 0; blk < NBLK; blk++) apply_attn_mask<T, true>(f, sacc[blk], mrow, kv0 + 32 * blk, lh, S, 1.f / f.scale);
      }
      float mloc = sacc[0][0];
#pragma unroll
      for (int blk = 0; blk < NBLK; blk++)
#pragma unroll
        for (int r = 0; r < 16; r++) mloc = fmaxf(mloc, sacc[blk][r]);
      mloc = fmaxf(mloc, __shfl_xor(mloc, 32));
      if (__builtin_expect(__builtin_amdgcn_ballot_w64(mloc > m_use + lazy) != 0, 0)) {
        const float m_new = fmaxf(m_use, mloc);
        const float alpha = fast_exp2((m_use - m_new) * c);
        m_use = m_new;
        mc = m_new * c;
        l_run *= alpha;
#pragma unroll
        for (int i = 0; i < DBLK; i++)
#pragma unroll
          for (int r = 0; r < 16; r++) dqacc[i][r] *= alpha;
      }
      // dP^T = V . dout^T
      f32x16 dpacc[NBLK];
#pragma unroll
      for (int blk = 0; blk < NBLK; blk++) {
#pragma unroll
        for (int r = 0; r < 16; r++) dpacc[blk][r] = 0.f;
        const T* vrow = Vr + r_lane + 32 * blk * RP;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ks++) dpacc[blk] = TR::mfma32(*(const vec8*)(vrow + 16 * ks), greg[ks], dpacc[blk]);
      }
      float psum = 0.f;
#pragma unroll
      for (int blk = 0; blk < NBLK; blk++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const float p = fast_exp2(fmaf(sacc[blk][r], c, -mc));  // relative to m_use; normalised at the end
          psum += p;
          sacc[blk][r] = p * (dpacc[blk][r] - delta);
        }
      l_run += psum;
      vec8 dsb[2 * NBLK];
#pragma unroll
      for (int t = 0; t < 2 * NBLK; t++) dsb[t] = regs_to_operand<vec8>(sacc[t >> 1], t & 1);
      // dq^T += K^T . dS^T
      const T* kl = Kt + t_lane;
#pragma unroll
      for (int db = 0; db < DBLK; db++)
#pragma unroll
        for (int t = 0; t < 2 * NBLK; t++) {
          const vec8 ka = transposed_operand<vec8>(kl, ((16 * t) * TP + 32 * db) * 2, ((16 * t + 8) * TP + 32 * db) * 2);
          dqacc[db] = TR::mfma32(ka, dsb[t], dqacc[db]);
        }
    }
    __syncthreads();
  }

  const float l_tot = l_run + __shfl_xor(l_run, 32);
  const int qi = qw0 + lq;
  if (a.dq_splits > 1) {
    if (qi < f.L) store_dq_partial<D>(a, piece, ((long long)b * f.Hq + h) * f.L + qi, lh, dqacc, m_use * c, l_tot, delta);
    return;
  }
  if (qi < f.L) {
    const long long row_id = ((long long)b * f.Hq + h) * f.L + qi;
    // log2 of the row's sum of exponentials, the unit the second kernel's exp2 wants
    // a row whose keys are all hidden (possible with an attnMask): dq = 0, and a statistic that gives it weight 0 below
    const bool seen = l_tot > 0.f;
    if (lh == 0) *(float2*)(a.stats + 2 * row_id) = make_float2(seen ? m_use * c + __log2f(l_tot) : 1e30f, delta);
    const float w = seen ? f.scale / l_tot : 0.f;
    T* dqp = (T*)a.dq + b * a.dqs[0] + h * a.dqs[1] + qi * a.dqs[2];
#pragma unroll
    for (int db = 0; db < DBLK; db++)
#pragma unroll
      for (int rg = 0; rg < 4; rg++) {
        f32x4 x;
#pragma unroll
        for (int i = 0; i < 4; i++) x[i] = seen ? dqacc[db][4 * rg + i] * w : 0.f;
        if (PAD && 32 * db + 8 * rg + 4 * lh >= f.D) continue;
        *(typename TR::vec4*)(dqp + 32 * db + 8 * rg + 4 * lh) = __builtin_convertvector(x, typename TR::vec4);
      }
  }
}

// ---- kernel 2: dk, dv ---------------------------------------------------------------------------------------------------
template <typename TR, int D, bool CAUSAL, bool MASKED, bool PAD>
__global__ __launch_bounds__(256, (D > 64 ? 1 : 2)) void backward_dkv_mfma_kernel(BwdArgs a) {
  typedef typename TR::elem T;
  typedef typename TR::vec8 vec8;
  typedef BwdLds<D> Lds;
  constexpr int RP = Lds::RP, TP = Lds::TP;
  constexpr int KSTEPS = D / 16, DBLK = D / 32;
  constexpr int NLD = (BQ * D / 8) / 256;
  const KArgs& f = a.f;

  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  T* smem = (T*)smem_raw;
  float* sstats = (float*)(smem_raw + 2 * Lds::KV_STAGE * 2);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lq = lane & 31, lh = lane >> 5;

  const int nkb = (f.S + BM - 1) / BM;
  const int nsplit = a.dkv_splits;
  int wg, split;  // this workgroup takes tiles split, split + nsplit, ... of key-block workgroup wg
  split_of_workgroup(blockIdx.x, nsplit, f.B * f.Hkv, &wg, &split);
  int pair, kb;  // the first key block is seen by every query row: the longest
  map_workgroup(wg, f.B * f.Hkv, nkb, &pair, &kb);
  const int hk = pair % f.Hkv, b = pair / f.Hkv;
  const int k0 = kb * BM, kw0 = k0 + wave * 32;
  const int S = keys_of_batch(f, b);  // rows of dk / dv from here to f.S are written as zeros
  if (k0 >= S) {
    zero_key_rows<TR, D, PAD>(a, split, b, hk, kw0 + lq, lh);
    return;
  }
  const bool wave_live = kw0 < S;
  const int coff = CAUSAL ? causal_offset(f, S) : 0;

  // ---- this lane's key: k and v rows as B operands -------------------------------------------------------------------------
  vec8 kreg[KSTEPS], vreg[KSTEPS];
  {
    int row = kw0 + lq;
    row = row < S ? row : S - 1;
    const T* kr = (const T*)f.k + b * f.ks[0] + hk * f.ks[1] + row * f.ks[2] + 8 * lh;
    const T* vr = (const T*)f.v + b * f.vs[0] + hk * f.vs[1] + row * f.vs[2] + 8 * lh;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) {
      if (PAD && 16 * ks + 8 * lh >= f.D) {
#pragma unroll
        for (int i = 0; i < 8; i++) kreg[ks][i] = (T)0.f, vreg[ks][i] = (T)0.f;
        continue;
      }
      kreg[ks] = *(const vec8*)(kr + 16 * ks);
      vreg[ks] = *(const vec8*)(vr + 16 * ks);
    }
  }
  f32x16 dkacc[DBLK], dvacc[DBLK];
#pragma unroll
  for (int i = 0; i < DBLK; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) dkacc[i][r] = 0.f, dvacc[i][r] = 0.f;
  const float c = f.scale * kLog2e;

  // Query tiles it0 .. ntq-1 of each of the G heads see keys of this workgroup.  They are taken from the last tile down,
  // the heads of a tile one after the other: every key block of a (batch, kv head) then starts at the same tile and walks
  // in step with the others (a block further down the causal triangle just stops earlier), so the tile one workgroup
  // fetches from HBM is in the XCD's L2 for the others.
  const int ntq = (f.L + BQ - 1) / BQ;
  int it0 = 0;
  if (CAUSAL) it0 = (k0 - coff > 0 ? k0 - coff : 0) / BQ;
  const int nt = ntq > it0 ? ntq - it0 : 0;
  const int total = f.G * nt;
  const bool walk_up = dkv_walks_up(a, CAUSAL);  // every second round of an XCD's workgroups (sdpa_common.h)
  auto tile_of = [&](int idx) __attribute__((always_inline)) { return walk_up ? it0 + idx / f.G : ntq - 1 - idx / f.G; };

  u32x4 qst[NLD], gst[NLD];
  float2 sst = make_float2(0.f, 0.f);
  int lrow[NLD], lcol[NLD], gcol[NLD];
  bool cval[NLD];  // PAD: as in the dq kernel
#pragma unroll
  for (int i = 0; i < NLD; i++) {
    const int cidx = tid + 256 * i;
    lrow[i] = cidx / (D / 8);
    lcol[i] = cidx % (D / 8);
    cval[i] = !PAD || 8 * lcol[i] < f.D;
    gcol[i] = cval[i] ? lcol[i] : 0;
  }
  const u32x4 zero4 = {0u, 0u, 0u, 0u};
  auto load_tile = [&](int idx) {
    const int h = hk * f.G + idx % f.G;
    const int i0 = tile_of(idx) * BQ;
    const T* qp = (const T*)f.q + b * f.qs[0] + h * f.qs[1];
    const T* gp = (const T*)a.dout + b * a.dos[0] + h * a.dos[1];
#pragma unroll
    for (int i = 0; i < NLD; i++) {
      int row = i0 + lrow[i];
      row = row < f.L ? row : f.L - 1;  // rows past the end re-read the last valid row (their weight is forced to 0)
      qst[i] = *(const u32x4*)(qp + row * f.qs[2] + 8 * gcol[i]);
      gst[i] = *(const u32x4*)(gp + row * a.dos[2] + 8 * gcol[i]);
    }
    if (tid < BQ) {
      const int row = i0 + tid;
      sst = row < f.L ? *(const float2*)(a.stats + 2 * (((long long)b * f.Hq + h) * f.L + row)) : make_float2(1e30f, 0.f);
    }
  };
  auto store_tile = [&](int stage) {
    T* Qr = smem + stage * Lds::KV_STAGE;
    T* Gr = Qr + BQ * RP;
    T* Qt = Gr + BQ * RP;
    T* Gt = Qt + BQ * TP;
#pragma unroll
    for (int i = 0; i < NLD; i++) {
      *(u32x4*)(Qr + lrow[i] * RP + 8 * lcol[i]) = cval[i] ? qst[i] : zero4;
      *(u32x4*)(Qt + lrow[i] * TP + 8 * lcol[i]) = cval[i] ? qst[i] : zero4;
      *(u32x4*)(Gr + lrow[i] * RP + 8 * lcol[i]) = cval[i] ? gst[i] : zero4;
      *(u32x4*)(Gt + lrow[i] * TP + 8 * lcol[i]) = cval[i] ? gst[i] : zero4;
    }
    if (tid < BQ) *(float2*)(sstats + stage * Lds::KV_STATS + 2 * tid) = sst;
  };
  const int r_lane = lq * RP + 8 * lh;
  const int t_lane = (4 * lh + ((lane & 15) >> 2)) * TP + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

  if (split < total) {
    load_tile(split);
    store_tile(0);
    if (split + nsplit < total) load_tile(split + nsplit);
  }
  __syncthreads();

  int cur = 0;
  for (int idx = split; idx < total; idx += nsplit, cur ^= 1) {
    if (idx + nsplit < total) {
      store_tile(cur ^ 1);
      if (idx + 2 * nsplit < total) load_tile(idx + 2 * nsplit);
    }
    const int i0 = tile_of(idx) * BQ;
    const int h_of_tile = hk * f.G + idx % f.G;
    if (wave_live && (!CAUSAL || kw0 <= i0 + BQ - 1 + coff)) {
      const T* Qr = smem + cur * Lds::KV_STAGE;
      const T* Gr = Qr + BQ * RP;
      const T* Qt = Gr + BQ * RP;
      const T* Gt = Qt + BQ * TP;
      const float* st = sstats + cur * Lds::KV_STATS;

      f32x16 sacc, dpacc;
#pragma unroll
      for (int r = 0; r < 16; r++) sacc[r] = 0.f, dpacc[r] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ks++) sacc = TR::mfma32(*(const vec8*)(Qr + r_lane + 16 * ks), kreg[ks], sacc);
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ks++) dpacc = TR::mfma32(*(const vec8*)(Gr + r_lane + 16 * ks), vreg[ks], dpacc);

      const int key = kw0 + lq;
      // only tiles on the diagonal, and the last key block, hide anything (rows past L carry lse = 1e30: weight 0)
      const bool need_mask = (CAUSAL && kw0 + 31 > i0 + coff) || kw0 + 32 > S;
#pragma unroll
      for (int rg = 0; rg < 4; rg++) {
        const f32x4 s0 = *(const f32x4*)(st + 2 * (8 * rg + 4 * lh));      // (lse2, delta) of rows 8rg+4lh+0, +1
        const f32x4 s1 = *(const f32x4*)(st + 2 * (8 * rg + 4 * lh) + 4);  // ... +2, +3
        const float lse2[4] = {s0[0], s0[2], s1[0], s1[2]};
        const float dl[4] = {s0[1], s0[3], s1[1], s1[3]};
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const int r = 4 * rg + e;
          float bias2 = 0.f;  // attnMask: the additive bias in log2 units, or -inf for a hidden key
          if (MASKED) {
            int qrow = i0 + 8 * rg + 4 * lh + e;
            qrow = qrow < f.L ? qrow : f.L - 1;
            const long long at = b * f.ms[0] + h_of_tile * f.ms[1] + qrow * f.ms[2] + (key < S ? key : S - 1) * f.ms[3];
            if (f.mask_kind == 1) {
              bias2 = ((const uint8_t*)f.mask)[at] == 0 ? -INFINITY : 0.f;
            } else {
              bias2 = (float)((const T*)f.mask)[at] * kLog2e;
            }
          }
          const float p = fast_exp2(fmaf(sacc[r], c, bias2 - lse2[e]));
          sacc[r] = p;
          dpacc[r] = p * (dpacc[r] - dl[e]);
        }
      }
      if (need_mask) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const int qrow = i0 + 8 * (r >> 2) + 4 * lh + (r & 3);
          if (key >= S || (CAUSAL && key > qrow + coff)) sacc[r] = 0.f, dpacc[r] = 0.f;
        }
      }
      vec8 pb[2], dsb[2];
#pragma unroll
      for (int t = 0; t < 2; t++) {
        pb[t] = regs_to_operand<vec8>(sacc, t);
        dsb[t] = regs_to_operand<vec8>(dpacc, t);
      }
      const T* gl = Gt + t_lane;
      const T* ql = Qt + t_lane;
#pragma unroll
      for (int db = 0; db < DBLK; db++)
#pragma unroll
        for (int t = 0; t < 2; t++) {
          const int lo = ((16 * t) * TP + 32 * db) * 2, hi = ((16 * t + 8) * TP + 32 * db) * 2;
          dvacc[db] = TR::mfma32(transposed_operand<vec8>(gl, lo, hi), pb[t], dvacc[db]);
          dkacc[db] = TR::mfma32(transposed_operand<vec8>(ql, lo, hi), dsb[t], dkacc[db]);
        }
    }
#pragma unroll
    for (int db = 0; db < DBLK; db++) pin_accumulator<(D > 64)>(dkacc[db]), pin_accumulator<(D > 64)>(dvacc[db]);
    __syncthreads();
  }

  store_key_grads<TR, D, PAD>(a, split, b, hk, kw0 + lq, lh, dkacc, dvacc, f.scale);
}

// ---- kernel 2 for head_dim 128: the same products with the tiles brought in by direct global->LDS loads ----------------
// With register-staged tiles the kernel above needs ~330 registers per lane at head_dim 128: one wavefront per SIMD,
// whose vector work nothing overlaps.  Here the Q / dout tiles (and the workgroup's V rows, once) go from global memory
// straight into LDS (global_load_lds_dwordx4: 64 lanes x 16 bytes = four 256-byte rows per instruction, unpadded), which
// frees the staging registers and the V fragments: under 256 registers, two wavefronts per SIMD.  Rows are 16 chunks of
// 16 bytes; chunk c of row r sits in slot c ^ f(r), f(r) = 4*(r%4) + (r/4)%4, which makes both the row-major operand
// reads (ds_read_b128) and the transposed ones (ds_read_b64_tr_b16) conflict-free on one copy of a tile.
//
// Eight wavefronts in two groups of four: both groups own the same 128 keys and take alternate tiles of the query
// stream, each with its own three-stage ring of tiles, and group 1's partial dk / dv are added to group 0's through
// LDS at the end.  Under a causal mask the first key block of a KV head sees every query row of every head of the
// group — the longest workgroup of the launch; two groups halve that critical path.
namespace dkv128 {
constexpr int D = 128;
constexpr int ROW_BYTES = D * 2;
constexpr int TILE_BYTES = BQ * ROW_BYTES;                // one 32-row tile of Q or dout
constexpr int STAGE_BYTES = 2 * TILE_BYTES + 2 * BQ * 4;  // Q, dout, (lse2, delta) per row
constexpr int NSTAGE = 3;
constexpr int V_BYTES = BM * ROW_BYTES;                   // the workgroup's V rows
constexpr int LDS_BYTES = V_BYTES + 2 * NSTAGE * STAGE_BYTES;
static_assert(LDS_BYTES >= 2 * 128 * 64 * 4, "the reduction of one gradient needs 64 KiB");
__device__ __forceinline__ int swz(int row) { return ((row & 3) << 2) | ((row >> 2) & 3); }
}  // namespace dkv128

typedef __attribute__((address_space(3))) void lds_void;

template <typename TR, bool CAUSAL>
__global__ __launch_bounds__(512, 1) void backward_dkv128_kernel(BwdArgs a) {
  using namespace dkv128;
  typedef typename TR::elem T;
  typedef typename TR::vec8 vec8;
  typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
  constexpr int KSTEPS = D / 16, DBLK = D / 32;
  const KArgs& f = a.f;

  extern __shared__ __attribute__((aligned(16))) char smem[];
  const unsigned smem_addr = (unsigned)(unsigned long)(lds_void*)smem;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int grp = wave >> 2, gw = wave & 3;  // group, wavefront inside the group
  const int lq = lane & 31, lh = lane >> 5;

  const int nkb = (f.S + BM - 1) / BM;
  const int nsplit = a.dkv_splits;
  int wg, split;  // this workgroup takes entries split, split + nsplit, ... of key-block workgroup wg
  split_of_workgroup(blockIdx.x, nsplit, f.B * f.Hkv, &wg, &split);
  int pair, kb;
  map_workgroup(wg, f.B * f.Hkv, nkb, &pair, &kb);
  const int hk = pair % f.Hkv, b = pair / f.Hkv;
  const int k0 = kb * BM, kw0 = k0 + gw * 32;
  const int S = keys_of_batch(f, b);  // rows of dk / dv from here to f.S are written as zeros
  if (k0 >= S) {
    if (grp == 0) zero_key_rows<TR, D>(a, split, b, hk, kw0 + lq, lh);
    return;
  }
  const int coff = CAUSAL ? causal_offset(f, S) : 0;

  // Issued as asm so that the compiler does not see stores to LDS (it would make every LDS read wait for all loads).
  auto dma16 = [&](const char* sbase, unsigned voff, unsigned lds_addr) __attribute__((always_inline)) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 3\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(sbase), "s"(lds_addr) : "memory", "m0");
  };
  auto dma4 = [&](const char* sbase, unsigned voff, unsigned lds_addr) __attribute__((always_inline)) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 3\n\tglobal_load_lds_dword %0, %1" ::"v"(voff), "s"(sbase), "s"(lds_addr) : "memory", "m0");
  };
  const int drow = lane >> 4, dslot = lane & 15;  // this lane's row and slot inside a 4-row group of a load

  // ---- the workgroup's V rows into LDS (wavefront w brings rows 16w .. 16w+15), this wavefront's K rows into registers ----
  {
    const char* vb = (const char*)((const T*)f.v + b * f.vs[0] + hk * f.vs[1] + (long long)k0 * f.vs[2]);
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int row = 16 * wave + 4 * i + drow;
      const int rowc = k0 + row < S ? row : S - 1 - k0;  // rows past the end re-read the last key (never stored)
      const unsigned voff = ((unsigned)rowc * (unsigned)f.vs[2] + 8u * (unsigned)(dslot ^ swz(row))) * 2u;
      dma16(vb, voff, smem_addr + (16 * wave + 4 * i) * ROW_BYTES);
    }
  }
  vec8 kreg[KSTEPS];
  {
    int row = kw0 + lq;
    row = row < S ? row : S - 1;
    const T* kr = (const T*)f.k + b * f.ks[0] + hk * f.ks[1] + row * f.ks[2] + 8 * lh;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) kreg[ks] = *(const vec8*)(kr + 16 * ks);
  }
  f32x16 dkacc[DBLK], dvacc[DBLK];
#pragma unroll
  for (int i = 0; i < DBLK; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) dkacc[i][r] = 0.f, dvacc[i][r] = 0.f;
  const float c = f.scale * kLog2e;

  // Query tiles it0 .. ntq-1 of each of the G heads see keys of this workgroup.  They are taken from the last tile down,
  // the heads of a tile one after the other: every key block of a (batch, kv head) then starts at the same tile and walks
  // in step with the others (a block further down the causal triangle just stops earlier), so the tile one workgroup
  // fetches from HBM is in the XCD's L2 for the others.  This workgroup's entries are split, split + nsplit, ... of that
  // list; entry idx of ITS list belongs to group idx % 2.
  const int ntq = (f.L + BQ - 1) / BQ;
  int it0 = 0;
  if (CAUSAL) it0 = (k0 - coff > 0 ? k0 - coff : 0) / BQ;
  const int nt = ntq > it0 ? ntq - it0 : 0;
  const int total = split < f.G * nt ? (f.G * nt - split + nsplit - 1) / nsplit : 0;
  const int niter = (total + 1) / 2;  // iterations of either group (the second may have one entry less)
  const bool walk_up = dkv_walks_up(a, CAUSAL);  // every second round of an XCD's workgroups (sdpa_common.h)
  auto tile_of = [&](int entry) __attribute__((always_inline)) { return walk_up ? it0 + entry / f.G : ntq - 1 - entry / f.G; };

  // wavefront gw of a group brings rows 8gw .. 8gw+7 of the Q tile and of the dout tile (two loads each) into the
  // group's ring; its first wavefront the statistics as well
  const unsigned ring_addr = smem_addr + V_BYTES + grp * NSTAGE * STAGE_BYTES;
  auto dma_tile = [&](int idx, int stage) __attribute__((always_inline)) {
    const int entry = split + nsplit * idx;
    const int h = hk * f.G + entry % f.G;
    const int i0 = tile_of(entry) * BQ;
    const char* qb = (const char*)((const T*)f.q + b * f.qs[0] + h * f.qs[1] + (long long)i0 * f.qs[2]);
    const char* gb = (const char*)((const T*)a.dout + b * a.dos[0] + h * a.dos[1] + (long long)i0 * a.dos[2]);
    const unsigned at = ring_addr + stage * STAGE_BYTES;
#pragma unroll
    for (int i = 0; i < 2; i++) {
      const int row = 8 * gw + 4 * i + drow;
      const int rowc = i0 + row < f.L ? row : f.L - 1 - i0;  // rows past the end re-read the last row (weight forced to 0)
      const unsigned chunk = (unsigned)(dslot ^ swz(row));
      dma16(qb, ((unsigned)rowc * (unsigned)f.qs[2] + 8u * chunk) * 2u, at + (8 * gw + 4 * i) * ROW_BYTES);
      dma16(gb, ((unsigned)rowc * (unsigned)a.dos[2] + 8u * chunk) * 2u, at + TILE_BYTES + (8 * gw + 4 * i) * ROW_BYTES);
    }
    if (gw == 0) {  // 32 rows x (lse2, delta): 64 floats, one per lane
      const char* sb = (const char*)(a.stats + 2 * (((long long)b * f.Hq + h) * f.L + i0));
      const int row = lane >> 1;
      const int rowc = i0 + row < f.L ? row : f.L - 1 - i0;
      dma4(sb, (unsigned)(2 * rowc + (lane & 1)) * 4u, at + 2 * TILE_BYTES);
    }
  };

  // ---- LDS operand addresses (bytes inside a tile), loop-invariant ----------------------------------------------------
  // row-major operand, k-step ks: row lq, chunk 2ks + lh  ->  lq*256 + 16*((2ks + lh) ^ f(lq)) = r_base ^ (32*ks)
  const unsigned r_base = (unsigned)(lq * ROW_BYTES + 16 * (lh ^ swz(lq)));
  // transposed operand (db, ld) of k-step t: this lane points at row 16t + 8ld + 4lh + s/4, elements
  // 32db + 16*dhalf + 4*(s%4) .. +3 (s = lane%16, dhalf = (lane/16)%2) and receives X[16t + 8ld + 4lh + 0..3][32db + lq]
  unsigned t_base[2];
  {
    const int s = lane & 15, dhalf = (lane >> 4) & 1;
#pragma unroll
    for (int ld = 0; ld < 2; ld++) {
      const int row = 8 * ld + 4 * lh + (s >> 2);  // f(row) does not depend on t
      const int c0 = 2 * dhalf + ((s & 3) >> 1);
      t_base[ld] = (unsigned)(row * ROW_BYTES + 16 * (c0 ^ swz(row)) + 8 * (s & 1));  // ^ (64*db) selects the 32-column block
    }
  }
  const char* vown = smem + 32 * gw * ROW_BYTES;
  const char* ring = smem + V_BYTES + grp * NSTAGE * STAGE_BYTES;

  // entries grp, grp + 2 of the list on their way, everything landed before the first use
  if (grp < total) dma_tile(grp, 0);
  if (grp + 2 < total) dma_tile(grp + 2, 1);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");

  const int key = kw0 + lq;
  int cur = 0;  // j % 3
  for (int j = 0; j < niter; j++) {
    const int idx = 2 * j + grp;
    const int nxt2 = cur == 0 ? 2 : cur - 1;  // (j + 2) % 3: last read in iteration j-1, which a barrier ended
    const bool more = idx + 4 < total;
    if (more) dma_tile(idx + 4, nxt2);
    if (idx < total) {
      const int i0 = tile_of(split + nsplit * idx) * BQ;
      const char* qt = ring + cur * STAGE_BYTES;
      const char* gt = qt + TILE_BYTES;
      const float* st = (const float*)(qt + 2 * TILE_BYTES);

      f32x16 sacc, dpacc;
#pragma unroll
      for (int r = 0; r < 16; r++) sacc[r] = 0.f, dpacc[r] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ks++) sacc = TR::mfma32(*(const vec8*)(qt + (r_base ^ (unsigned)(32 * ks))), kreg[ks], sacc);
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ks++)
        dpacc = TR::mfma32(*(const vec8*)(gt + (r_base ^ (unsigned)(32 * ks))), *(const vec8*)(vown + (r_base ^ (unsigned)(32 * ks))), dpacc);

#pragma unroll
      for (int rg = 0; rg < 4; rg++) {
        const f32x4 s0 = *(const f32x4*)(st + 2 * (8 * rg + 4 * lh));      // (lse2, delta) of rows 8rg+4lh+0, +1
        const f32x4 s1 = *(const f32x4*)(st + 2 * (8 * rg + 4 * lh) + 4);  // ... +2, +3
        const float lse2[4] = {s0[0], s0[2], s1[0], s1[2]};
        const float dl[4] = {s0[1], s0[3], s1[1], s1[3]};
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const int r = 4 * rg + e;
          const float p = fast_exp2(fmaf(sacc[r], c, -lse2[e]));
          sacc[r] = p;
          dpacc[r] = p * (dpacc[r] - dl[e]);
        }
      }
      // only tiles on or above the diagonal, the last key block and the last query tile hide anything; a wavefront whose
      // keys no row of the tile sees runs the tile with every weight 0
      if ((CAUSAL && kw0 + 31 > i0 + coff) || kw0 + 32 > S || i0 + BQ > f.L) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const int qrow = i0 + 8 * (r >> 2) + 4 * lh + (r & 3);
          if (key >= S || qrow >= f.L || (CAUSAL && key > qrow + coff)) sacc[r] = 0.f, dpacc[r] = 0.f;
        }
      }
      vec8 pb[2], dsb[2];
#pragma unroll
      for (int t = 0; t < 2; t++) {
        pb[t] = regs_to_operand<vec8>(sacc, t);
        dsb[t] = regs_to_operand<vec8>(dpacc, t);
      }
#pragma unroll
      for (int db = 0; db < DBLK; db++)
#pragma unroll
        for (int t = 0; t < 2; t++) {
          const unsigned lo = (t_base[0] ^ (unsigned)(64 * db)) + 16 * t * ROW_BYTES, hi = (t_base[1] ^ (unsigned)(64 * db)) + 16 * t * ROW_BYTES;
          const s16x4 glo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(gt + lo));
          const s16x4 ghi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(gt + hi));
          const s16x4 qlo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(qt + lo));
          const s16x4 qhi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(qt + hi));
          dvacc[db] = TR::mfma32(__builtin_bit_cast(vec8, __builtin_shufflevector(glo, ghi, 0, 1, 2, 3, 4, 5, 6, 7)), pb[t], dvacc[db]);
          dkacc[db] = TR::mfma32(__builtin_bit_cast(vec8, __builtin_shufflevector(qlo, qhi, 0, 1, 2, 3, 4, 5, 6, 7)), dsb[t], dkacc[db]);
        }
    }
    // Entry idx + 2 must have landed before the next iteration; the loads of entry idx + 4, issued above, may stay in
    // flight (four per wavefront, five for the one that also brings the statistics; they complete in issue order).
    if (more) {
      if (gw == 0) {
        asm volatile("s_waitcnt vmcnt(5)" ::: "memory");
      } else {
        asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
      }
    } else {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    __syncthreads();
    cur = cur == 2 ? 0 : cur + 1;
  }

  // ---- group 1's partial gradients join group 0's, one gradient (64 KiB of fp32) at a time ------------------------------
  float* red = (float*)smem;
  const int slot = gw * 64 + lane;
#pragma unroll
  for (int which = 0; which < 2; which++) {
    f32x16* acc = which == 0 ? dkacc : dvacc;
    if (grp == 1) {
#pragma unroll
      for (int db = 0; db < DBLK; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) red[(db * 16 + r) * 256 + slot] = acc[db][r];
    }
    __syncthreads();
    if (grp == 0) {
#pragma unroll
      for (int db = 0; db < DBLK; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[db][r] += red[(db * 16 + r) * 256 + slot];
    }
    __syncthreads();
  }

  if (grp == 0) store_key_grads<TR, D>(a, split, b, hk, key, lh, dkacc, dvacc, f.scale);
}

// ---- kernel 1 for head_dim 128 without an attnMask: the same products, K / V tiles by direct global->LDS loads ----------
// As in backward_dkv128_kernel: unpadded 256-byte rows, chunk c of row r at slot c ^ f(r), so one copy of the K tile
// serves the row-major reads (S^T = K.Q^T) and the transposed ones (dq^T += K^T.dS^T); a three-stage ring of 32-key tiles
// per workgroup, the loads of tile j+2 in flight while tile j is computed; no staging registers.
namespace dq128 {
using dkv128::ROW_BYTES;
using dkv128::swz;
constexpr int BN = 32;                        // keys per tile
constexpr int TILE_BYTES = BN * ROW_BYTES;    // one tile of K or V
constexpr int STAGE_BYTES = 2 * TILE_BYTES;
constexpr int NSTAGE = 3;
constexpr int LDS_BYTES = NSTAGE * STAGE_BYTES;
}  // namespace dq128

template <typename TR, bool CAUSAL>
__global__ __launch_bounds__(256, 2) void backward_dq128_kernel(BwdArgs a) {
  using namespace dq128;
  constexpr int D = 128;
  typedef typename TR::elem T;
  typedef typename TR::vec8 vec8;
  typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
  constexpr int KSTEPS = D / 16, DBLK = D / 32;
  const KArgs& f = a.f;

  extern __shared__ __attribute__((aligned(16))) char smem[];
  const unsigned smem_addr = (unsigned)(unsigned long)(lds_void*)smem;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lq = lane & 31, lh = lane >> 5;

  const int ntile = (f.L + BM - 1) / BM;
  int pair, in, piece;  // piece: this workgroup's share of the row block's key range (dq_splits > 1)
  {
    int n;
    split_of_workgroup(blockIdx.x, a.dq_splits, f.B * f.Hq, &n, &piece);
    map_workgroup(n, f.B * f.Hq, ntile, &pair, &in);
  }
  const int h = pair % f.Hq, b = pair / f.Hq;
  const int hk = h / f.G;
  const int rt = CAUSAL ? ntile - 1 - in : in;  // longest rows first
  const int q0 = rt * BM, qw0 = q0 + wave * 32;
  const bool wave_live = qw0 < f.L;

  // ---- this lane's query row: q and dout as B operands, delta = dout . out ------------------------------------------------
  vec8 qreg[KSTEPS], greg[KSTEPS];
  float delta;
  {
    int row = qw0 + lq;
    row = row < f.L ? row : f.L - 1;
    const T* qr = (const T*)f.q + b * f.qs[0] + h * f.qs[1] + row * f.qs[2] + 8 * lh;
    const T* gr = (const T*)a.dout + b * a.dos[0] + h * a.dos[1] + row * a.dos[2] + 8 * lh;
    const T* orow = (const T*)f.out + b * f.os[0] + h * f.os[1] + row * f.os[2] + 8 * lh;
    float part = 0.f;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) {
      qreg[ks] = *(const vec8*)(qr + 16 * ks);
      greg[ks] = *(const vec8*)(gr + 16 * ks);
      const vec8 o = *(const vec8*)(orow + 16 * ks);
#pragma unroll
      for (int i = 0; i < 8; i++) part = fmaf((float)o[i], (float)greg[ks][i], part);
    }
    delta = part + __shfl_xor(part, 32);
  }

  f32x16 dqacc[DBLK];
#pragma unroll
  for (int i = 0; i < DBLK; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) dqacc[i][r] = 0.f;
  const float c = f.scale * kLog2e;
  const float lazy = kLazyExp / c;
  float m_use = -1e30f, mc = m_use * c, l_run = 0.f;

  const int S = keys_of_batch(f, b);
  if (S == 0) {  // no keys (an empty cache entry): the output did not depend on q
    if (a.dq_splits > 1) return;  // the merge kernel writes the zeros
    const int qi = qw0 + lq;
    if (qi < f.L) {
      T* dqp = (T*)a.dq + b * a.dqs[0] + h * a.dqs[1] + qi * a.dqs[2];
      typename TR::vec4 zero;
#pragma unroll
      for (int i = 0; i < 4; i++) zero[i] = (T)0.f;
      for (int d = 4 * lh; d < D; d += 8) *(typename TR::vec4*)(dqp + d) = zero;
    }
    return;
  }
  const int coff = CAUSAL ? causal_offset(f, S) : 0;
  int ntiles_kv = (S + BN - 1) / BN;
  if (CAUSAL) {
    const int last = (q0 + BM - 1 < f.L - 1 ? q0 + BM - 1 : f.L - 1) + coff;  // last key any row of the workgroup sees
    const int lastkv = last < S - 1 ? last : S - 1;
    ntiles_kv = lastkv / BN + 1;
  }
  // this workgroup's tiles: all of them, or piece `piece` of dq_splits nearly equal ones (possibly none)
  const int t0 = (int)((long long)ntiles_kv * piece / a.dq_splits), t1 = (int)((long long)ntiles_kv * (piece + 1) / a.dq_splits);

  auto dma16 = [&](const char* sbase, unsigned voff, unsigned lds_addr) __attribute__((always_inline)) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 3\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(sbase), "s"(lds_addr) : "memory", "m0");
  };
  const int drow = lane >> 4, dslot = lane & 15;
  const T* kp = (const T*)f.k + b * f.ks[0] + hk * f.ks[1];
  const T* vp = (const T*)f.v + b * f.vs[0] + hk * f.vs[1];
  // wavefront w brings rows 8w .. 8w+7 of the K tile and of the V tile: two loads each
  auto dma_tile = [&](int jt, int stage) __attribute__((always_inline)) {
    const int kv0 = jt * BN;
    const char* kb = (const char*)(kp + (long long)kv0 * f.ks[2]);
    const char* vb = (const char*)(vp + (long long)kv0 * f.vs[2]);
    const unsigned at = smem_addr + stage * STAGE_BYTES;
#pragma unroll
    for (int i = 0; i < 2; i++) {
      const int row = 8 * wave + 4 * i + drow;
      const int rowc = kv0 + row < S ? row : S - 1 - kv0;  // rows past the end re-read the last key (hidden below)
      const unsigned chunk = (unsigned)(dslot ^ swz(row));
      dma16(kb, ((unsigned)rowc * (unsigned)f.ks[2] + 8u * chunk) * 2u, at + (8 * wave + 4 * i) * ROW_BYTES);
      dma16(vb, ((unsigned)rowc * (unsigned)f.vs[2] + 8u * chunk) * 2u, at + TILE_BYTES + (8 * wave + 4 * i) * ROW_BYTES);
    }
  };
  const unsigned r_base = (unsigned)(lq * ROW_BYTES + 16 * (lh ^ swz(lq)));
  unsigned t_base[2];
  {
    const int s = lane & 15, dhalf = (lane >> 4) & 1;
#pragma unroll
    for (int ld = 0; ld < 2; ld++) {
      const int row = 8 * ld + 4 * lh + (s >> 2);
      const int c0 = 2 * dhalf + ((s & 3) >> 1);
      t_base[ld] = (unsigned)(row * ROW_BYTES + 16 * (c0 ^ swz(row)) + 8 * (s & 1));
    }
  }

  if (t0 < t1) dma_tile(t0, 0);
  if (t0 + 1 < t1) dma_tile(t0 + 1, 1);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");

  int cur = 0;
  for (int jt = t0; jt < t1; jt++) {
    const int kv0 = jt * BN;
    const int nxt2 = cur == 0 ? 2 : cur - 1;  // stage of tile jt + 2: last read in iteration jt-1, which a barrier ended
    const bool more = jt + 2 < t1;
    if (more) dma_tile(jt + 2, nxt2);
    if (wave_live && (!CAUSAL || kv0 <= qw0 + 31 + coff)) {
      const char* kt = smem + cur * STAGE_BYTES;
      const char* vt = kt + TILE_BYTES;
      f32x16 sacc, dpacc;
#pragma unroll
      for (int r = 0; r < 16; r++) sacc[r] = 0.f, dpacc[r] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ks++) sacc = TR::mfma32(*(const vec8*)(kt + (r_base ^ (unsigned)(32 * ks))), qreg[ks], sacc);
      if ((CAUSAL && kv0 + BN - 1 > qw0 + coff) || kv0 + BN > S) {
        const int qi = qw0 + lq + coff;
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const int key = kv0 + 8 * (r >> 2) + 4 * lh + (r & 3);
          if (key >= S || (CAUSAL && key > qi)) sacc[r] = -INFINITY;
        }
      }
      float mloc = sacc[0];
#pragma unroll
      for (int r = 1; r < 16; r++) mloc = fmaxf(mloc, sacc[r]);
      mloc = fmaxf(mloc, __shfl_xor(mloc, 32));
      if (__builtin_expect(__builtin_amdgcn_ballot_w64(mloc > m_use + lazy) != 0, 0)) {
        const float m_new = fmaxf(m_use, mloc);
        const float alpha = fast_exp2((m_use - m_new) * c);
        m_use = m_new;
        mc = m_new * c;
        l_run *= alpha;
#pragma unroll
        for (int i = 0; i < DBLK; i++)
#pragma unroll
          for (int r = 0; r < 16; r++) dqacc[i][r] *= alpha;
      }
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ks++) dpacc = TR::mfma32(*(const vec8*)(vt + (r_base ^ (unsigned)(32 * ks))), greg[ks], dpacc);
      float psum = 0.f;
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const float p = fast_exp2(fmaf(sacc[r], c, -mc));  // relative to m_use; normalised at the end
        psum += p;
        sacc[r] = p * (dpacc[r] - delta);
      }
      l_run += psum;
      vec8 dsb[2];
#pragma unroll
      for (int t = 0; t < 2; t++) dsb[t] = regs_to_operand<vec8>(sacc, t);
#pragma unroll
      for (int db = 0; db < DBLK; db++)
#pragma unroll
        for (int t = 0; t < 2; t++) {
          const unsigned lo = (t_base[0] ^ (unsigned)(64 * db)) + 16 * t * ROW_BYTES, hi = (t_base[1] ^ (unsigned)(64 * db)) + 16 * t * ROW_BYTES;
          const s16x4 klo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(kt + lo));
          const s16x4 khi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(kt + hi));
          dqacc[db] = TR::mfma32(__builtin_bit_cast(vec8, __builtin_shufflevector(klo, khi, 0, 1, 2, 3, 4, 5, 6, 7)), dsb[t], dqacc[db]);
        }
    }
    // tile jt+1 must have landed before the next iteration; the four loads of tile jt+2 may stay in flight
    if (more) {
      asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
    } else {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    __syncthreads();
    cur = cur == 2 ? 0 : cur + 1;
  }

  const float l_tot = l_run + __shfl_xor(l_run, 32);
  const int qi = qw0 + lq;
  if (a.dq_splits > 1) {
    if (qi < f.L) store_dq_partial<D>(a, piece, ((long long)b * f.Hq + h) * f.L + qi, lh, dqacc, m_use * c, l_tot, delta);
    return;
  }
  if (qi < f.L) {
    const long long row_id = ((long long)b * f.Hq + h) * f.L + qi;
    if (lh == 0) *(float2*)(a.stats + 2 * row_id) = make_float2(m_use * c + __log2f(l_tot), delta);
    const float w = f.scale / l_tot;
    T* dqp = (T*)a.dq + b * a.dqs[0] + h * a.dqs[1] + qi * a.dqs[2];
#pragma unroll
    for (int db = 0; db < DBLK; db++)
#pragma unroll
      for (int rg = 0; rg < 4; rg++) {
        f32x4 x;
#pragma unroll
        for (int i = 0; i < 4; i++) x[i] = dqacc[db][4 * rg + i] * w;
        *(typename TR::vec4*)(dqp + 32 * db + 8 * rg + 4 * lh) = __builtin_convertvector(x, typename TR::vec4);
      }
  }
}

template <typename TR, int D, bool CAUSAL, bool MASKED, bool PAD>
int launch_k(const BwdArgs& args, hipStream_t stream) {
  BwdArgs a = args;
  // the callers keep to this (the records of a split are laid out for D, rows are read in 16-byte chunks)
  if (PAD && (a.dkv_splits > 1 || a.dq_splits > 1 || a.f.D % 8 != 0 || a.f.D >= D || a.f.D < 8)) return (int)hipErrorInvalidValue;
  typedef BwdLds<D> Lds;
  // with an attnMask, head_dim 128 takes the register-staged dk/dv kernel: the mask's 16 values per tile do not fit the
  // 256 registers of the direct-to-LDS one
  constexpr bool DMA = D == 128 && !MASKED && !PAD;
  static hipError_t state1[kMaxDevices], state2[kMaxDevices];
  static bool done1[kMaxDevices], done2[kMaxDevices];
  hipError_t e = DMA ? grant_dynamic_lds((const void*)backward_dq128_kernel<TR, CAUSAL>, dq128::LDS_BYTES, state1, done1)
                     : grant_dynamic_lds((const void*)backward_dq_mfma_kernel<TR, D, CAUSAL, MASKED, PAD>, DqTile<D>::BYTES, state1, done1);
  if (e != hipSuccess) return (int)e;
  if (DMA) {
    e = grant_dynamic_lds((const void*)backward_dkv128_kernel<TR, CAUSAL>, dkv128::LDS_BYTES, state2, done2);
  } else {
    e = grant_dynamic_lds((const void*)backward_dkv_mfma_kernel<TR, D, CAUSAL, MASKED, PAD>, Lds::KV_BYTES, state2, done2);
  }
  if (e != hipSuccess) return (int)e;
  const long long g1 = (long long)a.f.B * a.f.Hq * ((a.f.L + BM - 1) / BM) * a.dq_splits;
  const long long g2 = (long long)a.f.B * a.f.Hkv * ((a.f.S + BM - 1) / BM) * a.dkv_splits;
  static int round_cache[kMaxDevices];
  a.dkv_round = !CAUSAL ? 0
                : DMA   ? dkv_round_of((const void*)backward_dkv128_kernel<TR, CAUSAL>, 512, dkv128::LDS_BYTES, round_cache)
                        : dkv_round_of((const void*)backward_dkv_mfma_kernel<TR, D, CAUSAL, MASKED, PAD>, 256, Lds::KV_BYTES, round_cache);
  if (DMA) {
    hipLaunchKernelGGL((backward_dq128_kernel<TR, CAUSAL>), dim3((unsigned)g1), dim3(256), dq128::LDS_BYTES, stream, a);
  } else {
    hipLaunchKernelGGL((backward_dq_mfma_kernel<TR, D, CAUSAL, MASKED, PAD>), dim3((unsigned)g1), dim3(256), DqTile<D>::BYTES, stream, a);
  }
  e = hipGetLastError();
  if (e != hipSuccess) return (int)e;
  if (a.dq_splits > 1) {
    const int rc = launch_backward_dq_merge<typename TR::elem>(a, stream);
    if (rc != 0) return rc;
  }
  if (DMA) {
    hipLaunchKernelGGL((backward_dkv128_kernel<TR, CAUSAL>), dim3((unsigned)g2), dim3(512), dkv128::LDS_BYTES, stream, a);
  } else {
    hipLaunchKernelGGL((backward_dkv_mfma_kernel<TR, D, CAUSAL, MASKED, PAD>), dim3((unsigned)g2), dim3(256), Lds::KV_BYTES, stream, a);
  }
  e = hipGetLastError();
  if (e != hipSuccess || a.dkv_splits == 1) return (int)e;
  return launch_backward_dkv_sum<typename TR::elem>(a, stream);
}

template <typename TR, int D, bool PAD>
int launch_d(const BwdArgs& a, hipStream_t stream) {
  if (a.f.mask_kind != 0) return launch_k<TR, D, false, true, PAD>(a, stream);  // exclusive with causal (validated)
  return a.f.causal ? launch_k<TR, D, true, false, PAD>(a, stream) : launch_k<TR, D, false, false, PAD>(a, stream);
}

template <typename TR>
int launch_t(const BwdArgs& a, hipStream_t stream) {
  if (a.f.D == 64) return launch_d<TR, 64, false>(a, stream);
  if (a.f.D == 128) return launch_d<TR, 128, false>(a, stream);
  // any other multiple of 8 up to 128: the register-staged kernels of the next size up, the missing columns as zeros
  return a.f.D < 64 ? launch_d<TR, 64, true>(a, stream) : launch_d<TR, 128, true>(a, stream);
}

}  // namespace

int launch_backward_mfma(const BwdArgs& a, int dtype, hipStream_t stream) {
  return dtype == 1 ? launch_t<F16>(a, stream) : launch_t<BF16>(a, stream);
}

}  // namespace ttsdpa
