// Attention backward for fp32 tensors on the gfx950 fp32 matrix cores (v_mfma_f32_32x32x2_f32: full fp32 products and
// sums), head_dim 64 or 128, optional causal mask (either alignment) or attnMask, per-batch key counts, grouped heads.
// fp32 is the reference's default dtype.  The reference has no attention backward (reference
// src/Function/FuncNNLayer.h:267 is NOT_IMPLEMENTED); this is the chain rule through its forward chain matmul -> scale -> bias -> softmax -> matmul
// (src/Function/FuncNNLayer.h:237-265, softmax step as src/Operation/OpNNLayerCpu.h:79-109):
//   P_ij = exp(scale * q_i.k_j - lse_i)    dP_ij = dout_i.v_j    delta_i = dout_i.out_i    dS_ij = P_ij (dP_ij - delta_i)
//   dq_i = scale * sum_j dS_ij k_j         dk_j = scale * sum_i dS_ij q_i                  dv_j = sum_i P_ij dout_i
//
// The two kernels of the 16-bit matrix-core backward, restated for an instruction that contracts two elements at a
// time (A: 32 rows x 2, B: 2 x 32 columns, lane l supplies row / column l%32 and contraction element l/32; C: lane l
// holds column l%32 and rows 8*(r/4) + 4*(l/32) + r%4 in register r):
//   1. backward_dq_f32_kernel — a workgroup owns 128 query rows of one (batch, query head), a wavefront 32 of them (one
//      per lane column), and streams the keys in tiles of 32: S^T = K.Q^T, online softmax with a lazily raised maximum,
//      dP^T = V.dout^T, dS^T, dq^T += K^T.dS^T; at the end dq = scale/l * accumulator, (lse, delta) to scratch.
//   2. backward_dkv_f32_kernel — a workgroup owns 128 keys of one (batch, kv head), a wavefront 32 of them, and streams
//      the query rows of every head of the group in tiles of 32: S = Q.K^T, P from lse, dP = dout.V^T, dS,
//      dv^T += dout^T.P, dk^T += Q^T.dS.  When the launch has too few key blocks to fill and balance the chip (under a
//      causal mask the first key block sees every query tile, the last one a few), the tiles of a key block's query
//      stream are dealt out to 2-4 workgroups, which leave partial dk / dv in scratch, and
//   3. backward_dkv_sum_kernel adds the partials in a fixed order.
// In the score products MFMA ks contracts head_dim elements ks (lanes 0-31) and ks + D/2 (lanes 32-63): the operand a
// lane keeps in registers is one contiguous half of its row.  In the gradient products MFMA t contracts the two rows
// that the lane halves hold in accumulator register t, so P and dS feed the matrix cores straight from registers.
// The streamed tiles sit in LDS once, rows padded by one float: a column of 32 rows (score products) and a run of 32
// consecutive floats of one row (gradient products) both fall into 32 different banks.
// No atomics: a fixed summation order, reproducible results.

#include "sdpa_common.h"

namespace ttsdpa {

namespace {

constexpr int BM = 128;  // rows of the owning side per workgroup (queries in kernel 1, keys in kernel 2)
constexpr int BT = 32;   // rows of the streamed side per tile
constexpr float kLazyExp = 8.f;

template <int D>
struct BwdF32Lds {
  static constexpr int PITCH = D + 1;                 // floats per tile row
  static constexpr int TILE = BT * PITCH;             // K or V (kernel 1), Q or dout (kernel 2)
  static constexpr int STAGE = 2 * TILE + 2 * BT;     // two tiles and, in kernel 2, (lse2, delta) per query row
  static constexpr int BYTES = 2 * STAGE * 4;         // double-buffered
  static constexpr int NLD = BT * D / 4 / 256;        // 16-byte chunks per thread per tile
};

__device__ __forceinline__ f32x16 zero16() {
  f32x16 x;
#pragma unroll
  for (int r = 0; r < 16; r++) x[r] = 0.f;
  return x;
}

// acc0 + acc1 += X . Y^T over head_dim, X rows from LDS (this lane: row l%32, its half of head_dim), Y from registers;
// two accumulators over alternate steps, so that an MFMA never waits for the one before it.
template <int D>
__device__ __forceinline__ f32x16 score_product(const float* xrow, const float (&yreg)[D / 2]) {
  f32x16 s0 = zero16(), s1 = zero16();
#pragma unroll
  for (int ks = 0; ks < D / 2; ks += 2) {
    s0 = __builtin_amdgcn_mfma_f32_32x32x2f32(xrow[ks], yreg[ks], s0, 0, 0, 0);
    s1 = __builtin_amdgcn_mfma_f32_32x32x2f32(xrow[ks + 1], yreg[ks + 1], s1, 0, 0, 0);
  }
#pragma unroll
  for (int r = 0; r < 16; r++) s0[r] += s1[r];
  return s0;
}

// This lane's half (lh) of a row of D floats, 16 bytes at a time; the row holds `have` floats (a multiple of 4, at most
// D), the rest reads as zeros.
template <int D>
__device__ __forceinline__ void load_half_row(const float* row, int lh, float (&reg)[D / 2], int have) {
  const float* p = row + lh * (D / 2);
#pragma unroll
  for (int i = 0; i < D / 8; i++) {
    f32x4 t = {0.f, 0.f, 0.f, 0.f};
    if (lh * (D / 2) + 4 * i < have) t = *(const f32x4*)(p + 4 * i);
#pragma unroll
    for (int e = 0; e < 4; e++) reg[4 * i + e] = t[e];
  }
}

// ---- kernel 1: dq, lse, delta -------------------------------------------------------------------------------------
// MASKED: an attnMask (exclusive with CAUSAL) whose keys can be read four at a time, as in the forward kernel.
// PAD (both kernels): the tensors' head_dim f.D is a multiple of 4 below D.  The 16-byte chunks of a row beyond it are
// taken as zeros (q, k: nothing added to a score; dout, v: nothing added to dP or delta; gradient columns beyond f.D are
// not stored); everything else is the kernel for head_dim D.  No splits (their records are laid out for D).
template <int D, bool CAUSAL, bool MASKED, bool PAD>
__global__ __launch_bounds__(256, (D > 64 ? 1 : 2)) void backward_dq_f32_kernel(BwdArgs a) {
  typedef BwdF32Lds<D> Lds;
  constexpr int PITCH = Lds::PITCH, NLD = Lds::NLD, DBLK = D / 32;
  const KArgs& f = a.f;
  const int have = PAD ? f.D : D;  // floats of a row

  extern __shared__ __attribute__((aligned(16))) float smem_bwd_f32[];
  float* smem = smem_bwd_f32;

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

  const float* kp = (const float*)f.k + b * f.ks[0] + hk * f.ks[1];
  const float* vp = (const float*)f.v + b * f.vs[0] + hk * f.vs[1];

  // ---- this lane's query row: halves of q and dout as B operands, delta = dout . out --------------------------------------
  float qreg[D / 2], greg[D / 2];
  float delta;
  {
    int row = qw0 + lq;
    row = row < f.L ? row : f.L - 1;
    load_half_row<D>((const float*)f.q + b * f.qs[0] + h * f.qs[1] + row * f.qs[2], lh, qreg, have);
    load_half_row<D>((const float*)a.dout + b * a.dos[0] + h * a.dos[1] + row * a.dos[2], lh, greg, have);
    const float* orow = (const float*)f.out + b * f.os[0] + h * f.os[1] + row * f.os[2] + lh * (D / 2);
    float part = 0.f;
#pragma unroll
    for (int i = 0; i < D / 8; i++) {
      if (PAD && lh * (D / 2) + 4 * i >= have) continue;
      const f32x4 o = *(const f32x4*)(orow + 4 * i);
#pragma unroll
      for (int e = 0; e < 4; e++) part = fmaf(o[e], greg[4 * i + e], part);
    }
    delta = part + __shfl_xor(part, 32);
  }

  f32x16 dqacc[DBLK];
#pragma unroll
  for (int i = 0; i < DBLK; i++) dqacc[i] = zero16();
  const float c = f.scale * kLog2e;
  const float lazy = kLazyExp / c;
  float m_use = -1e30f, mc = m_use * c, l_run = 0.f;

  const int S = keys_of_batch(f, b);
  if (S == 0) {  // no keys (an empty cache entry): the output did not depend on q
    if (a.dq_splits > 1) return;  // the merge kernel writes the zeros
    const int qi = qw0 + lq;
    if (qi < f.L) {
      float* dqp = (float*)a.dq + b * a.dqs[0] + h * a.dqs[1] + qi * a.dqs[2];
      for (int d = 4 * lh; d < have; d += 8) *(f32x4*)(dqp + d) = (f32x4){0.f, 0.f, 0.f, 0.f};
    }
    return;
  }
  const int coff = CAUSAL ? causal_offset(f, S) : 0;
  int ntiles_kv = (S + BT - 1) / BT;
  if (CAUSAL) {
    const int last = (q0 + BM - 1 < f.L - 1 ? q0 + BM - 1 : f.L - 1) + coff;  // last key any row of the workgroup sees
    const int lastkv = last < S - 1 ? last : S - 1;
    ntiles_kv = lastkv / BT + 1;
  }
  // this workgroup's tiles: all of them, or piece `piece` of dq_splits nearly equal ones (possibly none)
  const int t0 = (int)((long long)ntiles_kv * piece / a.dq_splits), t1 = (int)((long long)ntiles_kv * (piece + 1) / a.dq_splits);

  // ---- global -> register -> LDS staging of one K/V tile (thread t moves 16-byte chunks t, t+256, ...) ----------------------
  f32x4 kst[NLD], vst[NLD];
  int lrow[NLD], lcol[NLD], gcol[NLD];
  bool cval[NLD];  // PAD: the chunk lies inside the tensors' rows; the others are loaded from the row's first chunk instead
                   // (the loads stay unconditional) and reach LDS as zeros
#pragma unroll
  for (int i = 0; i < NLD; i++) {
    const int cidx = tid + 256 * i;
    lrow[i] = cidx / (D / 4);
    lcol[i] = cidx % (D / 4);
    cval[i] = !PAD || 4 * lcol[i] < have;
    gcol[i] = cval[i] ? lcol[i] : 0;
  }
  auto load_tile = [&](int kv0) {
#pragma unroll
    for (int i = 0; i < NLD; i++) {
      int key = kv0 + lrow[i];
      key = key < S ? key : S - 1;  // rows past the end re-read the last valid row (hidden below)
      kst[i] = *(const f32x4*)(kp + key * f.ks[2] + 4 * gcol[i]);
      vst[i] = *(const f32x4*)(vp + key * f.vs[2] + 4 * gcol[i]);
    }
  };
  auto store_tile = [&](int stage) {
    float* Ks = smem + stage * Lds::STAGE;
    float* Vs = Ks + Lds::TILE;
#pragma unroll
    for (int i = 0; i < NLD; i++)
#pragma unroll
      for (int e = 0; e < 4; e++) {  // rows are not 16-byte aligned
        Ks[lrow[i] * PITCH + 4 * lcol[i] + e] = cval[i] ? kst[i][e] : 0.f;
        Vs[lrow[i] * PITCH + 4 * lcol[i] + e] = cval[i] ? vst[i][e] : 0.f;
      }
  };
  const int s_lane = lq * PITCH + lh * (D / 2);  // score products: row l%32, this lane's half of head_dim
  const int g_lane = 4 * lh * PITCH + lq;        // gradient product: + (8*(t/4) + t%4) * PITCH + 32*db

  if (t0 < t1) {
    load_tile(t0 * BT);
    store_tile(0);
    if (t0 + 1 < t1) load_tile((t0 + 1) * BT);
  }
  __syncthreads();

  for (int jt = t0; jt < t1; jt++) {
    const int kv0 = jt * BT;
    const int cur = (jt - t0) & 1;
    if (jt + 1 < t1) {
      store_tile(cur ^ 1);  // stage cur^1 was last read before the barrier that ended the previous iteration
      if (jt + 2 < t1) load_tile(kv0 + 2 * BT);
    }
    if (wave_live && (!CAUSAL || kv0 <= qw0 + 31 + coff)) {
      const float* Ks = smem + cur * Lds::STAGE;
      const float* Vs = Ks + Lds::TILE;

      f32x16 s = score_product<D>(Ks + s_lane, qreg);  // S^T = K . Q^T
      if ((CAUSAL && kv0 + BT - 1 > qw0 + coff) || kv0 + BT > S) {
        const int qi = qw0 + lq + coff;
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const int key = kv0 + 8 * (r >> 2) + 4 * lh + (r & 3);
          if (key >= S || (CAUSAL && key > qi)) s[r] = -INFINITY;
        }
      }
      if (MASKED) {
        int qi = qw0 + lq;
        qi = qi < f.L ? qi : f.L - 1;
        apply_attn_mask<float, true>(f, s, b * f.ms[0] + h * f.ms[1] + qi * f.ms[2], kv0, lh, S, 1.f / f.scale);
      }
      float mloc = s[0];
#pragma unroll
      for (int r = 1; r < 16; r++) mloc = fmaxf(mloc, s[r]);
      mloc = fmaxf(mloc, __shfl_xor(mloc, 32));
      if (__builtin_amdgcn_ballot_w64(mloc > m_use + lazy) != 0) {
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
      const f32x16 dp = score_product<D>(Vs + s_lane, greg);  // dP^T = V . dout^T
      float psum = 0.f;
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const float p = fast_exp2(fmaf(s[r], c, -mc));  // relative to m_use; normalised at the end
        psum += p;
        s[r] = p * (dp[r] - delta);
      }
      l_run += psum;
      // dq^T += K^T . dS^T
      const float* kl = Ks + g_lane;
#pragma unroll
      for (int t = 0; t < 16; t++)
#pragma unroll
        for (int db = 0; db < DBLK; db++)
          dqacc[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(kl[(8 * (t >> 2) + (t & 3)) * PITCH + 32 * db], s[t], dqacc[db], 0, 0, 0);
    }
#pragma unroll
    for (int db = 0; db < DBLK; db++) pin_accumulator<(D > 64)>(dqacc[db]);
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
    float* dqp = (float*)a.dq + b * a.dqs[0] + h * a.dqs[1] + qi * a.dqs[2];
#pragma unroll
    for (int db = 0; db < DBLK; db++)
#pragma unroll
      for (int rg = 0; rg < 4; rg++) {
        f32x4 x;
#pragma unroll
        for (int i = 0; i < 4; i++) x[i] = seen ? dqacc[db][4 * rg + i] * w : 0.f;
        if (PAD && 32 * db + 8 * rg + 4 * lh >= have) continue;
        *(f32x4*)(dqp + 32 * db + 8 * rg + 4 * lh) = x;
      }
  }
}

// ---- kernel 2: dk, dv -----------------------------------------------------------------------------------------------
// MASKED reads one mask value per score (a key is a lane column here, the mask's rows run across registers); with its
// addressing the head_dim-64 variant no longer fits two wavefronts per SIMD either.
template <int D, bool CAUSAL, bool MASKED, bool PAD>
__global__ __launch_bounds__(256, (D > 64 || MASKED ? 1 : 2)) void backward_dkv_f32_kernel(BwdArgs a) {
  typedef BwdF32Lds<D> Lds;
  constexpr int PITCH = Lds::PITCH, NLD = Lds::NLD, DBLK = D / 32;
  const KArgs& f = a.f;
  const int have = PAD ? f.D : D;  // floats of a row

  extern __shared__ __attribute__((aligned(16))) float smem_bwd_f32[];
  float* smem = smem_bwd_f32;

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
  const int S = keys_of_batch(f, b);
  const int key = kw0 + lq;
  float* dkp = (float*)a.dk + b * a.dks[0] + hk * a.dks[1] + key * a.dks[2];
  float* dvp = (float*)a.dv + b * a.dvs[0] + hk * a.dvs[1] + key * a.dvs[2];
  if (nsplit > 1) {  // partial sums: dense [split][dk | dv][B][Hkv][S][D]
    const long long plane = (long long)f.B * f.Hkv * f.S * D;
    dkp = a.partial + 2 * split * plane + (((long long)b * f.Hkv + hk) * f.S + key) * D;
    dvp = dkp + plane;
  }
  if (k0 >= S) {  // keys no query row attends to (at or beyond the batch entry's key count): zeros
    if (key < f.S)
      for (int d = 4 * lh; d < have; d += 8) {
        *(f32x4*)(dkp + d) = (f32x4){0.f, 0.f, 0.f, 0.f};
        *(f32x4*)(dvp + d) = (f32x4){0.f, 0.f, 0.f, 0.f};
      }
    return;
  }
  const bool wave_live = kw0 < S;
  const int coff = CAUSAL ? causal_offset(f, S) : 0;

  // ---- this lane's key: halves of its k and v rows as B operands ----------------------------------------------------------
  float kreg[D / 2], vreg[D / 2];
  {
    const int row = key < S ? key : S - 1;
    load_half_row<D>((const float*)f.k + b * f.ks[0] + hk * f.ks[1] + row * f.ks[2], lh, kreg, have);
    load_half_row<D>((const float*)f.v + b * f.vs[0] + hk * f.vs[1] + row * f.vs[2], lh, vreg, have);
  }
  f32x16 dkacc[DBLK], dvacc[DBLK];
#pragma unroll
  for (int i = 0; i < DBLK; i++) dkacc[i] = zero16(), dvacc[i] = zero16();
  const float c = f.scale * kLog2e;

  // Query tiles it0 .. ntq-1 of each of the G heads see keys of this workgroup; taken from the last tile down, the heads
  // of a tile one after the other, so that the key blocks of a (batch, kv head) — which share an XCD — walk in step and
  // find each other's tiles in the L2.
  const int ntq = (f.L + BT - 1) / BT;
  int it0 = 0;
  if (CAUSAL) it0 = (k0 - coff > 0 ? k0 - coff : 0) / BT;
  const int nt = ntq > it0 ? ntq - it0 : 0;
  const int total = f.G * nt;
  const bool walk_up = dkv_walks_up(a, CAUSAL);  // every second round of an XCD's workgroups (sdpa_common.h)
  auto tile_of = [&](int idx) __attribute__((always_inline)) { return walk_up ? it0 + idx / f.G : ntq - 1 - idx / f.G; };

  f32x4 qst[NLD], gst[NLD];
  float2 sst = make_float2(0.f, 0.f);
  int lrow[NLD], lcol[NLD], gcol[NLD];
  bool cval[NLD];  // PAD: as in the dq kernel
#pragma unroll
  for (int i = 0; i < NLD; i++) {
    const int cidx = tid + 256 * i;
    lrow[i] = cidx / (D / 4);
    lcol[i] = cidx % (D / 4);
    cval[i] = !PAD || 4 * lcol[i] < have;
    gcol[i] = cval[i] ? lcol[i] : 0;
  }
  auto load_tile = [&](int idx) {
    const int h = hk * f.G + idx % f.G;
    const int i0 = tile_of(idx) * BT;
    const float* qp = (const float*)f.q + b * f.qs[0] + h * f.qs[1];
    const float* gp = (const float*)a.dout + b * a.dos[0] + h * a.dos[1];
#pragma unroll
    for (int i = 0; i < NLD; i++) {
      int row = i0 + lrow[i];
      row = row < f.L ? row : f.L - 1;  // rows past the end re-read the last valid row (their weight is forced to 0)
      qst[i] = *(const f32x4*)(qp + row * f.qs[2] + 4 * gcol[i]);
      gst[i] = *(const f32x4*)(gp + row * a.dos[2] + 4 * gcol[i]);
    }
    if (tid < BT) {
      const int row = i0 + tid;
      sst = row < f.L ? *(const float2*)(a.stats + 2 * (((long long)b * f.Hq + h) * f.L + row)) : make_float2(1e30f, 0.f);
    }
  };
  auto store_tile = [&](int stage) {
    float* Qs = smem + stage * Lds::STAGE;
    float* Gs = Qs + Lds::TILE;
#pragma unroll
    for (int i = 0; i < NLD; i++)
#pragma unroll
      for (int e = 0; e < 4; e++) {
        Qs[lrow[i] * PITCH + 4 * lcol[i] + e] = cval[i] ? qst[i][e] : 0.f;
        Gs[lrow[i] * PITCH + 4 * lcol[i] + e] = cval[i] ? gst[i][e] : 0.f;
      }
    if (tid < BT) *(float2*)(Gs + Lds::TILE + 2 * tid) = sst;
  };
  const int s_lane = lq * PITCH + lh * (D / 2);
  const int g_lane = 4 * lh * PITCH + lq;

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
    const int i0 = tile_of(idx) * BT;
    const int h_of_tile = hk * f.G + idx % f.G;
    if (wave_live && (!CAUSAL || kw0 <= i0 + BT - 1 + coff)) {
      const float* Qs = smem + cur * Lds::STAGE;
      const float* Gs = Qs + Lds::TILE;
      const float* st = Gs + Lds::TILE;

      f32x16 s = score_product<D>(Qs + s_lane, kreg);   // S = Q . K^T
      f32x16 dp = score_product<D>(Gs + s_lane, vreg);  // dP = dout . V^T
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
              bias2 = ((const float*)f.mask)[at] * kLog2e;
            }
          }
          const float p = fast_exp2(fmaf(s[r], c, bias2 - lse2[e]));
          s[r] = p;
          dp[r] = p * (dp[r] - dl[e]);
        }
      }
      if (need_mask) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const int qrow = i0 + 8 * (r >> 2) + 4 * lh + (r & 3);
          if (key >= S || (CAUSAL && key > qrow + coff)) s[r] = 0.f, dp[r] = 0.f;
        }
      }
      // dv^T += dout^T . P, dk^T += Q^T . dS
      const float* gl = Gs + g_lane;
      const float* ql = Qs + g_lane;
#pragma unroll
      for (int t = 0; t < 16; t++)
#pragma unroll
        for (int db = 0; db < DBLK; db++) {
          const int at = (8 * (t >> 2) + (t & 3)) * PITCH + 32 * db;
          dvacc[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(gl[at], s[t], dvacc[db], 0, 0, 0);
          dkacc[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(ql[at], dp[t], dkacc[db], 0, 0, 0);
        }
    }
#pragma unroll
    for (int db = 0; db < DBLK; db++) pin_accumulator<(D > 64 || MASKED)>(dkacc[db]), pin_accumulator<(D > 64 || MASKED)>(dvacc[db]);
    __syncthreads();
  }

  if (key < f.S) {
#pragma unroll
    for (int db = 0; db < DBLK; db++)
#pragma unroll
      for (int rg = 0; rg < 4; rg++) {
        f32x4 x, y;
#pragma unroll
        for (int i = 0; i < 4; i++) x[i] = dkacc[db][4 * rg + i] * f.scale, y[i] = dvacc[db][4 * rg + i];
        if (PAD && 32 * db + 8 * rg + 4 * lh >= have) continue;
        *(f32x4*)(dkp + 32 * db + 8 * rg + 4 * lh) = x;
        *(f32x4*)(dvp + 32 * db + 8 * rg + 4 * lh) = y;
      }
  }
}

template <int D, bool CAUSAL, bool MASKED, bool PAD>
int launch_k(const BwdArgs& args, hipStream_t stream) {
  BwdArgs a = args;
  // the callers keep to this (the records of a split are laid out for D, rows are read in 16-byte chunks)
  if (PAD && (a.dkv_splits > 1 || a.dq_splits > 1 || a.f.D % 4 != 0 || a.f.D >= D || a.f.D < 4)) return (int)hipErrorInvalidValue;
  static hipError_t state1[kMaxDevices], state2[kMaxDevices];
  static bool done1[kMaxDevices], done2[kMaxDevices];
  hipError_t e = grant_dynamic_lds((const void*)backward_dq_f32_kernel<D, CAUSAL, MASKED, PAD>, BwdF32Lds<D>::BYTES, state1, done1);
  if (e != hipSuccess) return (int)e;
  e = grant_dynamic_lds((const void*)backward_dkv_f32_kernel<D, CAUSAL, MASKED, PAD>, BwdF32Lds<D>::BYTES, state2, done2);
  if (e != hipSuccess) return (int)e;
  const long long g1 = (long long)a.f.B * a.f.Hq * ((a.f.L + BM - 1) / BM) * a.dq_splits;
  const long long g2 = (long long)a.f.B * a.f.Hkv * ((a.f.S + BM - 1) / BM) * a.dkv_splits;
  static int round_cache[kMaxDevices];
  a.dkv_round = CAUSAL ? dkv_round_of((const void*)backward_dkv_f32_kernel<D, CAUSAL, MASKED, PAD>, 256, BwdF32Lds<D>::BYTES, round_cache) : 0;
  hipLaunchKernelGGL((backward_dq_f32_kernel<D, CAUSAL, MASKED, PAD>), dim3((unsigned)g1), dim3(256), BwdF32Lds<D>::BYTES, stream, a);
  e = hipGetLastError();
  if (e != hipSuccess) return (int)e;
  if (a.dq_splits > 1) {
    const int rc = launch_backward_dq_merge<float>(a, stream);
    if (rc != 0) return rc;
  }
  hipLaunchKernelGGL((backward_dkv_f32_kernel<D, CAUSAL, MASKED, PAD>), dim3((unsigned)g2), dim3(256), BwdF32Lds<D>::BYTES, stream, a);
  e = hipGetLastError();
  if (e != hipSuccess || a.dkv_splits == 1) return (int)e;
  return launch_backward_dkv_sum<float>(a, stream);
}

template <int D, bool PAD>
int launch_d(const BwdArgs& a, hipStream_t stream) {
  if (a.f.mask_kind != 0) return launch_k<D, false, true, PAD>(a, stream);  // exclusive with causal (validated by the caller, as the reference asserts)
  return a.f.causal ? launch_k<D, true, false, PAD>(a, stream) : launch_k<D, false, false, PAD>(a, stream);
}

}  // namespace

int launch_backward_f32(const BwdArgs& a, hipStream_t stream) {
  if (a.f.D == 128) return launch_d<128, false>(a, stream);
  if (a.f.D == 64) return launch_d<64, false>(a, stream);
  // any other multiple of 4 up to 128: the kernels of the next size up, the missing columns as zeros
  return a.f.D < 64 ? launch_d<64, true>(a, stream) : launch_d<128, true>(a, stream);
}

}  // namespace ttsdpa
