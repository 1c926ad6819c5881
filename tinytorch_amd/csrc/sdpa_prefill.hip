// Flash-attention forward for fp16 / bf16 on gfx950 matrix cores (prefill / training-shape attention).
//
// Replaces, in one kernel, the reference's device chain transpose -> batched GEMM -> scale -> causal bias ->
// softmax -> batched GEMM (reference src/Function/FuncNNLayer.h:237-265; device ops at
// src/Operation/OpLinalgCuda.cuh:239-293 and src/Operation/OpNNLayerCuda.cuh:36-145): the [L,S] score matrix
// never leaves registers.
//
// Tiling.  A workgroup of 4 wavefronts owns 128 query rows of one (batch, query head); each wavefront owns 32 of
// them.  Keys/values are consumed in tiles of 64 rows, staged row-major through a double-buffered LDS ring (one
// barrier per tile); the global loads of tile j+2 are in flight while tile j is computed.
//
// Per wavefront and KV tile, with v_mfma_f32_32x32x16 (A: 32 rows x 16, B: 16 x 32 cols, lane l supplies row/col
// l%32 and the 8 contraction elements of half l/32; C: lane l holds column l%32 and rows 8*(r/4) + 4*(l/32) + r%4):
//   S^T[64 keys x 32 queries] = K_tile . Q^T      A = K rows from LDS (ds_read_b128), B = Q rows held in registers
//   P^T = exp2((S^T - m) * scale*log2e)           a query is one lane column: its keys sit in that lane's registers
//                                                 and in lane l^32, so a row reduction is one cross-lane step
//   O^T[D x 32 queries] += V_tile^T . P^T         A = V^T, read from the row-major V tile with the LDS transpose
//                                                 load ds_read_b64_tr_b16; B = P^T taken straight from the S^T
//                                                 accumulator registers (the V side applies the same permutation
//                                                 of the contraction index, see v_operand)
// The maximum m the exponentials are taken against is raised lazily: a lane's 32 probabilities of a tile are summed
// anyway, and only when such a sum leaves [0, 1024] (which includes the first tile of a row, taken against -1e30) is
// the true row maximum formed, sum and accumulator rescaled and the tile's exponentials redone.  No per-tile row
// maximum: at small head sizes the vector ALUs, not the matrix pipe, bound this kernel (a score costs the same vector
// work whatever head_dim is).
// Causal masking (key j visible to query i iff j <= i, reference src/Operation/OpTransformCpu.h:202-209) skips
// tiles above the diagonal and applies the predicate only on tiles that straddle it.
// Grouped-query attention: kv head = query head / (Hq/Hkv), resolved in the kernel; the workgroup order puts the
// query heads and row tiles that share a KV head on the same XCD so its L2 holds that K/V once.

#include "sdpa_common.h"

namespace ttsdpa {

namespace {

constexpr int BM = 128;  // query rows per workgroup
constexpr int BN = 64;   // keys per tile
constexpr float kSumLimit = 1024.f;  // a lane's 32 probabilities of a tile may sum to this much before the maximum is raised

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));

template <int D>
struct PrefillLds {
  static constexpr int K_PITCH = D + 8;   // elements; rows 16 B apart in bank space: 32 rows x b128 conflict-free
  static constexpr int V_PITCH = D + 32;  // elements; rows 64 B apart in bank space: 4 rows x 64 B conflict-free
  static constexpr int STAGE = BN * (K_PITCH + V_PITCH);  // elements per stage
  static constexpr int BYTES = 2 * STAGE * 2;
};

// One MFMA A operand of V^T from a row-major V tile: lane l (column d = d0 + l%32, half h = l/32) receives the
// 8 keys kvbase + {4h + 0..3, 8 + 4h + 0..3}.  ds_read_b64_tr_b16 works on groups of 16 lanes: lane s of a group
// supplies the address of 4 consecutive elements, and receives element s%4 of the segments of lanes s/4, 4 + s/4,
// 8 + s/4, 12 + s/4.  With lane s pointing at V[k0 + s/4][c0 + 4*(s%4) ..], lane s ends up with V[k0 + 0..3][c0 + s].
template <typename vec8>
__device__ __forceinline__ vec8 v_operand(const void* lane_base, int byte_off_lo, int byte_off_hi) {
  typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
  s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)((const char*)lane_base + byte_off_lo));
  s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)((const char*)lane_base + byte_off_hi));
  s16x8 r = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(vec8, r);
}

// MASKED: an attnMask is applied (a variant of its own: the mask addressing costs registers the other variants keep).
// PAD: the tensors' head_dim a.D is a multiple of 8 below D.  The 16-byte chunks of a row beyond a.D are taken as zeros
// (Q and K: they add nothing to a score; V: columns of the output that are not stored), everything else is the
// kernel for head_dim D.  The reference takes any head size (src/Function/FuncNNLayer.h:231-236).
template <typename TR, int D, bool CAUSAL, bool MASKED, bool PAD>
__global__ __launch_bounds__(256, (D > 128 ? 1 : 2)) void prefill_kernel(KArgs a) {
  typedef typename TR::elem T;
  typedef typename TR::vec8 vec8;
  typedef PrefillLds<D> Lds;
  constexpr int K_PITCH = Lds::K_PITCH, V_PITCH = Lds::V_PITCH;
  constexpr int KSTEPS = D / 16;           // MFMAs along head_dim for S^T
  constexpr int DBLK = D / 32;             // 32-row blocks of O^T
  constexpr int NLD = (BN * D / 8) / 256;  // 16-byte chunks per thread per tile, for K and for V

  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  T* smem = (T*)smem_raw;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: branches on it are scalar
  const int lq = lane & 31;   // query column / operand row of this lane
  const int lh = lane >> 5;   // which half of the contraction elements this lane supplies

  // ---- workgroup -> (batch, kv head, query head in group, row tile) -------------------------------------------
  const int ntile = (a.L + BM - 1) / BM;
  const int inner = a.G * ntile;           // workgroups that share one (batch, kv head)
  const int npair = a.B * a.Hkv;
  int pair, in;
  const int nsplit = a.kv_splits > 1 ? a.kv_splits : 1;
  const int split = blockIdx.x % nsplit;    // key range of this workgroup (the only one unless the keys are split)
  {
    int n = blockIdx.x / nsplit;
    if ((npair & 7) == 0 && nsplit == 1) {  // workgroup n runs on XCD n % 8: keep a pair on one XCD
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
  const int rt = CAUSAL ? ntile - 1 - in / a.G : in / a.G;  // longest rows first
  const int h = hk * a.G + g;
  const int q0 = rt * BM;
  const int qw0 = q0 + wave * 32;

  const T* qp = (const T*)a.q + b * a.qs[0] + h * a.qs[1];
  const int* table = a.block_table ? a.block_table + (long long)b * a.bt_stride : nullptr;  // paged cache
  const T* kp = (const T*)a.k + (table ? 0 : b * a.ks[0]) + hk * a.ks[1];
  const T* vp = (const T*)a.v + (table ? 0 : b * a.vs[0]) + hk * a.vs[1];

  // ---- Q rows of this wavefront, kept in registers as MFMA B operands -----------------------------------------
  vec8 qreg[KSTEPS];
  {
    int row = qw0 + lq;
    row = row < a.L ? row : a.L - 1;
    const T* qr = qp + row * a.qs[2] + 8 * lh;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) {
      if (!PAD || 16 * ks + 8 * lh < a.D) {
        qreg[ks] = *(const vec8*)(qr + 16 * ks);
      } else {
#pragma unroll
        for (int i = 0; i < 8; i++) qreg[ks][i] = (T)0.f;
      }
    }
  }

  f32x16 oacc[DBLK];
#pragma unroll
  for (int i = 0; i < DBLK; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) oacc[i][r] = 0.f;
  const float c = a.scale * kLog2e;
  float m_use = -1e30f;  // maximum the exponentials are taken against (raw scores); finite: no inf - inf
  float mc = m_use * c;
  float l_run = 0.f;     // this lane's share of the running row sum

  int S = a.S;  // keys of this batch entry: all of them, or the filled prefix of a cache / the unpadded length
  if (a.kv_len) {
    int len = __builtin_amdgcn_readfirstlane(a.kv_len[b]);
    S = len < 0 ? 0 : (len < S ? len : S);
  }
  if (S == 0 && nsplit == 1) {  // no keys: zeros, the reference's empty contraction
    const int qi = qw0 + lq;
    if (qi < a.L) {
      T* op = (T*)a.out + b * a.os[0] + h * a.os[1] + qi * a.os[2];
      typename TR::vec4 zero;
#pragma unroll
      for (int i = 0; i < 4; i++) zero[i] = (T)0.f;
      for (int d = 4 * lh; d < (PAD ? a.D : D); d += 8) *(typename TR::vec4*)(op + d) = zero;
    }
    return;
  }
  int ntiles_kv = (S + BN - 1) / BN;
  const int coff = CAUSAL ? causal_offset(a, S) : 0;  // query position i sees keys up to i + coff
  // Query position of a row under the causal mask: the row itself, or with packed heads row % pack_L — then positions
  // are not monotone in the row, and the tile-level tests below use the range of all positions.
  const int pos_lo = a.pack_L ? 0 : qw0, pos_hi = a.pack_L ? a.pack_L - 1 : qw0 + 31;
  if (CAUSAL) {
    int last = (a.pack_L ? a.pack_L - 1 : (q0 + BM - 1 < a.L - 1 ? q0 + BM - 1 : a.L - 1)) + coff;  // last key any row of the workgroup sees
    int lastkv = last < S - 1 ? last : S - 1;
    ntiles_kv = S > 0 ? lastkv / BN + 1 : 0;
  }
  // tiles jt0 .. jt1-1 are this workgroup's: all of them, or those of its split (kv_chunk is a multiple of the tile)
  int jt0 = 0, jt1 = ntiles_kv;
  if (nsplit > 1) {
    jt0 = split * (a.kv_chunk / BN);
    const int end = jt0 + a.kv_chunk / BN;
    jt1 = end < jt1 ? end : jt1;
  }

  // ---- global -> register -> LDS staging of one K/V tile --------------------------------------------------------
  // thread t moves chunks t, t+256, ...: chunk c is row c / (D/8), 16-byte column c % (D/8)
  u32x4 kst[NLD], vst[NLD];
  unsigned koff[NLD], voff[NLD];  // byte offsets of this thread's chunks inside a full tile
  int lrow[NLD], lcol[NLD], gcol[NLD];
  bool cval[NLD];                 // PAD: the chunk lies inside the tensors' rows; the others are loaded from the row's
                                  // first chunk instead (the loads stay unconditional) and reach LDS as zeros
#pragma unroll
  for (int i = 0; i < NLD; i++) {
    int cidx = tid + 256 * i;
    lrow[i] = cidx / (D / 8);
    lcol[i] = cidx % (D / 8);
    cval[i] = !PAD || 8 * lcol[i] < a.D;
    gcol[i] = cval[i] ? lcol[i] : 0;
    koff[i] = (unsigned)(lrow[i] * a.ks[2] + 8 * gcol[i]) * 2u;
    voff[i] = (unsigned)(lrow[i] * a.vs[2] + 8 * gcol[i]) * 2u;
  }
  auto load_tile = [&](int kv0) {
    const T* ktile = kp + kv_tile_offset(a, table, kv0, a.ks[2], a.ks[0]);
    const T* vtile = vp + kv_tile_offset(a, table, kv0, a.vs[2], a.vs[0]);
    const char* kt = (const char*)ktile;
    const char* vt = (const char*)vtile;
    if (kv0 + BN <= S) {
#pragma unroll
      for (int i = 0; i < NLD; i++) {
        kst[i] = *(const u32x4*)(kt + koff[i]);
        vst[i] = *(const u32x4*)(vt + voff[i]);
      }
    } else {  // ragged last tile: rows past the end re-read the last valid row (masked later)
#pragma unroll
      for (int i = 0; i < NLD; i++) {
        int row = lrow[i];
        row = kv0 + row < S ? row : S - 1 - kv0;
        kst[i] = *(const u32x4*)(ktile + row * a.ks[2] + 8 * gcol[i]);
        vst[i] = *(const u32x4*)(vtile + row * a.vs[2] + 8 * gcol[i]);
      }
    }
  };
  auto store_tile = [&](int stage) {
    T* Ks = smem + stage * Lds::STAGE;
    T* Vs = Ks + BN * K_PITCH;
#pragma unroll
    for (int i = 0; i < NLD; i++) {
      const u32x4 zero = {0u, 0u, 0u, 0u};
      *(u32x4*)(Ks + lrow[i] * K_PITCH + 8 * lcol[i]) = cval[i] ? kst[i] : zero;
      *(u32x4*)(Vs + lrow[i] * V_PITCH + 8 * lcol[i]) = cval[i] ? vst[i] : zero;
    }
  };

  // lane-invariant part of the LDS operand addresses
  const int k_lane = lq * K_PITCH + 8 * lh;                                              // elements
  const int v_lane = (4 * lh + ((lane & 15) >> 2)) * V_PITCH + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);  // elements

  if (jt0 < jt1) {
    load_tile(jt0 * BN);
    store_tile(0);
    if (jt0 + 1 < jt1) load_tile((jt0 + 1) * BN);
  }
  __syncthreads();

  for (int jt = jt0; jt < jt1; jt++) {
    const int kv0 = jt * BN;
    const int cur = (jt - jt0) & 1;
    if (jt + 1 < jt1) {
      store_tile(cur ^ 1);  // stage cur^1 was last read before the barrier that ended the previous iteration
      if (jt + 2 < jt1) load_tile(kv0 + 2 * BN);
    }

    if (qw0 < a.L && (!CAUSAL || kv0 <= pos_hi + coff)) {  // else: no rows here, or the whole tile is above the diagonal
      const T* Ks = smem + cur * Lds::STAGE;
      const T* Vs = Ks + BN * K_PITCH;

      // ---- S^T = K . Q^T ----------------------------------------------------------------------------------------
      f32x16 sacc[2];
#pragma unroll
      for (int blk = 0; blk < 2; blk++) {
#pragma unroll
        for (int r = 0; r < 16; r++) sacc[blk][r] = 0.f;
        const T* krow = Ks + k_lane + 32 * blk * K_PITCH;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ks++) {
          vec8 ka = *(const vec8*)(krow + 16 * ks);
          sacc[blk] = TR::mfma32(ka, qreg[ks], sacc[blk]);
        }
      }

      // ---- mask the diagonal / ragged tile -----------------------------------------------------------------------
      const bool need_mask = (CAUSAL && kv0 + BN - 1 > pos_lo + coff) || (kv0 + BN > S);
      if (need_mask) {
        const int qi = (a.pack_L ? (qw0 + lq) % a.pack_L : qw0 + lq) + coff;
#pragma unroll
        for (int blk = 0; blk < 2; blk++)
#pragma unroll
          for (int r = 0; r < 16; r++) {
            int key = kv0 + 32 * blk + 8 * (r >> 2) + 4 * lh + (r & 3);
            bool hidden = key >= S || (CAUSAL && key > qi);
            if (hidden) sacc[blk][r] = -INFINITY;
          }
      }
      if (MASKED) {
        int qi = qw0 + lq;
        qi = qi < a.L ? qi : a.L - 1;
        const long long mrow = b * a.ms[0] + h * a.ms[1] + qi * a.ms[2];
#pragma unroll
        for (int blk = 0; blk < 2; blk++) apply_attn_mask<T, true>(a, sacc[blk], mrow, kv0 + 32 * blk, lh, S, 1.f / a.scale);
      }

      // ---- online softmax with a lazily raised maximum ---------------------------------------------------------------
      float psum = 0.f;
      f32x16 pr[2];
#pragma unroll
      for (int blk = 0; blk < 2; blk++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          pr[blk][r] = fast_exp2(fmaf(sacc[blk][r], c, -mc));
          psum += pr[blk][r];
        }
      if (__builtin_expect(__builtin_amdgcn_ballot_w64(!(psum <= kSumLimit)) != 0, 0)) {  // some row of the wavefront outgrew its maximum
        float mloc = sacc[0][0];
#pragma unroll
        for (int blk = 0; blk < 2; blk++)
#pragma unroll
          for (int r = 0; r < 16; r++) mloc = fmaxf(mloc, sacc[blk][r]);
        mloc = fmaxf(mloc, __shfl_xor(mloc, 32));
        const float m_new = fmaxf(m_use, mloc);
        const float alpha = fast_exp2((m_use - m_new) * c);
        m_use = m_new;
        mc = m_new * c;
        l_run *= alpha;
#pragma unroll
        for (int i = 0; i < DBLK; i++)
#pragma unroll
          for (int r = 0; r < 16; r++) oacc[i][r] *= alpha;
        psum = 0.f;
#pragma unroll
        for (int blk = 0; blk < 2; blk++)
#pragma unroll
          for (int r = 0; r < 16; r++) {
            pr[blk][r] = fast_exp2(fmaf(sacc[blk][r], c, -mc));
            psum += pr[blk][r];
          }
      }
      l_run += psum;

      // ---- P^T as B operands: MFMA t consumes accumulator registers 8*(t%2) .. +7 of block t/2 ------------------------
      vec8 pb[4];
#pragma unroll
      for (int t = 0; t < 4; t++) {
        f32x8 x;
#pragma unroll
        for (int i = 0; i < 8; i++) x[i] = pr[t >> 1][8 * (t & 1) + i];
        pb[t] = __builtin_convertvector(x, vec8);
      }

      // ---- O^T += V^T . P^T ---------------------------------------------------------------------------------------------
      const T* vl = Vs + v_lane;
#pragma unroll
      for (int db = 0; db < DBLK; db++) {
#pragma unroll
        for (int t = 0; t < 4; t++) {
          vec8 va = v_operand<vec8>(vl, ((16 * t) * V_PITCH + 32 * db) * 2, ((16 * t + 8) * V_PITCH + 32 * db) * 2);
          oacc[db] = TR::mfma32(va, pb[t], oacc[db]);
        }
      }
    }
    __syncthreads();
  }

  // ---- normalise and store ----------------------------------------------------------------------------------------------
  float l_tot = l_run + __shfl_xor(l_run, 32);
  const int qi = qw0 + lq;
  if (nsplit > 1) {  // a partial result: unnormalised accumulator, the maximum it is relative to, the sum
    if (qi < a.L) {
      float* rec = a.ws + ((long long)(pair * nsplit + split) * a.L + qi) * (D + 2);  // 8-byte aligned
#pragma unroll
      for (int db = 0; db < DBLK; db++)
#pragma unroll
        for (int rg = 0; rg < 4; rg++) {
          float* dst = rec + 32 * db + 8 * rg + 4 * lh;
          *(float2*)dst = make_float2(oacc[db][4 * rg], oacc[db][4 * rg + 1]);
          *(float2*)(dst + 2) = make_float2(oacc[db][4 * rg + 2], oacc[db][4 * rg + 3]);
        }
      if (lh == 0) rec[D] = m_use, rec[D + 1] = l_tot;
    }
    return;
  }
  const float inv = 1.f / l_tot;
  if (qi < a.L) {
    T* op = (T*)a.out + b * a.os[0] + h * a.os[1] + qi * a.os[2];
#pragma unroll
    for (int db = 0; db < DBLK; db++)
#pragma unroll
      for (int rg = 0; rg < 4; rg++) {
        f32x4 x;
#pragma unroll
        for (int i = 0; i < 4; i++) x[i] = oacc[db][4 * rg + i] * inv;
        typename TR::vec4 y = __builtin_convertvector(x, typename TR::vec4);
        if (!PAD || 32 * db + 8 * rg + 4 * lh < a.D) *(typename TR::vec4*)(op + 32 * db + 8 * rg + 4 * lh) = y;
      }
  }
}

template <typename TR, int D, bool CAUSAL, bool MASKED, bool PAD>
int launch_prefill_k(const KArgs& a, dim3 grid, hipStream_t stream) {
  static hipError_t state[kMaxDevices];
  static bool done[kMaxDevices];
  const hipError_t granted = grant_dynamic_lds((const void*)prefill_kernel<TR, D, CAUSAL, MASKED, PAD>, PrefillLds<D>::BYTES, state, done);
  if (granted != hipSuccess) return (int)granted;
  hipLaunchKernelGGL((prefill_kernel<TR, D, CAUSAL, MASKED, PAD>), grid, dim3(256), PrefillLds<D>::BYTES, stream, a);
  return (int)hipGetLastError();
}

template <typename TR, int D, bool PAD>
int launch_prefill_t(const KArgs& a, hipStream_t stream) {
  // the callers keep to this (the records of a split are laid out for D, rows are read in 16-byte chunks)
  if (PAD && (a.kv_splits > 1 || a.D % 8 != 0 || a.D >= D || a.D < 8)) return (int)hipErrorInvalidValue;
  long long nwg = (long long)a.B * a.Hq * ((a.L + BM - 1) / BM) * (a.kv_splits > 1 ? a.kv_splits : 1);
  dim3 grid((unsigned)nwg);
  if (a.mask_kind != 0) return launch_prefill_k<TR, D, false, true, PAD>(a, grid, stream);  // exclusive with causal (validated)
  return a.causal ? launch_prefill_k<TR, D, true, false, PAD>(a, grid, stream) : launch_prefill_k<TR, D, false, false, PAD>(a, grid, stream);
}

}  // namespace

template <typename TR>
int launch_prefill_d(const KArgs& a, hipStream_t stream) {
  switch (a.D) {
    case 32: return launch_prefill_t<TR, 32, false>(a, stream);
    case 64: return launch_prefill_t<TR, 64, false>(a, stream);
    case 96: return launch_prefill_t<TR, 96, false>(a, stream);
    case 128: return launch_prefill_t<TR, 128, false>(a, stream);
    case 192: return launch_prefill_t<TR, 192, false>(a, stream);
    case 256: return launch_prefill_t<TR, 256, false>(a, stream);
    default: break;
  }
  // any other multiple of 8 up to 256: the kernel of the next size up, the missing columns as zeros
  if (a.D < 32) return launch_prefill_t<TR, 32, true>(a, stream);
  if (a.D < 64) return launch_prefill_t<TR, 64, true>(a, stream);
  if (a.D < 96) return launch_prefill_t<TR, 96, true>(a, stream);
  if (a.D < 128) return launch_prefill_t<TR, 128, true>(a, stream);
  if (a.D < 192) return launch_prefill_t<TR, 192, true>(a, stream);
  return launch_prefill_t<TR, 256, true>(a, stream);
}

int launch_prefill(const KArgs& a, int dtype, hipStream_t stream) {
  return dtype == 1 ? launch_prefill_d<F16>(a, stream) : launch_prefill_d<BF16>(a, stream);
}

}  // namespace ttsdpa
