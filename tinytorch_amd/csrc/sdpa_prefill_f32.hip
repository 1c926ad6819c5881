// Flash-attention forward for fp32 tensors on the gfx950 matrix cores (v_mfma_f32_32x32x2_f32, full fp32 products
// and sums): fp32 is the reference's default dtype, and its fp32 path is what the 1e-4 parity bar is stated against.
// Replaces the same device chain as the 16-bit kernels (reference src/Function/FuncNNLayer.h:237-265): the score
// matrix never leaves registers.  head_dim 64 or 128; attnMask and per-batch key counts are applied in the kernel.
//
// A workgroup of 4 wavefronts owns 128 query rows of one (batch, query head), 32 rows per wavefront; keys/values come
// in tiles of 32, staged global -> registers -> LDS, double-buffered.
// Per wavefront and tile, with v_mfma_f32_32x32x2 (A: 32 rows x 2, B: 2 x 32 cols, lane l supplies row/col l%32 and
// contraction element l/32; C: lane l holds column l%32 and rows 8*(r/4) + 4*(l/32) + r%4):
//   S^T[32 keys x 32 queries] = K . Q^T   MFMA ks contracts head_dim elements ks (lanes 0-31) and ks + D/2 (lanes 32-63),
//                                         so a lane's Q operands are one contiguous half of its query row (registers)
//                                         and K comes from LDS rows padded by one float (conflict-free columns);
//                                         two accumulators take alternate ks so the chain never waits on itself
//   P^T = exp2((S^T - m) * scale*log2e)   a query is one lane column; its other 16 keys sit in lane l^32
//   O^T[D x 32 queries] += V^T . P^T      MFMA t contracts the two keys that the lane halves hold in accumulator
//                                         register t, so P^T feeds the pipe straight from those registers and
//                                         V^T[d][key] is a plain row-major LDS read along d
// The running maximum is raised only when exceeded by 2^8 in the exponent.  Causal masking as in the 16-bit kernels
// (top-left aligned, reference src/Operation/OpTransformCpu.h:202-209): tiles above the diagonal are skipped.

#include "sdpa_common.h"

namespace ttsdpa {

namespace {

constexpr int BM = 128;  // query rows per workgroup
constexpr int BN = 32;   // keys per tile
constexpr float kLazyExp = 8.f;

template <int D>
struct F32Lds {
  static constexpr int K_PITCH = D + 1;   // floats; a column of 32 keys falls into 32 different banks
  static constexpr int V_PITCH = D + 32;  // floats; rows stay 16-byte aligned, the two lane halves use disjoint banks
  static constexpr int STAGE = BN * (K_PITCH + V_PITCH);
  static constexpr int BYTES = 2 * STAGE * 4;
};

// MASKED: an attnMask is applied (a variant of its own: the mask addressing costs registers the other variants keep).
// PAD: the tensors' head_dim a.D is a multiple of 4 below D; the 16-byte chunks of a row beyond it are taken as zeros (Q
// and K: nothing added to a score; V: output columns that are not stored).  The reference takes any head size
// (src/Function/FuncNNLayer.h:231-236).
template <int D, bool CAUSAL, bool MASKED, bool PAD>
__global__ __launch_bounds__(256, 2) void prefill_f32_kernel(KArgs a) {
  typedef F32Lds<D> Lds;
  constexpr int K_PITCH = Lds::K_PITCH, V_PITCH = Lds::V_PITCH;
  constexpr int KSTEPS = D / 2;   // MFMAs along head_dim for S^T
  constexpr int DBLK = D / 32;    // 32-row blocks of O^T
  constexpr int NLD = BN * D / 4 / 256;  // 16-byte chunks per thread per tile, for K and for V

  extern __shared__ __attribute__((aligned(16))) float smem_f32[];
  float* smem = smem_f32;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lq = lane & 31;
  const int lh = lane >> 5;

  // ---- workgroup -> (batch, kv head, query head in group, row tile); workgroup n runs on XCD n % 8 -------------
  const int ntile = (a.L + BM - 1) / BM;
  const int inner = a.G * ntile;
  const int npair = a.B * a.Hkv;
  int pair, in;
  const int nsplit = a.kv_splits > 1 ? a.kv_splits : 1;
  const int split = blockIdx.x % nsplit;  // key range of this workgroup (the only one unless the keys are split)
  {
    int n = blockIdx.x / nsplit;
    if ((npair & 7) == 0 && nsplit == 1) {
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

  const float* qp = (const float*)a.q + b * a.qs[0] + h * a.qs[1];
  const int* table = a.block_table ? a.block_table + (long long)b * a.bt_stride : nullptr;  // paged cache
  const float* kp = (const float*)a.k + (table ? 0 : b * a.ks[0]) + hk * a.ks[1];
  const float* vp = (const float*)a.v + (table ? 0 : b * a.vs[0]) + hk * a.vs[1];

  // ---- Q: this lane's half of its query row, the B operands of the S^T MFMAs ---------------------------------------
  float qreg[KSTEPS];
  {
    int row = qw0 + lq;
    row = row < a.L ? row : a.L - 1;
    const float* qr = qp + row * a.qs[2] + lh * (D / 2);
#pragma unroll
    for (int i = 0; i < KSTEPS / 4; i++) {
      f32x4 t = {0.f, 0.f, 0.f, 0.f};
      if (!PAD || lh * (D / 2) + 4 * i < a.D) t = *(const f32x4*)(qr + 4 * i);
#pragma unroll
      for (int e = 0; e < 4; e++) qreg[4 * i + e] = t[e];
    }
  }

  f32x16 oacc[DBLK];
#pragma unroll
  for (int i = 0; i < DBLK; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) oacc[i][r] = 0.f;
  const float c = a.scale * kLog2e;
  const float lazy = kLazyExp / c;
  float m_use = -1e30f;
  float mc = m_use * c;
  float l_run = 0.f;

  int S = a.S;  // keys of this batch entry: all of them, or the filled prefix of a cache / the unpadded length
  if (a.kv_len) {
    int len = __builtin_amdgcn_readfirstlane(a.kv_len[b]);
    S = len < 0 ? 0 : (len < S ? len : S);
  }
  if (S == 0 && nsplit == 1) {  // no keys: zeros, the reference's empty contraction
    const int qi = qw0 + lq;
    if (qi < a.L) {
      float* op = (float*)a.out + b * a.os[0] + h * a.os[1] + qi * a.os[2];
      for (int d = 4 * lh; d < (PAD ? a.D : D); d += 8) *(f32x4*)(op + d) = (f32x4){0.f, 0.f, 0.f, 0.f};
    }
    return;
  }
  int ntiles_kv = (S + BN - 1) / BN;
  const int coff = CAUSAL ? causal_offset(a, S) : 0;  // query position i sees keys up to i + coff
  // Query position of a row under the causal mask: the row itself, or with packed heads row % pack_L — then positions
  // are not monotone in the row, and the tile-level tests below use the range of all positions.
  const int pos_lo = a.pack_L ? 0 : qw0, pos_hi = a.pack_L ? a.pack_L - 1 : qw0 + 31;
  if (CAUSAL) {
    int last = (a.pack_L ? a.pack_L - 1 : (q0 + BM - 1 < a.L - 1 ? q0 + BM - 1 : a.L - 1)) + coff;
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
  const bool wave_live = qw0 < a.L;  // a wavefront without query rows only helps to stage the tiles

  // ---- global -> register -> LDS staging: thread t moves 16-byte chunks t, t+256, ... of a tile ----------------------
  f32x4 kst[NLD], vst[NLD];
  int lrow[NLD], lcol[NLD], gcol[NLD];
  bool cval[NLD];  // PAD: the chunk lies inside the tensors' rows; the others are loaded from the row's first chunk instead
                   // (the loads stay unconditional) and reach LDS as zeros
#pragma unroll
  for (int i = 0; i < NLD; i++) {
    int cidx = tid + 256 * i;
    lrow[i] = cidx / (D / 4);
    lcol[i] = cidx % (D / 4);
    cval[i] = !PAD || 4 * lcol[i] < a.D;
    gcol[i] = cval[i] ? lcol[i] : 0;
  }
  auto load_tile = [&](int kv0) {
    const float* ktile = kp + kv_tile_offset(a, table, kv0, a.ks[2], a.ks[0]);
    const float* vtile = vp + kv_tile_offset(a, table, kv0, a.vs[2], a.vs[0]);
#pragma unroll
    for (int i = 0; i < NLD; i++) {
      int row = lrow[i];
      row = kv0 + row < S ? row : S - 1 - kv0;  // rows past the end re-read the last valid row (masked later)
      kst[i] = *(const f32x4*)(ktile + row * a.ks[2] + 4 * gcol[i]);
      vst[i] = *(const f32x4*)(vtile + row * a.vs[2] + 4 * gcol[i]);
    }
  };
  auto store_tile = [&](int stage) {
    float* Ks = smem + stage * Lds::STAGE;
    float* Vs = Ks + BN * K_PITCH;
#pragma unroll
    for (int i = 0; i < NLD; i++) {
#pragma unroll
      for (int e = 0; e < 4; e++) Ks[lrow[i] * K_PITCH + 4 * lcol[i] + e] = cval[i] ? kst[i][e] : 0.f;  // rows are not 16-byte aligned
      *(f32x4*)(Vs + lrow[i] * V_PITCH + 4 * lcol[i]) = cval[i] ? vst[i] : (f32x4){0.f, 0.f, 0.f, 0.f};
    }
  };

  const int k_lane = lq * K_PITCH + lh * (D / 2);  // floats
  const int v_lane = 4 * lh * V_PITCH + lq;        // floats; + (8*(t/4) + t%4) * V_PITCH + 32*db

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

    if (wave_live && (!CAUSAL || kv0 <= pos_hi + coff)) {  // else: the whole tile is above this wavefront's diagonal
      const float* Ks = smem + cur * Lds::STAGE;
      const float* Vs = Ks + BN * K_PITCH;

      // ---- S^T = K . Q^T, two accumulators over alternate k-steps ----------------------------------------------------
      f32x16 s0, s1;
#pragma unroll
      for (int r = 0; r < 16; r++) s0[r] = 0.f, s1[r] = 0.f;
      const float* krow = Ks + k_lane;
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ks += 2) {
        s0 = __builtin_amdgcn_mfma_f32_32x32x2f32(krow[ks], qreg[ks], s0, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_32x32x2f32(krow[ks + 1], qreg[ks + 1], s1, 0, 0, 0);
      }
      f32x16 s;
#pragma unroll
      for (int r = 0; r < 16; r++) s[r] = s0[r] + s1[r];

      // ---- mask the diagonal / ragged tile -----------------------------------------------------------------------------
      if ((CAUSAL && kv0 + BN - 1 > pos_lo + coff) || (kv0 + BN > S)) {
        const int qi = (a.pack_L ? (qw0 + lq) % a.pack_L : qw0 + lq) + coff;
#pragma unroll
        for (int r = 0; r < 16; r++) {
          int key = kv0 + 8 * (r >> 2) + 4 * lh + (r & 3);
          bool hidden = key >= S || (CAUSAL && key > qi);
          if (hidden) s[r] = -INFINITY;
        }
      }
      if (MASKED) {
        int qi = qw0 + lq;
        qi = qi < a.L ? qi : a.L - 1;
        apply_attn_mask<float, true>(a, s, b * a.ms[0] + h * a.ms[1] + qi * a.ms[2], kv0, lh, S, 1.f / a.scale);
      }

      // ---- online softmax with a lazily raised maximum -----------------------------------------------------------------
      float mloc = s[0];
#pragma unroll
      for (int r = 1; r < 16; r++) mloc = fmaxf(mloc, s[r]);
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
          for (int r = 0; r < 16; r++) oacc[i][r] *= alpha;
      }
      float psum = 0.f;
#pragma unroll
      for (int r = 0; r < 16; r++) {
        s[r] = fast_exp2(fmaf(s[r], c, -mc));
        psum += s[r];
      }
      l_run += psum;

      // ---- O^T += V^T . P^T: MFMA t contracts the keys held in accumulator register t of the two lane halves -------------
      const float* vl = Vs + v_lane;
#pragma unroll
      for (int t = 0; t < 16; t++) {
#pragma unroll
        for (int db = 0; db < DBLK; db++) {
          float va = vl[(8 * (t >> 2) + (t & 3)) * V_PITCH + 32 * db];
          oacc[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(va, s[t], oacc[db], 0, 0, 0);
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
    float* op = (float*)a.out + b * a.os[0] + h * a.os[1] + qi * a.os[2];
#pragma unroll
    for (int db = 0; db < DBLK; db++)
#pragma unroll
      for (int rg = 0; rg < 4; rg++) {
        f32x4 x;
#pragma unroll
        for (int i = 0; i < 4; i++) x[i] = oacc[db][4 * rg + i] * inv;
        if (!PAD || 32 * db + 8 * rg + 4 * lh < a.D) *(f32x4*)(op + 32 * db + 8 * rg + 4 * lh) = x;
      }
  }
}

template <int D, bool CAUSAL, bool MASKED, bool PAD>
int launch_f32_k(const KArgs& a, dim3 grid, hipStream_t stream) {
  static hipError_t state[kMaxDevices];
  static bool done[kMaxDevices];
  const hipError_t granted = grant_dynamic_lds((const void*)prefill_f32_kernel<D, CAUSAL, MASKED, PAD>, F32Lds<D>::BYTES, state, done);
  if (granted != hipSuccess) return (int)granted;
  hipLaunchKernelGGL((prefill_f32_kernel<D, CAUSAL, MASKED, PAD>), grid, dim3(256), F32Lds<D>::BYTES, stream, a);
  return (int)hipGetLastError();
}

template <int D, bool PAD>
int launch_f32_d(const KArgs& a, dim3 grid, hipStream_t stream) {
  // the callers keep to this (the records of a split are laid out for D, rows are read in 16-byte chunks)
  if (PAD && (a.kv_splits > 1 || a.D % 4 != 0 || a.D >= D || a.D < 4)) return (int)hipErrorInvalidValue;
  if (a.mask_kind != 0) return launch_f32_k<D, false, true, PAD>(a, grid, stream);  // exclusive with causal (validated by the caller, as the reference asserts)
  return a.causal ? launch_f32_k<D, true, false, PAD>(a, grid, stream) : launch_f32_k<D, false, false, PAD>(a, grid, stream);
}

}  // namespace

int launch_prefill_f32(const KArgs& a, hipStream_t stream) {
  long long nwg = (long long)a.B * a.Hq * ((a.L + BM - 1) / BM) * (a.kv_splits > 1 ? a.kv_splits : 1);
  dim3 grid((unsigned)nwg);
  if (a.D == 128) return launch_f32_d<128, false>(a, grid, stream);
  if (a.D == 64) return launch_f32_d<64, false>(a, grid, stream);
  // any other multiple of 4 up to 128: the kernel of the next size up, the missing columns as zeros
  return a.D < 64 ? launch_f32_d<64, true>(a, grid, stream) : launch_f32_d<128, true>(a, grid, stream);
}

}  // namespace ttsdpa
