// Flash-attention forward for fp16 / bf16 on gfx950 matrix cores (prefill / training-shape attention).
//
// Replaces, in one kernel, the reference's device chain transpose -> batched GEMM -> scale -> causal bias ->
// softmax -> batched GEMM (reference src/Function/FuncNNLayer.h:237-265; device ops at
// src/Operation/OpLinalgCuda.cuh:239-293 and src/Operation/OpNNLayerCuda.cuh:36-145): the [L,S] score matrix
// never leaves registers.
//
// Tiling.  A workgroup of 4 wavefronts owns 128 query rows of one (batch, query head); each wavefront owns 32 of
// them.  Keys/values are consumed in tiles of 64, staged through LDS (K row-major, V transposed so that the key
// axis is contiguous), the next tile's global loads being in flight while the current one is computed.
//
// Per wavefront and KV tile, with v_mfma_f32_32x32x16 (A: 32 rows x 16, B: 16 x 32 cols, lane l supplies row/col
// l%32 and the 8 contraction elements of half l/32; C: lane l holds column l%32 and rows 8*(r/4) + 4*(l/32) + r%4):
//   S^T[64 keys x 32 queries] = K_tile . Q^T      A = K rows from LDS, B = Q rows held in registers
//   P^T = exp2((S^T - rowmax) * scale*log2e)      a query is one lane column: its keys sit in that lane's registers
//                                                 and in lane l^32, so a row reduction is one cross-lane step
//   O^T[D x 32 queries] += V_tile^T . P^T         A = V^T rows from LDS, B = P^T taken straight from the S^T
//                                                 accumulator registers (the contraction order is permuted
//                                                 identically on the V^T side, see vt_pos)
// Causal masking (key j visible to query i iff j <= i, reference src/Operation/OpTransformCpu.h:202-209) skips
// tiles above the diagonal and applies the predicate only on tiles that straddle it.
// Grouped-query attention: kv head = query head / (Hq/Hkv), resolved in the kernel; the workgroup order puts the
// query heads and row tiles that share a KV head on the same XCD so its L2 holds that K/V once.

#include "sdpa_common.h"

namespace ttsdpa {

namespace {

constexpr int BM = 128;  // query rows per workgroup
constexpr int BN = 64;   // keys per tile
constexpr int VT_PITCH = BN + 8;  // elements per V^T row in LDS (144 B: 16 consecutive rows hit distinct banks)

// Position of key kv (0..63) inside a V^T row: the 8 keys one lane feeds to one MFMA become contiguous.
// kv = 16*t + 8*a + 4*h + c  ->  16*t + 8*h + 4*a + c
__device__ __forceinline__ int vt_pos(int kv) { return (kv & ~15) | ((kv & 4) << 1) | ((kv & 8) >> 1) | (kv & 3); }

template <typename TR, int D, bool CAUSAL>
__global__ __launch_bounds__(256, 2) void prefill_kernel(KArgs a) {
  typedef typename TR::elem T;
  typedef typename TR::vec8 vec8;
  constexpr int K_PITCH = D + 8;     // elements per K row in LDS
  constexpr int KSTEPS = D / 16;     // MFMAs along head_dim for S^T
  constexpr int DBLK = D / 32;       // 32-row blocks of O^T
  constexpr int KLD = (BN * D / 8) / 256;  // 16-byte K chunks per thread per tile
  constexpr int VBLOCKS = (BN / 4) * (D / 8);  // 4-key x 8-dim blocks per tile
  constexpr int VLD = (VBLOCKS + 255) / 256;

  __shared__ __attribute__((aligned(16))) T Ks[BN * K_PITCH];
  __shared__ __attribute__((aligned(16))) T Vt[D * VT_PITCH];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int lq = lane & 31;   // query column / operand row of this lane
  const int lh = lane >> 5;   // which half of the contraction elements this lane supplies

  // ---- workgroup -> (batch, kv head, query head in group, row tile) -------------------------------------------
  const int ntile = (a.L + BM - 1) / BM;
  const int inner = a.G * ntile;           // workgroups that share one (batch, kv head)
  const int npair = a.B * a.Hkv;
  int pair, in;
  {
    int n = blockIdx.x;
    if ((npair & 7) == 0) {                // workgroup n runs on XCD n % 8: keep a pair on one XCD
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
  const T* kp = (const T*)a.k + b * a.ks[0] + hk * a.ks[1];
  const T* vp = (const T*)a.v + b * a.vs[0] + hk * a.vs[1];

  // ---- Q rows of this wavefront, kept in registers as MFMA B operands -----------------------------------------
  vec8 qreg[KSTEPS];
  {
    int row = qw0 + lq;
    row = row < a.L ? row : a.L - 1;
    const T* qr = qp + row * a.qs[2] + 8 * lh;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) qreg[ks] = *(const vec8*)(qr + 16 * ks);
  }

  f32x16 oacc[DBLK];
#pragma unroll
  for (int i = 0; i < DBLK; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) oacc[i][r] = 0.f;
  float m_run = -1e30f;  // running row maximum (raw scores), finite so that (m_run - m_new) never is inf - inf
  float l_run = 0.f;     // this lane's share of the running row sum
  const float c = a.scale * kLog2e;

  int ntiles_kv = (a.S + BN - 1) / BN;
  if (CAUSAL) {
    int last = q0 + BM - 1 < a.L - 1 ? q0 + BM - 1 : a.L - 1;  // last query row of the workgroup
    int lastkv = last < a.S - 1 ? last : a.S - 1;
    ntiles_kv = lastkv / BN + 1;
  }

  // ---- global -> register staging of one K/V tile ------------------------------------------------------------
  u32x4 kst[KLD];
  u32x4 vst[VLD][4];
  auto load_tile = [&](int kv0) {
#pragma unroll
    for (int i = 0; i < KLD; i++) {
      int cidx = tid + 256 * i;
      int r = cidx / (D / 8), cc = cidx % (D / 8);
      int key = kv0 + r;
      key = key < a.S ? key : a.S - 1;
      kst[i] = *(const u32x4*)(kp + key * a.ks[2] + 8 * cc);
    }
#pragma unroll
    for (int i = 0; i < VLD; i++) {
      int blk = tid + 256 * i;
      if (VBLOCKS % 256 == 0 || blk < VBLOCKS) {
        int kg = blk / (D / 8), dc = blk % (D / 8);
#pragma unroll
        for (int j = 0; j < 4; j++) {
          int key = kv0 + 4 * kg + j;
          key = key < a.S ? key : a.S - 1;
          vst[i][j] = *(const u32x4*)(vp + key * a.vs[2] + 8 * dc);
        }
      }
    }
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int i = 0; i < KLD; i++) {
      int cidx = tid + 256 * i;
      int r = cidx / (D / 8), cc = cidx % (D / 8);
      *(u32x4*)(Ks + r * K_PITCH + 8 * cc) = kst[i];
    }
#pragma unroll
    for (int i = 0; i < VLD; i++) {
      int blk = tid + 256 * i;
      if (VBLOCKS % 256 == 0 || blk < VBLOCKS) {
        int kg = blk / (D / 8), dc = blk % (D / 8);
        int pos = vt_pos(4 * kg);
#pragma unroll
        for (int w = 0; w < 4; w++) {
          // dims 8*dc + 2w (low halves) and 8*dc + 2w + 1 (high halves) of the four keys 4*kg .. 4*kg+3
          uint32_t r0 = vst[i][0][w], r1 = vst[i][1][w], r2 = vst[i][2][w], r3 = vst[i][3][w];
          u32x2 lo, hi;
          lo[0] = __builtin_amdgcn_perm(r1, r0, 0x05040100u);
          lo[1] = __builtin_amdgcn_perm(r3, r2, 0x05040100u);
          hi[0] = __builtin_amdgcn_perm(r1, r0, 0x07060302u);
          hi[1] = __builtin_amdgcn_perm(r3, r2, 0x07060302u);
          *(u32x2*)(Vt + (8 * dc + 2 * w) * VT_PITCH + pos) = lo;
          *(u32x2*)(Vt + (8 * dc + 2 * w + 1) * VT_PITCH + pos) = hi;
        }
      }
    }
  };

  load_tile(0);
  for (int jt = 0; jt < ntiles_kv; jt++) {
    const int kv0 = jt * BN;
    __syncthreads();  // every wavefront is done reading the previous tile
    store_tile();
    __syncthreads();
    if (jt + 1 < ntiles_kv) load_tile(kv0 + BN);

    if (CAUSAL && kv0 > qw0 + 31) continue;  // the whole tile is above this wavefront's diagonal

    // ---- S^T = K . Q^T ------------------------------------------------------------------------------------------
    f32x16 sacc[2];
#pragma unroll
    for (int blk = 0; blk < 2; blk++) {
#pragma unroll
      for (int r = 0; r < 16; r++) sacc[blk][r] = 0.f;
      const T* krow = Ks + (32 * blk + lq) * K_PITCH + 8 * lh;
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ks++) {
        vec8 ka = *(const vec8*)(krow + 16 * ks);
        sacc[blk] = TR::mfma32(ka, qreg[ks], sacc[blk]);
      }
    }

    // ---- mask the diagonal / ragged tile -------------------------------------------------------------------------
    const bool need_mask = (CAUSAL && kv0 + BN - 1 > qw0) || (kv0 + BN > a.S);
    if (need_mask) {
      const int qi = qw0 + lq;
#pragma unroll
      for (int blk = 0; blk < 2; blk++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          int key = kv0 + 32 * blk + 8 * (r >> 2) + 4 * lh + (r & 3);
          bool hidden = key >= a.S || (CAUSAL && key > qi);
          if (hidden) sacc[blk][r] = -INFINITY;
        }
    }

    // ---- online softmax --------------------------------------------------------------------------------------------
    float mloc = sacc[0][0];
#pragma unroll
    for (int blk = 0; blk < 2; blk++)
#pragma unroll
      for (int r = 0; r < 16; r++) mloc = fmaxf(mloc, sacc[blk][r]);
    mloc = fmaxf(mloc, __shfl_xor(mloc, 32));
    const float m_new = fmaxf(m_run, mloc);
    const float alpha = fast_exp2((m_run - m_new) * c);
    const float mc = m_new * c;
    m_run = m_new;
    float psum = 0.f;
#pragma unroll
    for (int blk = 0; blk < 2; blk++)
#pragma unroll
      for (int r = 0; r < 16; r++) {
        float p = fast_exp2(fmaf(sacc[blk][r], c, -mc));
        sacc[blk][r] = p;
        psum += p;
      }
    l_run = l_run * alpha + psum;
#pragma unroll
    for (int i = 0; i < DBLK; i++)
#pragma unroll
      for (int r = 0; r < 16; r++) oacc[i][r] *= alpha;

    // ---- P^T as B operands: MFMA t consumes accumulator registers 8*(t%2) .. +7 of block t/2 ------------------------
    vec8 pb[4];
#pragma unroll
    for (int t = 0; t < 4; t++) {
      f32x8 x;
#pragma unroll
      for (int i = 0; i < 8; i++) x[i] = sacc[t >> 1][8 * (t & 1) + i];
      pb[t] = __builtin_convertvector(x, vec8);
    }

    // ---- O^T += V^T . P^T ---------------------------------------------------------------------------------------------
#pragma unroll
    for (int db = 0; db < DBLK; db++) {
      const T* vrow = Vt + (32 * db + lq) * VT_PITCH + 8 * lh;
#pragma unroll
      for (int t = 0; t < 4; t++) {
        vec8 va = *(const vec8*)(vrow + 16 * t);
        oacc[db] = TR::mfma32(va, pb[t], oacc[db]);
      }
    }
  }

  // ---- normalise and store ----------------------------------------------------------------------------------------------
  float l_tot = l_run + __shfl_xor(l_run, 32);
  const float inv = 1.f / l_tot;
  const int qi = qw0 + lq;
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
        *(typename TR::vec4*)(op + 32 * db + 8 * rg + 4 * lh) = y;
      }
  }
}

template <typename TR, int D>
int launch_prefill_t(const KArgs& a, hipStream_t stream) {
  long long nwg = (long long)a.B * a.Hq * ((a.L + BM - 1) / BM);
  dim3 grid((unsigned)nwg), block(256);
  if (a.causal) {
    hipLaunchKernelGGL((prefill_kernel<TR, D, true>), grid, block, 0, stream, a);
  } else {
    hipLaunchKernelGGL((prefill_kernel<TR, D, false>), grid, block, 0, stream, a);
  }
  return (int)hipGetLastError();
}

}  // namespace

int launch_prefill(const KArgs& a, int dtype, hipStream_t stream) {
  if (dtype == 1) {
    return a.D == 128 ? launch_prefill_t<F16, 128>(a, stream) : launch_prefill_t<F16, 64>(a, stream);
  }
  return a.D == 128 ? launch_prefill_t<BF16, 128>(a, stream) : launch_prefill_t<BF16, 64>(a, stream);
}

}  // namespace ttsdpa
