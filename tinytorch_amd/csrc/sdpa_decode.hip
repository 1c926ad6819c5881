// Split-KV attention for decode: a few query rows per KV head against a long, contiguous KV cache (fp16 / bf16,
// head_dim 128 or 64).  Memory-bound: every K and V byte is read exactly once with 16-byte loads, whatever the number of
// query heads sharing the KV head, instead of the reference's GEMM -> scale -> softmax -> GEMM chain over a
// materialised score tensor (reference src/Function/FuncNNLayer.h:237-265).
//
// Work split.  Grid = splits x Hkv x B workgroups of 4 wavefronts.  A split is a contiguous range of keys; its
// wavefronts take 32-key blocks round-robin.  All query rows that read this KV head — the L * (Hq/Hkv) rows
// (l, g), at most 16 — are handled together, so the cache is streamed once for the whole group.
//
// Per 32-key block and wavefront:
//   scores  v_mfma_f32_16x16x32: A = the query rows (16 x 32 slice of head_dim, zero rows where unused), B = K^T taken
//           straight from global memory: lane l supplies key l%16 and the 8 head_dim elements of group l/16, i.e. one
//           16-byte load; head_dim/32 MFMAs cover the head.  Query row x sits at MFMA row 4*(x%4) + x/4, so the
//           result lane (key l%16, group l/16) holds rows l/16, l/16+4, ... in registers 0, 1, ...
//   softmax running max per row (reduced over the 16 key lanes with DPP row rotations), exp2 with scale*log2e folded
//   P.V     on the vector ALUs: with C = head_dim/8 chunks per row, lane l owns head_dim elements 8*(l%C) .. +7 of keys
//           l/C, l/C + 64/C, ... (one 16-byte load per key, a wavefront load instruction covers 64/C whole V rows =
//           1 KiB contiguous); the probabilities
//           travel from the score lanes to the value lanes through a per-wavefront LDS patch.
// Each wavefront ends with (max, sum, acc) per row; the workgroup merges its four, then either writes the final
// output (splits == 1) or a partial (max, sum, acc) record that merge_kernel combines by log-sum-exp.

#include "sdpa_common.h"

namespace ttsdpa {

namespace {

constexpr int KB = 32;       // keys per wavefront block
constexpr int NWAVE = 4;

// max over the 16 lanes of a DPP row (lanes 16*i .. 16*i+15), result in every lane of the row
__device__ __forceinline__ float row16_max(float x) {
  x = fmaxf(x, __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, x), 0x128, 0xf, 0xf, false)));  // row_ror:8
  x = fmaxf(x, __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, x), 0x124, 0xf, 0xf, false)));  // row_ror:4
  x = fmaxf(x, __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, x), 0x122, 0xf, 0xf, false)));  // row_ror:2
  x = fmaxf(x, __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, x), 0x121, 0xf, 0xf, false)));  // row_ror:1
  return x;
}
__device__ __forceinline__ float row16_sum(float x) {
  x += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, x), 0x128, 0xf, 0xf, false));
  x += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, x), 0x124, 0xf, 0xf, false));
  x += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, x), 0x122, 0xf, 0xf, false));
  x += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, x), 0x121, 0xf, 0xf, false));
  return x;
}

// Make this wavefront's LDS writes visible to its own later reads and keep the compiler from reordering across.
__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// R = registers of query rows per score lane: rows handled = up to 4*R.
// PAGED: K/V are page pools addressed through a block table (a variant of its own, so that the contiguous kernel
// carries none of the lookups).
// PAD: the tensors' head_dim a.D is a multiple of 8 below DD.  The 16-byte chunks of a row beyond it read as zeros (q, k)
// or are left out of the output (v: the lanes of those chunks fetch the row's first chunk instead, so that the loads stay
// unconditional); the split records keep the pitch DD + 2.
template <typename TR, int R, int DD, bool PAGED, bool PAD>
__global__ __launch_bounds__(256, 2) void decode_kernel(KArgs a, int splits, int chunk, float* __restrict__ ws) {
  typedef typename TR::elem T;
  typedef typename TR::vec8 vec8;
  constexpr int NR = 4 * R;    // row slots
  constexpr int KS = DD / 32;  // MFMAs along head_dim per 16 keys
  constexpr int CH = DD / 8;   // 16-byte chunks of a V row = value lanes per key
  constexpr int PH = 64 / CH;  // keys a wavefront V load covers (key phases)

  // per-wavefront patch: probabilities [KB keys][NR rows] + rescale factors [NR]; reused for the final merge
  __shared__ __attribute__((aligned(16))) float Pl[NWAVE][KB * NR + NR];
  __shared__ __attribute__((aligned(16))) float Om[NWAVE][NR][DD + 2];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;  // (forcing it scalar measured slower, also for the page lookups)
  const int l16 = lane & 15;  // score lanes: key within a 16-key group
  const int lg = lane >> 4;   // score lanes: row group
  const int vc = lane % CH;   // value lanes: 16-byte chunk of the row
  const int vph = lane / CH;  // value lanes: key phase

  int n = blockIdx.x;
  const int split = n % splits;
  n /= splits;
  const int hk = n % a.Hkv;
  const int b = n / a.Hkv;
  const int rows = a.L * a.G;  // query rows sharing this KV head, row x = (l, g) = (x / G, x % G)
  int S = a.S;                 // keys of this batch entry: the whole cache, or its filled prefix
  if (a.kv_len) {
    int len = a.kv_len[b];
    S = len < 0 ? 0 : (len < S ? len : S);
  }

  const T* kp = (const T*)a.k + b * a.ks[0] + hk * a.ks[1];
  const T* vp = (const T*)a.v + b * a.vs[0] + hk * a.vs[1];

  // ---- query rows as MFMA A operands: lane l supplies MFMA row l%16, head_dim 32*ks + 8*(l/16) .. +7 --------------
  vec8 qa[KS];
  {
    int mrow = l16;                       // MFMA row
    int x = (mrow & 3) * 4 + (mrow >> 2); // query row stored there: row x sits at 4*(x%4) + x/4
    bool used = (mrow & 3) < R && x < rows;
    int xl = used ? x / a.G : 0, xg = used ? x % a.G : 0;
    const T* qr = (const T*)a.q + b * a.qs[0] + (hk * a.G + xg) * a.qs[1] + xl * a.qs[2] + 8 * lg;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      const bool there = used && (!PAD || 32 * ks + 8 * lg < a.D);
      vec8 t = *(const vec8*)(there ? qr + 32 * ks : qr - 8 * lg);
#pragma unroll
      for (int i = 0; i < 8; i++) qa[ks][i] = there ? t[i] : (T)0.f;
    }
  }

  // lane-local state: score lanes track rows lg + 4r; value lanes accumulate all rows for their 8 dims
  float m_run[R], l_run[R];
#pragma unroll
  for (int r = 0; r < R; r++) m_run[r] = -1e30f, l_run[r] = 0.f;
  float acc[NR][8];
#pragma unroll
  for (int x = 0; x < NR; x++)
#pragma unroll
    for (int i = 0; i < 8; i++) acc[x][i] = 0.f;
  const float c = a.scale * kLog2e;

  const int s_begin = split * chunk;
  const int s_end = s_begin + chunk < S ? s_begin + chunk : S;
  float* pl = Pl[wave];
  // First hidden key per row of this score lane: the end of the split, or under a (bottom-right aligned) causal mask
  // the key after the row's own position S - L + l.
  int klim[R], klim_min = s_end;
#pragma unroll
  for (int r = 0; r < R; r++) {
    klim[r] = s_end;
    if (a.causal) {
      int own = causal_offset(a, S) + (lg + 4 * r) / a.G + 1;
      klim[r] = own < s_end ? own : s_end;
    }
    klim_min = klim[r] < klim_min ? klim[r] : klim_min;
  }

  // Paged cache: the 32 keys of a block lie in one page (pages hold a power of two >= 32 rows and blocks start at
  // multiples of 32); its number is read one block ahead.
  const int* table = PAGED ? a.block_table + (long long)b * a.bt_stride : nullptr;
  int page_next = 0;
  if (PAGED && s_begin + wave * KB < s_end) page_next = table[(s_begin + wave * KB) >> a.page_shift];

  for (int k0 = s_begin + wave * KB; k0 < s_end; k0 += NWAVE * KB) {
    const T* kpb = kp;
    const T* vpb = vp;
    int key0 = 0;  // first key of the memory region kpb / vpb point to
    if (PAGED) {
      kpb = (const T*)a.k + (long long)page_next * a.ks[0] + hk * a.ks[1];
      vpb = (const T*)a.v + (long long)page_next * a.vs[0] + hk * a.vs[1];
      key0 = (k0 >> a.page_shift) << a.page_shift;
      if (k0 + NWAVE * KB < s_end) page_next = table[(k0 + NWAVE * KB) >> a.page_shift];
    }
    // ---- issue all loads of the block: K for the score MFMAs, V for the accumulation ----------------------------------
    u32x4 kreg[2][KS];
#pragma unroll
    for (int gi = 0; gi < 2; gi++) {
      int key = k0 + 16 * gi + l16;
      key = (key < S ? key : S - 1) - key0;
      const T* kr = kpb + key * a.ks[2] + 8 * lg;
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        if (!PAD) {
          kreg[gi][ks] = __builtin_nontemporal_load((const u32x4*)(kr + 32 * ks));  // read once: keep it out of the caches
        } else {
          const bool there = 32 * ks + 8 * lg < a.D;
          const u32x4 t = __builtin_nontemporal_load((const u32x4*)(there ? kr + 32 * ks : kr - 8 * lg));
          kreg[gi][ks] = there ? t : u32x4{0u, 0u, 0u, 0u};
        }
      }
    }
    u32x4 vreg[KB / PH];
#pragma unroll
    for (int i = 0; i < KB / PH; i++) {
      int key = k0 + PH * i + vph;
      key = (key < S ? key : S - 1) - key0;
      vreg[i] = __builtin_nontemporal_load((const u32x4*)(vpb + key * a.vs[2] + (PAD && 8 * vc >= a.D ? 0 : 8 * vc)));
    }

    // ---- scores --------------------------------------------------------------------------------------------------------
    f32x4 sc[2];
#pragma unroll
    for (int gi = 0; gi < 2; gi++) {
      sc[gi] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ks++)
        sc[gi] = TR::mfma16(qa[ks], __builtin_bit_cast(vec8, kreg[gi][ks]), sc[gi]);
      if (k0 + 16 * gi + l16 >= klim_min) {
#pragma unroll
        for (int r = 0; r < 4; r++)
          if (r >= R || k0 + 16 * gi + l16 >= klim[r < R ? r : 0]) sc[gi][r] = -INFINITY;
      }
    }

    // ---- running softmax per row (register r of score-lane group lg is row lg + 4r) -----------------------------------
#pragma unroll
    for (int r = 0; r < R; r++) {
      float mloc = row16_max(fmaxf(sc[0][r], sc[1][r]));
      float m_new = fmaxf(m_run[r], mloc);
      float alpha = fast_exp2((m_run[r] - m_new) * c);
      float mc = m_new * c;
      m_run[r] = m_new;
      float p0 = fast_exp2(fmaf(sc[0][r], c, -mc));
      float p1 = fast_exp2(fmaf(sc[1][r], c, -mc));
      l_run[r] = l_run[r] * alpha + p0 + p1;
      pl[(l16)*NR + 4 * r + lg] = p0;
      pl[(16 + l16) * NR + 4 * r + lg] = p1;
      if (l16 == 0) pl[KB * NR + 4 * r + lg] = alpha;
    }
    wave_lds_sync();

    // ---- rescale and accumulate P.V -------------------------------------------------------------------------------------
#pragma unroll
    for (int r = 0; r < R; r++) {
      f32x4 al = *(const f32x4*)(pl + KB * NR + 4 * r);
#pragma unroll
      for (int j = 0; j < 4; j++)
#pragma unroll
        for (int i = 0; i < 8; i++) acc[4 * r + j][i] *= al[j];
    }
#pragma unroll
    for (int i = 0; i < KB / PH; i++) {
      float vf[8];
#pragma unroll
      for (int w = 0; w < 4; w++) {
        vf[2 * w] = TR::lo(vreg[i][w]);
        vf[2 * w + 1] = TR::hi(vreg[i][w]);
      }
#pragma unroll
      for (int r = 0; r < R; r++) {
        f32x4 p = *(const f32x4*)(pl + (PH * i + vph) * NR + 4 * r);
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
          for (int e = 0; e < 8; e++) acc[4 * r + j][e] = fmaf(p[j], vf[e], acc[4 * r + j][e]);
      }
    }
    wave_lds_sync();
  }

  // ---- wavefront totals: sums over the 16 key lanes; accumulators over the 4 key phases ------------------------------------
#pragma unroll
  for (int r = 0; r < R; r++) l_run[r] = row16_sum(l_run[r]);
#pragma unroll
  for (int x = 0; x < NR; x++)
#pragma unroll
    for (int i = 0; i < 8; i++) {
      float t = acc[x][i];
      if (CH <= 8) t += __shfl_xor(t, 8);
      t += __shfl_xor(t, 16);
      t += __shfl_xor(t, 32);
      acc[x][i] = t;
    }
  if (vph == 0) {
#pragma unroll
    for (int x = 0; x < NR; x++)
#pragma unroll
      for (int i = 0; i < 8; i++) Om[wave][x][8 * vc + i] = acc[x][i];
  }
  if (l16 == 0) {
#pragma unroll
    for (int r = 0; r < R; r++) {
      Om[wave][4 * r + lg][DD] = m_run[r];
      Om[wave][4 * r + lg][DD + 1] = l_run[r];
    }
  }
  __syncthreads();

  // ---- merge the four wavefronts; thread t handles (row slot, dim) pairs ------------------------------------------------------
  for (int e = tid; e < NR * DD; e += 256) {
    int x = e / DD, d = e % DD;  // row slot x holds query row x (slot index == query row index)
    if (x >= rows) continue;
    float mx = Om[0][x][DD];
#pragma unroll
    for (int w = 1; w < NWAVE; w++) mx = fmaxf(mx, Om[w][x][DD]);
    float lsum = 0.f, o = 0.f;
#pragma unroll
    for (int w = 0; w < NWAVE; w++) {
      float f = fast_exp2((Om[w][x][DD] - mx) * c);
      lsum += f * Om[w][x][DD + 1];
      o += f * Om[w][x][d];
    }
    if (splits == 1) {
      int xl = x / a.G, xg = x % a.G;
      T* op = (T*)a.out + b * a.os[0] + (hk * a.G + xg) * a.os[1] + xl * a.os[2];
      if (!PAD || d < a.D) store_from_float(op + d, lsum > 0.f ? o / lsum : 0.f);  // no keys at all: zeros, as the reference's empty contraction
    } else {
      float* rec = ws + ((long long)blockIdx.x * rows + x) * (DD + 2);
      rec[d] = o;
      if (d == 0) {
        rec[DD] = mx;
        rec[DD + 1] = lsum;
      }
    }
  }
}

// Combine the per-split records of one query row: one workgroup of head_dim threads per (batch, kv head, row).  The first
// wavefront turns the (max, sum) pairs of the up to 64 splits into weights (one split per lane, wave reductions);
// then thread d accumulates head_dim element d over the splits with independent, coalesced loads.
constexpr int kMaxSplits = 64;
template <typename T, int DD>
__global__ __launch_bounds__(DD) void merge_kernel(KArgs a, int splits, const float* __restrict__ ws) {
  __shared__ float weight[kMaxSplits];
  __shared__ float total;
  const int rows = a.L * a.G;
  const int pair = blockIdx.x / rows, x = blockIdx.x % rows;  // pair = b * Hkv + hk
  const int hk = pair % a.Hkv, b = pair / a.Hkv;
  const float c = a.scale * kLog2e;
  const float* rec0 = ws + ((long long)pair * splits * rows + x) * (DD + 2);
  const long long step = (long long)rows * (DD + 2);
  const int t = threadIdx.x;
  if (t < 64) {
    const bool have = t < splits;
    const float m = have ? rec0[t * step + DD] : -1e30f;
    const float l = have ? rec0[t * step + DD + 1] : 0.f;
    float mx = m;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
    const float f = have ? fast_exp2((m - mx) * c) : 0.f;
    float lsum = f * l;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) lsum += __shfl_xor(lsum, off);
    weight[t] = f;
    if (t == 0) total = lsum;
  }
  __syncthreads();
  float o = 0.f;
#pragma unroll 8
  for (int s = 0; s < splits; s++) o = fmaf(weight[s], rec0[s * step + t], o);
  const int xl = x / a.G, xg = x % a.G;
  T* op = (T*)a.out + b * a.os[0] + (hk * a.G + xg) * a.os[1] + xl * a.os[2];
  if (t < a.D) store_from_float(op + t, total > 0.f ? o / total : 0.f);  // (a.D < DD: the decode kernel's zero-column variant)
}

template <typename TR, int DD, bool PAD>
int launch_decode_t(const KArgs& a, const DecodePlan& pl, float* ws, hipStream_t stream) {
  typedef typename TR::elem T;
  dim3 grid((unsigned)((long long)a.B * a.Hkv * pl.splits)), block(256);
  int R = (pl.rows + 3) / 4;
#define TT_DECODE(R_)                                                                                                      \
  if (a.block_table)                                                                                                       \
    hipLaunchKernelGGL((decode_kernel<TR, R_, DD, true, PAD>), grid, block, 0, stream, a, pl.splits, pl.chunk, ws);       \
  else                                                                                                                     \
    hipLaunchKernelGGL((decode_kernel<TR, R_, DD, false, PAD>), grid, block, 0, stream, a, pl.splits, pl.chunk, ws)
  switch (R) {
    case 1: TT_DECODE(1); break;
    case 2: TT_DECODE(2); break;
    case 3: TT_DECODE(3); break;
    default: TT_DECODE(4); break;
  }
#undef TT_DECODE
  int rc = (int)hipGetLastError();
  if (rc != 0 || pl.splits == 1) return rc;
  hipLaunchKernelGGL((merge_kernel<T, DD>), dim3((unsigned)((long long)a.B * a.Hkv * pl.rows)), dim3(DD), 0, stream, a, pl.splits, ws);
  return (int)hipGetLastError();
}

}  // namespace

DecodePlan plan_decode(const KArgs& a) {
  DecodePlan p;
  p.rows = a.L * a.G;
  const int round = NWAVE * KB;
  long long pairs = (long long)a.B * a.Hkv;
  int max_splits = (a.S + 2 * round - 1) / (2 * round);
  if (max_splits < 1) max_splits = 1;
  long long want = (2 * 256 + pairs - 1) / pairs;  // aim for >= 2 workgroups per CU
  int splits = (int)(want < 1 ? 1 : want);
  if (splits > max_splits) splits = max_splits;
  if (splits > kMaxSplits) splits = kMaxSplits;
  int chunk = (a.S + splits - 1) / splits;
  chunk = (chunk + round - 1) / round * round;
  if (chunk < round) chunk = round;
  splits = (a.S + chunk - 1) / chunk;
  if (splits < 1) splits = 1;
  p.splits = splits;
  p.chunk = chunk;
  p.ws_bytes = splits > 1 ? (size_t)pairs * splits * p.rows * ((a.D <= 64 ? 64 : 128) + 2) * sizeof(float) : 0;  // the kernel's head_dim: 64 or 128
  return p;
}

int launch_merge(const KArgs& a, int dtype, int splits, const float* ws, hipStream_t stream) {
  const dim3 grid((unsigned)((long long)a.B * a.Hkv * a.L * a.G));
  if (dtype == 0) {
    if (a.D == 64) hipLaunchKernelGGL((merge_kernel<float, 64>), grid, dim3(64), 0, stream, a, splits, ws);
    else hipLaunchKernelGGL((merge_kernel<float, 128>), grid, dim3(128), 0, stream, a, splits, ws);
  } else if (a.D == 64) {
    if (dtype == 1) hipLaunchKernelGGL((merge_kernel<_Float16, 64>), grid, dim3(64), 0, stream, a, splits, ws);
    else hipLaunchKernelGGL((merge_kernel<__bf16, 64>), grid, dim3(64), 0, stream, a, splits, ws);
  } else {
    if (dtype == 1) hipLaunchKernelGGL((merge_kernel<_Float16, 128>), grid, dim3(128), 0, stream, a, splits, ws);
    else hipLaunchKernelGGL((merge_kernel<__bf16, 128>), grid, dim3(128), 0, stream, a, splits, ws);
  }
  return (int)hipGetLastError();
}

int launch_decode(const KArgs& a, int dtype, void* workspace, hipStream_t stream) {
  DecodePlan pl = plan_decode(a);
  if (a.D == 64)
    return dtype == 1 ? launch_decode_t<F16, 64, false>(a, pl, (float*)workspace, stream)
                      : launch_decode_t<BF16, 64, false>(a, pl, (float*)workspace, stream);
  if (a.D == 128)
    return dtype == 1 ? launch_decode_t<F16, 128, false>(a, pl, (float*)workspace, stream)
                      : launch_decode_t<BF16, 128, false>(a, pl, (float*)workspace, stream);
  // any other multiple of 8 up to 128: the kernel of the next size up, the missing columns as zeros
  if (a.D % 8 != 0 || a.D < 8 || a.D > 128) return (int)hipErrorInvalidValue;  // (the callers keep to this)
  if (a.D < 64)
    return dtype == 1 ? launch_decode_t<F16, 64, true>(a, pl, (float*)workspace, stream)
                      : launch_decode_t<BF16, 64, true>(a, pl, (float*)workspace, stream);
  return dtype == 1 ? launch_decode_t<F16, 128, true>(a, pl, (float*)workspace, stream)
                    : launch_decode_t<BF16, 128, true>(a, pl, (float*)workspace, stream);
}

}  // namespace ttsdpa
