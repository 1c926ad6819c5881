// Flash-attention forward for fp16 / bf16, head_dim 64, on gfx950 matrix cores: the pipelined prefill kernel of
// sdpa_prefill_d128.hip restated for rows of 128 bytes.  Same work split (8 wavefronts x 32 query rows, 64-key tiles by
// direct global->LDS loads, four K and four V stages), same three-strand software pipeline with the steady state as
// generated instruction streams, lazy maximum, mirrored causal row tiles, diagonal tile in the pipelined form; that file's
// header has the design.  What differs at head_dim 64:
//   * a half tile of 32 keys is 4 + 4 matrix instructions (S^T over 4 k-steps, P.V over 2 key steps x 2 head_dim blocks)
//     for the same 16 score registers, so a step is 8 slots that carry two scores' vector work each
//     (prefill64_steps.inc, written by gen_prefill128_steps.py 64);
//   * a tile row is 8 chunks of 16 bytes; chunk c of row r sits at slot c ^ f(r), f(r) = 4*((r/2)%2) + (r/4)%4: the 16
//     lanes a ds_read_b128 serves per cycle (16 rows, one chunk index) and the 32 lanes of a transposing read (4 rows x
//     4 chunks x 2 halves) each cover all 64 banks once;
//   * a wavefront brings its 8 rows of a tile with one load instruction (1 KiB), so the waits count one load per tile
//     and stream;
//   * the 32 rows of a wavefront leave through LDS in one round (4 KiB of staging each).
// A Bool attnMask whose keys can be read four at a time is applied in the streams as in that file (variant MASKB: the
// wavefront's mask bytes of a tile come into a ring in LDS two tiles ahead, a step reads the lane's dwords of the half
// after next and keeps a probability iff its byte is set).  Calls with another attnMask or a paged cache stay on the
// 4-wavefront kernel (sdpa_prefill.hip).

#include "sdpa_common.h"
#include "prefill64_steps.inc"  // hand-ordered instruction streams of the steady state (gen_prefill128_steps.py 64)

namespace ttsdpa {

namespace {

constexpr int D = 64;
constexpr int NW = 8;    // wavefronts per workgroup
constexpr int WM = 32;   // query rows per wavefront
constexpr int BM = NW * WM;  // query rows per workgroup
constexpr int BN = 64;   // keys per tile
constexpr int ROW_BYTES = D * 2;
constexpr int STAGE_BYTES = BN * ROW_BYTES;  // 8 KiB
constexpr int KSTAGES = 4, VSTAGES = 4;     // K and V tiles are requested three tiles before use
constexpr int OUT_BYTES = NW * WM * ROW_BYTES;  // output staging: the 32 rows of every wavefront
constexpr int LDS_BYTES = (KSTAGES + VSTAGES) * STAGE_BYTES + OUT_BYTES;
constexpr float kSumLimit = 1024.f;  // a lane's 16 probabilities of a half may sum to this much before the maximum is raised

typedef uint32_t u32x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x32 __attribute__((ext_vector_type(32)));
typedef uint32_t u32x16 __attribute__((ext_vector_type(16)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
typedef __attribute__((address_space(3))) void lds_void;
typedef __attribute__((address_space(1))) const void gbl_void;

__device__ __forceinline__ int swz(int row) { return (((row >> 1) & 1) << 2) | ((row >> 2) & 3); }

// SPLIT (launches with very few row tiles): a workgroup takes key tiles kt0 .. kt0 + kv_chunk/64 - 1 of its row tile (kt0 a
// multiple of 4, so the stages keep their constants) and leaves (unnormalised accumulator, maximum, sum) records in a.ws
// for prefill_split_merge_kernel; row tiles are single (no mirror pairs).
// MASKB (calls without a causal mask or splits): a.mask is a Bool mask with unit key stride, dword-aligned rows and row
// offsets below 2^32; the steady state applies it in the streams.
template <typename TR, bool CAUSAL, bool SPLIT, bool MASKB = false>
__global__ __launch_bounds__(NW * 64, 2) void prefill64_kernel(KArgs a) {
  static_assert(!MASKB || (!CAUSAL && !SPLIT), "the Bool-mask streams exist for the plain variant only");
  constexpr bool PAGED = false;  // paged caches stay on the 4-wavefront kernel
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
  const bool paired = CAUSAL && !SPLIT && !a.single_tiles;  // else one row tile per workgroup, longest first
  const bool by_length = CAUSAL && !paired;  // work items ordered by row tile across the pairs of a class
  const int nslot = paired ? (ntile + 1) / 2 : ntile;
  const int inner = a.G * nslot;
  const int npair = a.B * a.Hkv;
  int pair, in;
  {
    // Workgroup n runs on XCD n % 8, and the workgroups of one (batch, kv head) share its K/V through an XCD's L2: with
    // g = gcd(pairs, 8) the XCDs form g classes of 8/g, class x % g serves the pairs congruent to it and deals the
    // work items (heads x row tiles) of those pairs out to its XCDs in turn.  A multiple of 8 pairs puts every pair on
    // one XCD; 4 pairs (config 5) give each pair two XCDs instead of all eight streaming all four.
    int n = blockIdx.x;
    if (SPLIT) n = (int)(blockIdx.x / (8u * a.kv_splits)) * 8 + (blockIdx.x & 7);  // the splits of a work item follow each other on its XCD
    const int gq = (npair & 7) == 0 ? 8 : ((npair & 3) == 0 ? 4 : ((npair & 1) == 0 ? 2 : 1));
    const int xcd = n & 7, slot = n >> 3;
    const int cls = xcd % gq, sub = xcd / gq;
    const long long item = (long long)slot * (8 / gq) + sub;  // work item of the class
    const long long items = (long long)(npair / gq) * inner;
    if (item >= items) return;  // the grid is rounded up to a multiple of 8
    if (by_length) {  // longest tiles first across all the pairs of the class
      const int ppc = npair / gq;
      pair = cls + gq * (int)(item % ppc);
      in = (int)(item / ppc);
    } else {
      pair = cls + gq * (int)(item / inner);
      in = (int)(item % inner);
    }
  }
  const int b = pair / a.Hkv, hk = pair % a.Hkv;
  const int g = in % a.G;
  const int slot_rt = in / a.G;
  const int h = hk * a.G + g;
  const int split = SPLIT ? (int)(blockIdx.x % (8u * a.kv_splits)) >> 3 : 0;
  const int kt0 = SPLIT ? split * (a.kv_chunk / BN) : 0;  // first key tile of this workgroup

  const T* qp = (const T*)a.q + b * a.qs[0] + h * a.qs[1];
  const int* table = PAGED ? a.block_table + (long long)b * a.bt_stride : nullptr;
  const T* kp = (const T*)a.k + (PAGED ? 0 : b * a.ks[0]) + hk * a.ks[1];
  const T* vp = (const T*)a.v + (PAGED ? 0 : b * a.vs[0]) + hk * a.vs[1];
  int S = a.S;  // keys of this batch entry: all of them, or the filled prefix of a cache / the unpadded length
  if (a.kv_len) {
    int len = __builtin_amdgcn_readfirstlane(a.kv_len[b]);
    S = len < 0 ? 0 : (len < S ? len : S);
  }

  // Every workgroup takes its long tile first: the workgroups of a head that run together then walk its keys from the
  // first one on in step, and an XCD's L2 serves all but the first of them.  (With neighbouring workgroups in opposite
  // order a head's K/V came from memory about three times where one KV head serves one query head: B4 32 heads of 2048
  // rows, fp16: 468 -> 275 MB read per launch, same time; grouped heads were and are read once.)
  const bool long_first = true;
  // Wavefronts w and w+4 share a SIMD.  Under a causal mask the row group g of a tile has g+1 halves of work on the
  // diagonal, so the second four wavefronts take the groups in reverse: every SIMD then carries groups g and 7-g.
  const int rowgroup = (CAUSAL && wave >= 4) ? 11 - wave : wave;

  if (S == 0) {  // no keys for this batch entry: zeros, the reference's empty contraction (kept out of the main loop)
    if (SPLIT) return;  // the merge kernel writes them
    T* obase = (T*)a.out + b * a.os[0] + h * a.os[1];
    vec8 zero;
#pragma unroll
    for (int i = 0; i < 8; i++) zero[i] = (T)0.f;
    for (int part = 0; part < (CAUSAL ? 2 : 1); part++) {
      if (part == 1 && (!paired || slot_rt >= ntile - 1 - slot_rt)) break;
      const int rt = (CAUSAL && part == 0) ? ntile - 1 - slot_rt : slot_rt;
      for (int i = 0; i < 4; i++) {
        const int qi = rt * BM + rowgroup * WM + 8 * i + (lane >> 3);
        if (qi < a.L) *(vec8*)(obase + qi * a.os[2] + 8 * (lane & 7)) = zero;
      }
    }
    return;
  }

  // ---- geometry of a part: first query row of the workgroup's row tile and its KV tile count ----------------------
  auto part_rows = [&](int part, int& q0, int& ntiles_kv) __attribute__((always_inline)) {
    const int rt = (CAUSAL && (part == 0) == long_first) ? ntile - 1 - slot_rt : slot_rt;
    q0 = rt * BM;
    ntiles_kv = (S + BN - 1) / BN;
    if (CAUSAL) {
      const int coff = causal_offset(a, S);
      int last = (q0 + BM - 1 < a.L - 1 ? q0 + BM - 1 : a.L - 1) + coff;
      int lastkv = last < S - 1 ? last : S - 1;
      ntiles_kv = lastkv / BN + 1;
    }
    if (SPLIT) {  // this workgroup's tiles end with its split (none at all: ntiles_kv <= kt0)
      const int end = kt0 + a.kv_chunk / BN;
      ntiles_kv = end < ntiles_kv ? end : ntiles_kv;
    }
  };
  if (SPLIT) {  // a split beyond the row tile's keys has nothing to do; the merge kernel knows which those are
    int q0, ntiles_kv;
    part_rows(0, q0, ntiles_kv);
    if (ntiles_kv <= kt0) return;
  }
  const bool two_parts = paired && slot_rt < ntile - 1 - slot_rt;  // odd count: the middle tile has no mirror

  // ---- global -> LDS: wavefront w moves rows 8w .. 8w+7 of a tile with one instruction (8 rows, 1 KiB) -----------
  // lane l fills slot (row l/8, chunk slot l%8) and therefore fetches chunk (l%8) ^ f(row)
  unsigned ld_koff[1], ld_voff[1];
  {
    int row = 8 * wave + (lane >> 3);
    int chunk = (lane & 7) ^ swz(row);
    ld_koff[0] = ((unsigned)row * (unsigned)a.ks[2] + 8u * chunk) * 2u;  // the host checks that 64 rows fit 32 bits
    ld_voff[0] = ((unsigned)row * (unsigned)a.vs[2] + 8u * chunk) * 2u;
  }
  // Issued as asm so that the compiler does not see a store to LDS: it would otherwise make every later LDS read
  // wait for all outstanding loads (vmcnt(0)).  The waits are placed by hand in dma_wait_and_sync.
  // s_nop 3: the compiler's hazard pass does not look into the statement, and a scalar base that it restored with a
  // vector instruction (v_readlane of a spilled scalar register, v_readfirstlane) just before is only valid for a
  // memory instruction five wait states later; s_mov + s_nop 3 make five.
  auto dma_issue = [&](const char* sbase, unsigned voff, unsigned lds_addr) __attribute__((always_inline)) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 3\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(sbase), "s"(lds_addr) : "memory", "m0");
  };
  const unsigned smem_addr = (unsigned)(unsigned long)(lds_void*)smem;
  // Paged cache: the table entry of a tile is fetched while the previous tile of the same stream (K or V) is issued,
  // so that the address of a tile does not wait for a scalar load: {entry index, page} of the prefetched entry.
  int kpage[2] = {-1, 0}, vpage[2] = {-1, 0};
  auto dma_tile = [&](const T* base, long long rstride, long long pstride, int (&pc)[2], const unsigned (&off)[1], int kv0, unsigned stage_addr) __attribute__((always_inline)) {
    long long toff = (long long)kv0 * rstride;
    if (PAGED) {
      const int want = kv0 >> a.page_shift;
      int page = pc[1];
      if (pc[0] != want) page = __builtin_amdgcn_readfirstlane(table[want]);
      toff = (long long)page * pstride + (long long)(kv0 & ((1 << a.page_shift) - 1)) * rstride;
      const int nxt = (kv0 + BN) >> a.page_shift;
      pc[0] = want, pc[1] = page;
      if (nxt != want && kv0 + BN < S) pc[0] = nxt, pc[1] = __builtin_amdgcn_readfirstlane(table[nxt]);
    }
    const T* tile = base + toff;
    if (__builtin_expect(kv0 + BN <= S, 1)) {
      const char* src = (const char*)tile;
      dma_issue(src, off[0], stage_addr + (8 * wave) * ROW_BYTES);
    } else {  // ragged last tile: rows past the end re-read the last valid row (their scores are masked)
      int row = 8 * wave + (lane >> 3);
      asm volatile("" : "+v"(row));  // keeps this rarely taken path's address arithmetic inside the branch
      int chunk = (lane & 7) ^ swz(row);
      int rowc = row < S - kv0 ? row : S - 1 - kv0;
      unsigned voff = ((unsigned)rowc * (unsigned)rstride + 8u * chunk) * 2u;
      dma_issue((const char*)tile, voff, stage_addr + (8 * wave) * ROW_BYTES);
    }
  };
  auto dma_k = [&](int tile, int stage) __attribute__((always_inline)) { dma_tile(kp, a.ks[2], a.ks[0], kpage, ld_koff, tile * BN, smem_addr + stage * STAGE_BYTES); };
  auto dma_v = [&](int tile, int stage) __attribute__((always_inline)) { dma_tile(vp, a.vs[2], a.vs[0], vpage, ld_voff, tile * BN, smem_addr + (KSTAGES + stage) * STAGE_BYTES); };
  // Wait until at most `keep` of this wavefront's global->LDS loads are still in flight (they complete in issue
  // order), then meet the other wavefronts: what was issued before the newest `keep` loads is visible to all.
  auto dma_wait_and_sync = [&](int keep) __attribute__((always_inline)) {
    // (`keep` counts as in the head_dim-128 kernel, two loads per tile; here a tile is one load)
    if (__builtin_expect(keep >= 4, 1)) {
      asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
    } else if (keep >= 2) {
      asm volatile("s_waitcnt vmcnt(1)" ::: "memory");
    } else {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    // bare barrier: the loads above carry the ordering; __syncthreads() would also drain the LDS operand prefetch
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };

  // ---- LDS operand addresses (bytes), loop-invariant ---------------------------------------------------------------
  // K operand (half, ks): row 32*half + lq, chunk 2*ks + lh  ->  row*256 + 16*((2ks + lh) ^ f(row))
  u32x4 k_addr;
  {
    unsigned base = (unsigned)(lq * ROW_BYTES + 16 * (lh ^ swz(lq)));  // f(32*half + lq) == f(lq)
#pragma unroll
    for (int ks = 0; ks < 4; ks++) k_addr[ks] = base ^ (unsigned)(32 * ks);
  }
  // V operand part (db, ld) of k-step t via the transpose load: this lane points at row 16t + 8ld + 4lh + s/4,
  // elements 32db + 16*dhalf + 4*(s%4) .. +3 (s = lane%16, dhalf = (lane/16)%2) and receives
  // V[16t + 8ld + 4lh + 0..3][32db + lq]
  u32x4 v_addr;  // index 2 * db + ld
  {
    const int s = lane & 15, dhalf = (lane >> 4) & 1;
#pragma unroll
    for (int ld = 0; ld < 2; ld++) {
      int row = 8 * ld + 4 * lh + (s >> 2);  // + 16t later: f(row) does not depend on t
#pragma unroll
      for (int db = 0; db < 2; db++) {
        int chunk = 4 * db + 2 * dhalf + ((s & 3) >> 1);
        // the V region's base is folded in here so that stage and k-step offsets fit the 16-bit ds_read immediate
        v_addr[2 * db + ld] = (unsigned)(KSTAGES * STAGE_BYTES + row * ROW_BYTES + 16 * (chunk ^ swz(row)) + 8 * (s & 1));
      }
    }
  }


  // ---- first loads of a part ---------------------------------------------------------------------------------------------
  // K runs one tile ahead of V in consumption (scores are formed two halves before their P.V), so K is requested
  // four tiles ahead and V three: iteration j sends for K(j+4) (stage of K(j), last read in iteration j-1) and
  // V(j+3) (stage of V(j-1)).  A part starts with K(0..3) and V(0..2) on their way.  For the second part they are sent
  // for before the first part's output is written: every stage is free then (all wavefronts passed the closing barrier
  // of the last tile; the output passes through a staging area of its own).
  auto issue_tiles = [&](int part) __attribute__((always_inline)) {
    int q0, ntiles_kv;
    part_rows(part, q0, ntiles_kv);
    kpage[0] = -1, vpage[0] = -1;
    dma_k(kt0, 0);
    if (kt0 + 1 < ntiles_kv) dma_k(kt0 + 1, 1);
    dma_v(kt0, 0);
    if (kt0 + 2 < ntiles_kv) dma_k(kt0 + 2, 2);
    if (kt0 + 1 < ntiles_kv) dma_v(kt0 + 1, 1);
    if (kt0 + 3 < ntiles_kv) dma_k(kt0 + 3, 3);
    if (kt0 + 2 < ntiles_kv) dma_v(kt0 + 2, 2);
  };
  issue_tiles(0);
  // ---- Bool attnMask in the streams (MASKB): the scheme of sdpa_prefill_d128.hip ------------------------------------------
  // Ring in LDS: two tiles of 2 KiB per wavefront in the output staging area (idle during the loop).  Load i of a tile
  // (two per tile) brings the 64-byte segments of rows 16i .. 16i+15 of the wavefront, 16 bytes per lane: chunk c of row q
  // lands at 1024 (q/16) + 256 c + 16 (q%16).  A lane (row q, h = lane/32) needs dwords h and h + 2 of chunks 2H and 2H + 1
  // of its row for half H of a tile; registers: half H of the workgroup's keys in places 4(H%2) .. +3.  Tile j sends for
  // the mask bytes of tile j+2 ahead of its K/V loads (the wait at the tile's end covers them), and its two steps read
  // halves 2j+2 and 2j+3 into registers for the steps after them.
  u32x8 mring;
  unsigned mrow_off[2];           // the lane's byte offset in a (batch, head)'s mask for the two loads of a tile
  unsigned mlds = 0;              // LDS address of the lane's row in the wavefront's ring, plus 4 * (lane/32)
  const char* mbase = nullptr;    // first mask byte of this (batch, head); uniform
  unsigned mring_addr = 0;        // LDS address of the wavefront's ring
  if constexpr (MASKB) {
#pragma unroll
    for (int i = 0; i < 8; i++) mring[i] = 0u;
    int q0, ntiles_kv;
    part_rows(0, q0, ntiles_kv);
    const int qw = q0 + rowgroup * WM;
#pragma unroll
    for (int i = 0; i < 2; i++) {
      int row = qw + 16 * i + (lane & 15);
      row = row < a.L ? row : a.L - 1;  // rows past the end re-read the last one
      mrow_off[i] = (unsigned)row * (unsigned)a.ms[2] + 16u * (lane >> 4);  // the host checks that the last row's offset fits 32 bits
    }
    mbase = (const char*)a.mask + b * a.ms[0] + h * a.ms[1];
    mring_addr = smem_addr + (KSTAGES + VSTAGES) * STAGE_BYTES + wave * 4096;
    mlds = mring_addr + 1024 * (lq >> 4) + 16 * (lq & 15) + 4 * lh;
  }
  // a tile's mask bytes into ring place `place`; tiles beyond the row's last whole one are moved back into it (nobody takes them)
  auto mask_dma = [&](int tile, int place) __attribute__((always_inline)) {
    const int k0 = 64 * tile < S - 64 ? 64 * tile : S - 64;
    asm volatile(TT_P64_MDMA
                 :
                 : [o0] "v"(mrow_off[0]), [o1] "v"(mrow_off[1]), [mtile] "s"(mbase + k0),
                   [dst] "s"(mring_addr + 2048 * place)
                 : "memory", "m0", "scc");
  };
  if constexpr (MASKB) {
    if (S >= 160) {  // (shorter rows have no tile in the fast form)
      mask_dma(kt0, 0);
      mask_dma(kt0 + 1, 1);
    }
  }
  u32x16 qv;  // the lane's Q operands, k-step ks in elements 4ks .. 4ks+3
  // Q of a part into its registers, and everything sent for so far in place.  One statement: the compiler takes a statement's
  // results as valid when it ends, so the wait has to be part of it (and, not knowing of the tile loads, the compiler
  // would place waits of its own for plain loads that in effect wait for every tile).
  auto load_q = [&](int part) __attribute__((always_inline)) {
    int q0, ntiles_kv;
    part_rows(part, q0, ntiles_kv);
    const int qw0 = q0 + rowgroup * WM;
    const int first = qw0 < a.L ? qw0 : a.L - 1;  // rows past the end re-read the last row (never stored)
    int row = qw0 + lq;
    row = row < a.L ? row : a.L - 1;
    const char* qbase = (const char*)(qp + (long long)first * a.qs[2]);
    const unsigned qoff = ((unsigned)(row - first) * (unsigned)a.qs[2] + 8u * lh) * 2u;  // the host checks that 32 rows fit 32 bits
    asm volatile(
        "s_nop 4\n\t"  // the base may have been written by a vector instruction (a restored scalar register): 5 wait states
        "global_load_dwordx4 v[120:123], %1, %2\n\t"
        "global_load_dwordx4 v[124:127], %1, %2 offset:32\n\t"
        "global_load_dwordx4 v[128:131], %1, %2 offset:64\n\t"
        "global_load_dwordx4 v[132:135], %1, %2 offset:96\n\t"
        "s_waitcnt vmcnt(0)"
        : "={v[120:135]}"(qv)
        : "v"(qoff), "s"(qbase)
        : "memory");
  };
  load_q(0);


  for (int part = 0; part < (CAUSAL ? 2 : 1); part++) {
  if (part == 1 && !two_parts) break;
  int q0, ntiles_kv;
  part_rows(part, q0, ntiles_kv);
  const int qw0 = q0 + rowgroup * WM;

  // Query row i sees keys up to i + coff (coff = 0: the reference's top-left aligned mask); qc0 is this wavefront's
  // first row in key coordinates.
  const int coff = CAUSAL ? causal_offset(a, S) : 0;
  const int qc0 = qw0 + coff;
  // 32-key halves this wavefront computes on: under a causal mask those that start at or before its last row
  int my_halves = 2 * ntiles_kv;
  if (CAUSAL) {
    int t = (qc0 + WM - 1) / 32 + 1;
    my_halves = t < my_halves ? t : my_halves;
  }
  // Tiles j whose two steps take the fast form: halves up to 2j+3 are this wavefront's, tile j+1 is complete, and
  // half 2j+2 (whose exponentials step 2j+1 takes) needs no mask.
  int nfast = (my_halves - 2) / 2;
  {
    int f = S >= 96 ? (S - 32) / BN : 0;
    nfast = f < nfast ? f : nfast;
    if (CAUSAL) {
      f = qc0 >= 95 ? (qc0 - 31) / BN : 0;
      nfast = f < nfast ? f : nfast;
    }
  }
  if (nfast < 0) nfast = 0;
  // Tiles in the fast form including those whose exponentials take the causal predicate (a variant of the streams):
  // both steps of tile j accumulate a half of this wavefront's (2j+1 < my_halves) and half 2j+2 is complete.
  int nfast_all = nfast;
  if (CAUSAL) {
    int t = my_halves / 2;
    const int f = S >= 96 ? (S - 32) / BN : 0;
    t = f < t ? f : t;
    nfast_all = t > nfast ? t : nfast;
  }
  if (MASKB ? S < 160 : a.mask_kind != 0) nfast = 0, nfast_all = 0;  // other attnMasks are applied in the general form of a step
  // The fast form requests its tiles without the ragged-tile case: iteration j sends for K(j+4) and V(j+3), which have to
  // be whole tiles.
  if (!PAGED && (S % BN) != 0) {
    int lim = S / BN - 4;
    lim = lim < 0 ? 0 : lim;
    nfast_all = lim < nfast_all ? lim : nfast_all;
    nfast = nfast_all < nfast ? nfast_all : nfast;
  }
  if (CAUSAL) {  // scalar registers: operands of the step statements derive from them
    nfast = __builtin_amdgcn_readfirstlane(nfast);
    nfast_all = __builtin_amdgcn_readfirstlane(nfast_all);
  }

  // ---- prologue: the part's first loads were sent for by issue_part ------------------------------------------------
  auto q_of = [&](int ks) __attribute__((always_inline)) {
    u32x4 w;
#pragma unroll
    for (int i = 0; i < 4; i++) w[i] = qv[4 * ks + i];
    return __builtin_bit_cast(vec8, w);
  };
  f32x16 oacc[2];
#pragma unroll
  for (int db = 0; db < 2; db++)
#pragma unroll
    for (int r = 0; r < 16; r++) oacc[db][r] = 0.f;
  const float c = a.scale * kLog2e;
  // the same, in a scalar register (causal step statements: their predicate operands take the freed vector register)
  const float c_s = CAUSAL ? __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, c))) : 0.f;
  float m_use = -1e30f;  // maximum the exponentials are taken against (raw scores)
  float mc = -1e30f * c;
  float l_run = 0.f;

  // S^T of one half tile (32 keys); kh = LDS address of the half's first K row
  auto qk_half = [&](f32x16& s, const char* kh) __attribute__((always_inline)) {
#pragma unroll
    for (int r = 0; r < 16; r++) s[r] = 0.f;
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
      vec8 ka = *(const vec8*)(kh + k_addr[ks]);
      s = TR::mfma32(ka, q_of(ks), s);
    }
  };

  auto mask_half = [&](f32x16& s, int kv0) __attribute__((always_inline)) {
    const int qi = qc0 + lq;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      int key = kv0 + 8 * (r >> 2) + 4 * lh + (r & 3);
      bool hidden = key >= S || (CAUSAL && key > qi);
      if (hidden) s[r] = -INFINITY;
    }
  };

  auto user_mask_half = [&](f32x16& s, int kv0) __attribute__((always_inline)) {
    int qi = qw0 + lq;
    qi = qi < a.L ? qi : a.L - 1;
    apply_attn_mask<T, false>(a, s, b * a.ms[0] + h * a.ms[1] + qi * a.ms[2], kv0, lh, S, 1.f / a.scale);
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

  // exponentials of one half against the current maximum -> P^T as MFMA B operands pb[k-step of 16 keys];
  // returns this lane's sum of the 16 probabilities
  auto exp_half = [&](const f32x16& s, vec8 (&pb)[2]) __attribute__((always_inline)) {
    float psum = 0.f;
#pragma unroll
    for (int t = 0; t < 2; t++) {
      f32x8 x;
#pragma unroll
      for (int i = 0; i < 8; i++) {
        x[i] = fast_exp2(fmaf(s[8 * t + i], c, -mc));
        psum += x[i];
      }
      pb[t] = __builtin_convertvector(x, vec8);
    }
    return psum;
  };

  // The exponentials are taken against a maximum that is only raised when a lane's sum of probabilities shows that
  // some probability left the range [0, kSumLimit] (which includes the first half of a row, taken against -1e30):
  // then the true row maximum is formed, sum and accumulator are rescaled and the half is redone.  Every
  // probability that reaches the matrix pipe is therefore at most kSumLimit.
  const int rl = CAUSAL ? qc0 + lq - 4 * lh : 0;  // the causal predicate's lane operand: key k of a score is visible iff k - 4*(lane/32) <= rl
  auto settle_half = [&](f32x16& s, vec8 (&pb)[2], float psum, int masked_kv0 = -1, int mask_place = -1) __attribute__((always_inline)) {
    if (__builtin_expect(__builtin_amdgcn_ballot_w64(!(psum <= kSumLimit)) != 0, 0)) {
      // after a step that applied a Bool attnMask in the stream: scores whose mask byte is clear must not enter the maximum
      if (MASKB && mask_place >= 0) {
#pragma unroll
        for (int r = 0; r < 16; r++)
          if (((mring[4 * mask_place + (r >> 2)] >> (8 * (r & 3))) & 0xffu) == 0u) s[r] = -INFINITY;
      }
      // after a step whose exponentials took the causal predicate in the stream, the scores themselves are masked only
      // here (hidden scores, or what a stage held beyond the workgroup's last tile, must not enter the maximum)
      if (CAUSAL && masked_kv0 >= 0) {
#pragma unroll
        for (int r = 0; r < 16; r++)
          if (masked_kv0 + 8 * (r >> 2) + (r & 3) > rl) s[r] = -INFINITY;  // the streams' predicate
      }
      const float m_new = fmaxf(m_use, row_max(s));
      const float alpha = fast_exp2((m_use - m_new) * c);
      m_use = m_new;
      mc = m_new * c;
      l_run *= alpha;
#pragma unroll
      for (int db = 0; db < 2; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) oacc[db][r] *= alpha;
      psum = exp_half(s, pb);
    }
    l_run += psum;
  };

  // O^T += V_half^T . P^T; vh = LDS address of the half's first V row
  auto pv_half = [&](const vec8 (&pb)[2], const char* vh) __attribute__((always_inline)) {
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
      for (int db = 0; db < 2; db++) {
        s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(vh + v_addr[2 * db] + 16 * t * ROW_BYTES));
        s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(vh + v_addr[2 * db + 1] + 16 * t * ROW_BYTES));
        vec8 va = __builtin_bit_cast(vec8, (s16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
        oacc[db] = TR::mfma32(va, pb[t], oacc[db]);
      }
  };

  // LDS address of the first K row of half h (v_addr carries the V region's base, so the same value serves V)
  auto half_base = [&](int h) __attribute__((always_inline)) {
    return smem + ((h >> 1) & 3) * STAGE_BYTES + (h & 1) * 32 * ROW_BYTES;
  };

  // Pipeline state between steps: P of half h (ready for the matrix pipe) and the raw scores of half h+1.
  // Step h:  matrix pipe: S^T(h+2) and O^T += V(h)^T . P(h);  vector ALU: P(h+1) = exp2(...) of the scores of h+1.
  // General form of a step (any half may be masked or missing); the compiler orders it.
  auto slow_step = [&](int h, const vec8 (&p_cur)[2], f32x16& s_nxt, f32x16& s_new, vec8 (&p_nxt)[2]) __attribute__((always_inline)) {
    if (h + 2 < my_halves) qk_half(s_new, half_base(h + 2));
    if (h < my_halves) pv_half(p_cur, half_base(h));
    if (h + 1 < my_halves) {
      const int kv0 = 32 * (h + 1);
      if ((CAUSAL && kv0 + 31 > qc0) || kv0 + 32 > S) mask_half(s_nxt, kv0);
      if (!CAUSAL && a.mask_kind != 0) user_mask_half(s_nxt, kv0);
      settle_half(s_nxt, p_nxt, exp_half(s_nxt, p_nxt));
    }
  };

  // ---- fast form: the 16 slots of a step as one statement of hand-ordered instructions (prefill128_steps.inc) ---------
  // A tile iteration has 32 slots (two steps of 16).  Even slot 2i of a step is the S^T MFMA of k-step i, odd slot
  // 2i+1 the P.V MFMA (t = i/4, db = i%4): the dependent S^T chain is spaced by independent P.V MFMAs.  Each slot
  // also carries one score's scale / exp2 / sum (and every second slot a pair's conversion), each issued a slot
  // apart from the instruction it depends on, and requests the LDS operand of the slot 6 places further on into a
  // ring of 8 operand registers.  The statements name fixed registers for everything a vector instruction touches
  // piecewise (scores, probabilities, operand ring, Q, LDS addresses); the output accumulators are ordinary operands.
  u32x32 ring;
#pragma unroll
  for (int i = 0; i < 32; i++) ring[i] = 0u;
#define TT_P64_RUN_STEP(TXT)                                                                                          \
  asm volatile(TXT                                                                                                     \
               : [o0] "+v"(oacc[0]), [o1] "+v"(oacc[1]), [ps] "=&v"(psum_step),                                          \
                 "+{v[160:175]}"(sB), "+{v[176:191]}"(sC), "+{v[192:199]}"(pAv), "+{v[200:207]}"(pBv),                   \
                 "+{v[208:239]}"(ring)                                                                                 \
               : [c] "s"(c_s), [mc] "v"(mc), [rl] "v"(rl), [mk] "s"(mk), [kvs] "s"(kvs), "{v[120:135]}"(qv), "{v[152:155]}"(v_addr), "{v[248:251]}"(k_addr) \
               : "v240", "v241", "v242", "v243", "v244", "v245", "vcc", "scc", "m0", "memory")
// the plain step alone (calls without a causal mask): no predicate operands
#define TT_P64_RUN_PSTEP(TXT)                                                                                         \
  asm volatile(TXT                                                                                                     \
               : [o0] "+v"(oacc[0]), [o1] "+v"(oacc[1]), [ps] "=&v"(psum_step),                                          \
                 "+{v[160:175]}"(sB), "+{v[176:191]}"(sC), "+{v[192:199]}"(pAv), "+{v[200:207]}"(pBv),                   \
                 "+{v[208:239]}"(ring)                                                                                 \
               : [c] "v"(c), [mc] "v"(mc), "{v[120:135]}"(qv), "{v[152:155]}"(v_addr), "{v[248:251]}"(k_addr)            \
               : "v240", "v241", "v242", "v243", "v244", "v245", "memory")
// the plain step with a Bool attnMask applied to each probability (mask registers v[112:119], a zero in a scalar register)
#define TT_P64_RUN_MSTEP(TXT)                                                                                         \
  asm volatile(TXT                                                                                                     \
               : [o0] "+v"(oacc[0]), [o1] "+v"(oacc[1]), [ps] "=&v"(psum_step),                                          \
                 "+{v[160:175]}"(sB), "+{v[176:191]}"(sC), "+{v[192:199]}"(pAv), "+{v[200:207]}"(pBv),                   \
                 "+{v[208:239]}"(ring), "+{v[112:119]}"(mring)                                                          \
               : [c] "v"(c), [mc] "v"(mc), [zero] "s"(0), [mlds] "v"(mlds), [mlds1] "v"(mlds + 2048), "{v[120:135]}"(qv), "{v[152:155]}"(v_addr), "{v[248:251]}"(k_addr) \
               : "v240", "v241", "v242", "v243", "v244", "v245", "vcc", "memory")
  constexpr bool kIsBf16 = sizeof(typename TR::elem) == 2 && __is_same(typename TR::elem, __bf16);

  f32x16 sB, sC;
  vec8 pA[2], pB[2];
  u32x8 pAv, pBv;  // P of a half as two MFMA B operands (k-steps of 16 keys), 4 registers each
  float psum_step;
  auto p_load = [&](const u32x8& pv, vec8 (&p)[2]) __attribute__((always_inline)) {
#pragma unroll
    for (int t = 0; t < 2; t++) {
      u32x4 w;
#pragma unroll
      for (int i = 0; i < 4; i++) w[i] = pv[4 * t + i];
      p[t] = __builtin_bit_cast(vec8, w);
    }
  };
  auto p_store = [&](u32x8& pv, const vec8 (&p)[2]) __attribute__((always_inline)) {
#pragma unroll
    for (int t = 0; t < 2; t++) {
      const u32x4 w = __builtin_bit_cast(u32x4, p[t]);
#pragma unroll
      for (int i = 0; i < 4; i++) pv[4 * t + i] = w[i];
    }
  };
  // every wavefront's waits for the part's first tiles (in load_q) are behind it: the tiles are visible to all
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  {  // P(0) and the scores of half 1
    const int kb = BN * kt0;  // the workgroup's first key (kt0 is a multiple of 4: its tile sits in stage 0)
    qk_half(sC, half_base(0));
    if (2 * kt0 + 1 < my_halves) qk_half(sB, half_base(1));
    if ((CAUSAL && kb + 31 > qc0) || kb + 32 > S) mask_half(sC, kb);
    if (!CAUSAL && a.mask_kind != 0) user_mask_half(sC, kb);
    // first half of a row: the maximum is formed directly (what the lazy rule arrives at after exponentials against
    // -1e30, with nothing to rescale yet); a fully hidden half keeps -1e30 and gives zeros
    m_use = fmaxf(m_use, row_max(sC));
    mc = m_use * c;
    l_run = exp_half(sC, pA);
  }
  // Every wavefront has read K(0): iteration 0 may overwrite its stage.  K(1), V(0), K(2), V(1) must be visible
  // before iteration 0; K(3) and V(2) (4 loads) are waited for at its end.
  if (CAUSAL && part == 1) {  // all of this part's loads so far were waited for in load_q; what is in flight are part 0's output stores
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  } else {
    dma_wait_and_sync(0);
  }

  auto tile_dma = [&](int j) __attribute__((always_inline)) {
    int keep = 0;
    if (__builtin_expect(j + 3 < ntiles_kv, 1)) {
      if (__builtin_expect(j + 4 < ntiles_kv, 1)) {
        dma_k(j + 4, j & 3);
        keep = 4;
      } else {
        keep = 2;
      }
      dma_v(j + 3, (j + 3) & 3);
    }
    return keep;
  };
  // The fast form's requests: whole tiles through two running pointers (the general form multiplies the tile number
  // out and carries the ragged and paged cases); U = j % 4 makes the stages constants.
  const char* kfast = (const char*)(kp + (long long)((kt0 + 4) * BN) * a.ks[2]);
  const char* vfast = (const char*)(vp + (long long)((kt0 + 3) * BN) * a.vs[2]);
  const long long kfast_step = (long long)BN * a.ks[2] * 2, vfast_step = (long long)BN * a.vs[2] * 2;
  auto tile_dma_fast = [&](int j, int U) __attribute__((always_inline)) {
    int keep = 0;
    if (__builtin_expect(j + 3 < ntiles_kv, 1)) {
      if (__builtin_expect(j + 4 < ntiles_kv, 1)) {
        dma_issue(kfast, ld_koff[0], smem_addr + U * STAGE_BYTES + (8 * wave) * ROW_BYTES);
        keep = 4;
      } else {
        keep = 2;
      }
      dma_issue(vfast, ld_voff[0], smem_addr + (KSTAGES + ((U + 3) & 3)) * STAGE_BYTES + (8 * wave) * ROW_BYTES);
    }
    kfast += kfast_step;
    vfast += vfast_step;
    return keep;
  };
  int j = kt0;
  if (nfast_all >= kt0 + 1) {
    auto settle_fast = [&](f32x16& s, u32x8& pv, int masked_kv0, int mask_place) __attribute__((always_inline)) {
      vec8 p[2];
      p_load(pv, p);
      settle_half(s, p, psum_step, masked_kv0, mask_place);
      p_store(pv, p);
    };
    if constexpr (MASKB)  // the mask bytes of the half the first step takes (the steps read those of the halves after it)
      asm volatile(TT_P64_MREAD_FIRST : "+{v[112:119]}"(mring) : [mlds] "v"(mlds), [mlds1] "v"(mlds + 2048) : "memory");
    p_store(pAv, pA);
    p_store(pBv, pB);
    asm volatile(TT_P64_PREFETCH : "+{v[208:239]}"(ring) : "{v[152:155]}"(v_addr), "{v[248:251]}"(k_addr) : "memory");
    // Four tiles per trip so that the stage of a tile is a constant of its statement; the trip may end after any of them.
#define TT_P64_TILE(U)                                                                                  \
    if (__builtin_expect(j >= nfast_all, 0)) break;                                                       \
    {                                                                                                    \
      if constexpr (MASKB) mask_dma(j + 2, U & 1);                                                       \
      const int keep = PAGED ? tile_dma(j) : tile_dma_fast(j, U);                                        \
      /* mk = 1: the tile's exponentials take the causal predicate; kvs = first key of the half whose exponentials   \
         the step takes; kvm = kvs on such a tile, else -1.  As scalar instructions: the compiler's own form of     \
         these selects passes through vector registers. */                                                         \
      int mk = 0, kvs = 64 * j + 32, kvm0 = -1, kvm1 = -1;                                               \
      if constexpr (CAUSAL)                                                                              \
        asm("s_cmp_ge_i32 %3, %4\n\ts_cselect_b32 %0, 1, 0\n\ts_cselect_b32 %1, %5, -1\n\ts_cselect_b32 %2, %6, -1"     \
            : "=&s"(mk), "=&s"(kvm0), "=&s"(kvm1) : "s"(j), "s"(nfast), "s"(kvs), "s"(kvs + 32) : "scc"); \
      if constexpr (kIsBf16 && CAUSAL) TT_P64_RUN_STEP(TT_P64_STEP_BF16_U##U##_K0);                    \
      else if constexpr (CAUSAL) TT_P64_RUN_STEP(TT_P64_STEP_F16_U##U##_K0);                           \
      else if constexpr (MASKB && kIsBf16) TT_P64_RUN_MSTEP(TT_P64_MSTEP_BF16_U##U##_K0);              \
      else if constexpr (MASKB) TT_P64_RUN_MSTEP(TT_P64_MSTEP_F16_U##U##_K0);                          \
      else if constexpr (kIsBf16) TT_P64_RUN_PSTEP(TT_P64_PSTEP_BF16_U##U##_K0);                       \
      else TT_P64_RUN_PSTEP(TT_P64_PSTEP_F16_U##U##_K0);                                               \
      settle_fast(sB, pBv, kvm0, MASKB ? 1 : -1);                                                                      \
      kvs += 32;                                                                                         \
      if constexpr (kIsBf16 && CAUSAL) TT_P64_RUN_STEP(TT_P64_STEP_BF16_U##U##_K1);                    \
      else if constexpr (CAUSAL) TT_P64_RUN_STEP(TT_P64_STEP_F16_U##U##_K1);                           \
      else if constexpr (MASKB && kIsBf16) TT_P64_RUN_MSTEP(TT_P64_MSTEP_BF16_U##U##_K1);              \
      else if constexpr (MASKB) TT_P64_RUN_MSTEP(TT_P64_MSTEP_F16_U##U##_K1);                          \
      else if constexpr (kIsBf16) TT_P64_RUN_PSTEP(TT_P64_PSTEP_BF16_U##U##_K1);                       \
      else TT_P64_RUN_PSTEP(TT_P64_PSTEP_F16_U##U##_K1);                                               \
      settle_fast(sC, pAv, kvm1, MASKB ? 0 : -1);                                                                      \
      dma_wait_and_sync(keep);                                                                           \
      j++;                                                                                               \
    }
    for (;;) {
      TT_P64_TILE(0)
      TT_P64_TILE(1)
      TT_P64_TILE(2)
      TT_P64_TILE(3)
    }
#undef TT_P64_TILE
    // the ring's last requests belong to a step that takes the general form: let them land before the registers are reused
    asm volatile("s_waitcnt lgkmcnt(0)" : "+{v[208:239]}"(ring) : : "memory");
    p_load(pAv, pA);
    p_load(pBv, pB);
  }
  for (; j < ntiles_kv; j++) {
    const int keep = tile_dma(j);
    slow_step(2 * j, pA, sB, sC, pB);
    slow_step(2 * j + 1, pB, sC, sB, pA);
    dma_wait_and_sync(keep);
  }

  if (CAUSAL && part == 0 && two_parts) {
    issue_tiles(1);
    load_q(1);
  }

  if constexpr (SPLIT) {  // a partial result: unnormalised accumulator, the maximum it is relative to, the sum
    const float l_part = l_run + __shfl_xor(l_run, 32);
    int ln;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(ln));
    const int qi = qw0 + (ln & 31);
    if (qi < a.L) {
      float* rec = a.ws + (((long long)(b * a.Hq + h) * a.kv_splits + split) * a.L + qi) * (D + 2);  // 8-byte aligned
#pragma unroll
      for (int db = 0; db < 2; db++)
#pragma unroll
        for (int rg = 0; rg < 4; rg++) {
          float* dst = rec + 32 * db + 8 * rg + 4 * (ln >> 5);
          *(float2*)dst = make_float2(oacc[db][4 * rg], oacc[db][4 * rg + 1]);
          *(float2*)(dst + 2) = make_float2(oacc[db][4 * rg + 2], oacc[db][4 * rg + 3]);
        }
      if ((ln >> 5) == 0) rec[D] = m_use, rec[D + 1] = l_part;
    }
    return;
  }

  // ---- normalise, transpose through LDS, store whole rows -----------------------------------------------------------------
  // A lane holds 4 consecutive head_dim elements per register group of its query row: stored directly, every store
  // instruction would touch 32 rows with 16 bytes each.  Instead each wavefront stages its 32 rows in its 4 KiB of the
  // staging area behind the tile stages and writes them out as whole 128-byte rows.  16-byte chunk c of staged row r sits
  // at chunk slot c ^ (r % 8).
  {
    float l_tot = l_run + __shfl_xor(l_run, 32);
    const float inv = 1.f / l_tot;
    typename TR::vec4 y[2][4];
#pragma unroll
    for (int db = 0; db < 2; db++)
#pragma unroll
      for (int rg = 0; rg < 4; rg++) {
        f32x4 x;
#pragma unroll
        for (int i = 0; i < 4; i++) x[i] = oacc[db][4 * rg + i] * inv;
        y[db][rg] = __builtin_convertvector(x, typename TR::vec4);
      }
    char* tbuf = smem + (KSTAGES + VSTAGES) * STAGE_BYTES + wave * (WM * ROW_BYTES);
    T* obase = (T*)a.out + b * a.os[0] + h * a.os[1];
    // the lane number anew (as asm: the compiler would otherwise keep the values derived from it alive, or spilled,
    // through the whole kernel)
    int ln;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(ln));
    const int rr = ln & 31;
    const int cc = ln & 7;
    const int lho = ln >> 5;
#pragma unroll
    for (int db = 0; db < 2; db++)
#pragma unroll
      for (int rg = 0; rg < 4; rg++)
        *(typename TR::vec4*)(tbuf + rr * ROW_BYTES + (((4 * db + rg) ^ (rr & 7)) << 4) + 8 * lho) = y[db][rg];
    // the reads below fetch what other lanes of the wavefront wrote: keep the compiler from relating them to this lane's
    // own accesses.  The LDS runs a wavefront's instructions in order; nothing else is needed.
    asm volatile("" ::: "memory");
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int row = 8 * i + (ln >> 3);
      vec8 v = *(const vec8*)(tbuf + row * ROW_BYTES + ((cc ^ (row & 7)) << 4));
      const int qi = qw0 + row;
      if (qi < a.L) __builtin_nontemporal_store(v, (vec8*)(obase + qi * a.os[2] + 8 * cc));  // written once, not read here
    }
  }
  }  // part
}

template <typename TR, bool CAUSAL, bool SPLIT, bool MASKB = false>
int launch_v(const KArgs& a, dim3 grid, hipStream_t stream) {
  static hipError_t state[kMaxDevices];
  static bool done[kMaxDevices];
  const hipError_t granted = grant_dynamic_lds((const void*)prefill64_kernel<TR, CAUSAL, SPLIT, MASKB>, LDS_BYTES, state, done);
  if (granted != hipSuccess) return (int)granted;
  hipLaunchKernelGGL((prefill64_kernel<TR, CAUSAL, SPLIT, MASKB>), grid, dim3(NW * 64), LDS_BYTES, stream, a);
  return (int)hipGetLastError();
}

template <typename TR, bool CAUSAL>
int launch_k(const KArgs& a, dim3 grid, hipStream_t stream) {
  if constexpr (!CAUSAL)
    if (a.mask_kind != 0) {  // the host sends only Bool masks the streams can apply (bool_mask_streams_ok)
      if (!bool_mask_streams_ok(a)) return (int)hipErrorInvalidValue;
      return launch_v<TR, false, false, true>(a, grid, stream);
    }
  return a.kv_splits > 1 ? launch_v<TR, CAUSAL, true>(a, grid, stream) : launch_v<TR, CAUSAL, false>(a, grid, stream);
}

}  // namespace

int launch_prefill_d64(const KArgs& args, int dtype, hipStream_t stream) {
  KArgs a = args;
  const int ntile = (a.L + BM - 1) / BM;
  long long nwg = (long long)a.B * a.Hq * (a.causal ? (ntile + 1) / 2 : ntile);
  // Mirror pairs are equal work, so a launch of them ends evenly only when the pairs fill whole rounds of the chip's 256
  // CUs.  Fewer pairs than CUs, or a last round under 90 % full: one row tile per workgroup instead, longest first across
  // all the (batch, kv head) pairs of an XCD (more CUs get one, and the launch ends with short tiles).  Measured at
  // head_dim 128, bf16, against pairs: 128 pairs of 2048 rows +19 %, 224 of 1024 rows +28 %, 320 of 4096 rows +25 %,
  // of 2048 rows +17 %, 640 of 2048 rows +4.5 %, 896 of 2048 rows +4 %, of 16384 rows +4 %; with full rounds -2.5 %
  // to +0.5 % (512 pairs of 1024 / 2048 / 4096 rows, 768 of 4096 rows).
  if (a.kv_splits > 1) {  // split keys: single row tiles whether causal or not
    a.single_tiles = 1;
    nwg = (long long)a.B * a.Hq * ntile;
  } else if (a.causal && ntile > 1) {
    const long long rounds = (nwg + 255) / 256;
    if (nwg < 256 || nwg * 10 < rounds * 256 * 9) {
      a.single_tiles = 1;
      nwg = (long long)a.B * a.Hq * ntile;
    }
  }
  // the kernel's XCD-aware numbering addresses workgroups in groups of 8 (classes of XCDs): round up, the extras return
  {
    const int npair = a.B * a.Hkv;
    const int gq = (npair & 7) == 0 ? 8 : ((npair & 3) == 0 ? 4 : ((npair & 1) == 0 ? 2 : 1));
    const long long per_class = nwg / gq;                       // work items of one class of XCDs
    const long long slots = (per_class + 8 / gq - 1) / (8 / gq);  // per XCD of the class
    nwg = slots * 8;
  }
  if (a.kv_splits > 1) nwg *= a.kv_splits;
  dim3 grid((unsigned)nwg);
  int rc;
  if (dtype == 1) rc = a.causal ? launch_k<F16, true>(a, grid, stream) : launch_k<F16, false>(a, grid, stream);
  else rc = a.causal ? launch_k<BF16, true>(a, grid, stream) : launch_k<BF16, false>(a, grid, stream);
  if (rc != 0 || a.kv_splits <= 1) return rc;
  return launch_prefill_split_merge<D>(a, dtype, stream);
}

}  // namespace ttsdpa
