// The linear layer y = x . w^T + bias on gfx950 (reference: op::matmul(input, weight, false, true, bias) behind
// function::linear, src/Function/FuncNNLayer.h:14-19; device GEMM src/Operation/OpLinalgCuda.cuh:239-293).
//
// linear_mfma_kernel (fp16 / bf16 on v_mfma_f32_32x32x16, fp32 on v_mfma_f32_32x32x2 with full fp32 products): a workgroup of 8 wavefronts owns a 256 x 256 tile of the output and walks K in
// steps of 128 bytes (64 or 32 elements).  Both operands have K contiguous ("NT"), which is the layout v_mfma_f32_32x32x16 wants for both inputs:
// a lane supplies 8 consecutive k of one row, so operand fragments are plain 16-byte LDS reads, no transposes.
//   global -> LDS   global_load_lds_dwordx4, two stages of 64 KB (x tile 256 x 64, w tile 256 x 64); the 16-byte chunks
//                   of a 128-byte LDS row are XOR-swizzled with half the row number so that the 32 rows a fragment read
//                   touches spread over the banks; the loads for tile t+2 are requested while tile t's last k-step
//                   runs, one barrier per tile
//   MFMA            the wavefront's 64 (n) x 128 (m) part is computed transposed, A = w rows, B = x rows, so that an
//                   accumulator register group holds 4 consecutive n of one m: the output is stored as 8-byte pieces
//                   along its contiguous axis without a transpose
//   accumulators    start from the bias (the reference writes the bias into C and accumulates onto it), fp32
// Workgroups are numbered so that the 32 that run together on one XCD (workgroup i runs on XCD i % 8) form a 4 x 8
// block of tiles: they share their x and w panels through that XCD's L2.
//
// linear_general_kernel: any element type and shape, fp32 arithmetic on the vector ALUs (64 x 64 tiles).

#include <type_traits>
#include "../../include/ttlinear.h"
#include "sdpa_common.h"

namespace ttsdpa {
namespace {

struct LinArgs {
  const void* x;
  const void* w;
  const void* bias;
  void* out;
  long long M, N, K, ldx, ldw, ldo;
  // general kernel only: x is stored [K, M] (x(m,k) = x[k*ldx + m]) / w is stored [K, N] (w(n,k) = w[k*ldw + n])
  int xt = 0, wt = 0;
  // batch entries of one launch (linear_mfma_kernel: blockIdx.y, linear_general_kernel: blockIdx.z): entry e reads
  // x + e*bsx, w + e*bsw and writes out + e*bso (elements; 0 = the operand is shared by all entries)
  long long bsx = 0, bsw = 0, bso = 0;
};

typedef __attribute__((address_space(3))) void lds_void_t;

constexpr int ROWB = 128;  // bytes of an LDS row: 64 k of a 16-bit type, 32 k of fp32

// What the kernel needs to know about the element type.  A fragment is the 16 bytes a lane reads per 32 x 32 block and
// k-step: 8 consecutive k (16-bit: one v_mfma_f32_32x32x16) or 4 (fp32: four v_mfma_f32_32x32x2, MFMA e contracting the
// lanes' e-th elements — lanes 0-31 hold k .. k+3, lanes 32-63 k+4 .. k+7, the same pairing for both operands).
template <typename TR>
struct Gemm {
  typedef typename TR::elem elem;
  typedef typename TR::vec8 frag;
  typedef typename TR::vec4 out4;
  static constexpr int KPC = 8;  // elements per 16-byte chunk
  static __device__ __forceinline__ f32x16 mma(frag a, frag b, f32x16 c) { return TR::mfma32(a, b, c); }
  static __device__ __forceinline__ out4 cvt(f32x4 v) { return __builtin_convertvector(v, out4); }
};
struct F32 {};
template <>
struct Gemm<F32> {
  typedef float elem;
  typedef f32x4 frag;
  typedef f32x4 out4;
  static constexpr int KPC = 4;
  static __device__ __forceinline__ f32x16 mma(frag a, frag b, f32x16 c) {
#pragma unroll
    for (int e = 0; e < 4; e++) c = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], b[e], c, 0, 0, 0);
    return c;
  }
  static __device__ __forceinline__ out4 cvt(f32x4 v) { return v; }
};

// TM x TN: the workgroup's output tile, 256 x 256 (two stages of 64 KB) or 128 x 128 for problems with too few large
// tiles to fill the chip.
// WN x WM wavefronts share the tile: a wavefront's part is (TN/WN n) x (TM/WM m).
template <typename TR, int TM, int TN, int WN, int WM>
__global__ __launch_bounds__(WN * WM * 64, 1) void linear_mfma_kernel(LinArgs a) {
  constexpr int NW = WN * WM;
  constexpr int XTILE = TM * ROWB;
  constexpr int STAGE = (TM + TN) * ROWB;
  constexpr int XI = TM / NW / 8, WI = TN / NW / 8;  // load instructions per wavefront and tile
  constexpr int NI = TN / WN / 32, MJ = TM / WM / 32;  // 32 x 32 blocks of a wavefront's part
  typedef Gemm<TR> G;
  typedef typename G::elem T;
  typedef typename G::frag vec8;  // the 16-byte operand fragment
  constexpr int BK = (ROWB / 16) * G::KPC;  // k per tile
  constexpr int ESZ = 16 / G::KPC;
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lq = lane & 31, lh = lane >> 5;

  // ---- workgroup -> tile: 4 x 8 tile blocks per XCD ---------------------------------------------------------------
  const int tiles_m = (int)((a.M + TM - 1) / TM), tiles_n = (int)((a.N + TN - 1) / TN);
  const int super_n = (tiles_n + 7) / 8;
  const int nsuper = ((tiles_m + 3) / 4) * super_n;
  const int slot = blockIdx.x >> 3;
  const int super = (slot >> 5) * 8 + (blockIdx.x & 7);
  if (super >= nsuper) return;
  const int tm = (super / super_n) * 4 + ((slot & 31) >> 3);
  const int tn = (super % super_n) * 8 + (slot & 7);
  if (tm >= tiles_m || tn >= tiles_n) return;
  const long long m0 = (long long)tm * TM, n0 = (long long)tn * TN;

  // ---- global -> LDS: wavefront w moves rows (TM/8)w .. of the x tile and (TN/8)w .. of the w tile, 8 rows (1 KB) per instruction
  // lane l fills (row l/8, chunk slot l%8) and therefore fetches chunk (l%8) ^ ((row / 2) % 8) — two rows share 256
  // bytes of LDS, so 16 consecutive rows of one logical chunk land in 16 different bank groups; rows past the end of the
  // matrix re-read its last row (their products land in outputs that are not stored)
  // The byte offset of a lane's chunk is recomputed per request (a handful of vector-ALU operations against the 2048+
  // MFMA cycles of a tile) rather than held in registers for every row group.
  const long long mlim = a.M - 1 - m0, nlim = a.N - 1 - n0;  // last valid row of the tiles
  auto lane_off = [&](int row, long long lim, long long ld) __attribute__((always_inline)) {
    const int chunk = (lane & 7) ^ ((row >> 1) & 7);
    const long long r = row < lim ? row : lim;
    return (unsigned)((r * ld + G::KPC * chunk) * ESZ);
  };
  const char* xbase = (const char*)((const T*)a.x + (long long)blockIdx.y * a.bsx + m0 * a.ldx);
  const char* wbase = (const char*)((const T*)a.w + (long long)blockIdx.y * a.bsw + n0 * a.ldw);
  const unsigned smem_addr = (unsigned)(unsigned long)(lds_void_t*)smem;
  // issued as asm so that the compiler does not treat it as an LDS store it must order every later LDS read behind
  // (the lane's full address goes in a register pair: a scalar base operand is not always kept in scalar registers by
  // the compiler once the tile requests are unrolled)
  auto dma_issue = [&](const char* sbase, unsigned voff, unsigned lds_addr) __attribute__((always_inline)) {
    const char* p = sbase + voff;
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(p), "s"(lds_addr) : "memory", "m0");
  };
  auto dma_tile = [&](int t, int stage) __attribute__((always_inline)) {
    const char* xs = xbase + (long long)t * ROWB;
    const char* ws = wbase + (long long)t * ROWB;
    const unsigned dst = smem_addr + stage * STAGE;
#pragma unroll
    for (int i = 0; i < XI; i++) {
      const int row = (TM / NW) * wave + 8 * i + (lane >> 3);
      dma_issue(xs, lane_off(row, mlim, a.ldx), dst + ((TM / NW) * wave + 8 * i) * ROWB);
    }
#pragma unroll
    for (int i = 0; i < WI; i++) {
      const int row = (TN / NW) * wave + 8 * i + (lane >> 3);
      dma_issue(ws, lane_off(row, nlim, a.ldw), dst + XTILE + ((TN / NW) * wave + 8 * i) * ROWB);
    }
  };

  // ---- this wavefront's part: n rows (TN/4)*wn .. of the w tile (A operand), m rows (TM/2)*wm .. of the x tile (B) ---------
  const int wn = wave % WN, wm = wave / WN;
  // fragment (block, ks): row 32*block + lq, chunk 2*ks + lh at row*128 + 16 * (chunk ^ ((row/2) % 8)); (row/2) % 8 == (lq/2) % 8
  const unsigned frag = (unsigned)(lq * ROWB + 16 * (lh ^ ((lq >> 1) & 7)));
  const unsigned wfrag = XTILE + ((TN / WN) * wn) * ROWB + frag;
  const unsigned xfrag = ((TM / WM) * wm) * ROWB + frag;

  f32x16 acc[NI][MJ];
#pragma unroll
  for (int i = 0; i < NI; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const long long n = n0 + (TN / WN) * wn + 32 * i + 8 * (r >> 2) + 4 * lh + (r & 3);
      const float b = (a.bias && n < a.N) ? (float)((const T*)a.bias)[n] : 0.f;
#pragma unroll
      for (int j = 0; j < MJ; j++) acc[i][j][r] = b;
    }

  // Operand fragments are double-buffered in registers: while the MFMAs of k-step ks run, the fragments of ks+1 are
  // on their way from LDS.  The one barrier per tile sits before the MFMAs of a tile's last k-step: by then every
  // wavefront has taken its last fragment of tile t (its stage may be overwritten: tile t+2 is requested) and its own
  // loads of tile t+1 have landed (requested a tile earlier), so right after the barrier the first fragments of tile
  // t+1 are requested and arrive while the last 8 MFMAs of tile t run.
  vec8 fw[2][NI], fx[2][MJ];
  auto load_frag = [&](int buf, const char* st, int ks) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < NI; i++) fw[buf][i] = *(const vec8*)(st + ((wfrag + 32 * i * ROWB) ^ (unsigned)(32 * ks)));
#pragma unroll
    for (int j = 0; j < MJ; j++) fx[buf][j] = *(const vec8*)(st + ((xfrag + 32 * j * ROWB) ^ (unsigned)(32 * ks)));
  };
  auto mma = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < NI; i++)
#pragma unroll
      for (int j = 0; j < MJ; j++) acc[i][j] = G::mma(fw[buf][i], fx[buf][j], acc[i][j]);
  };

  const int ntk = (int)(a.K / BK);
  if (ntk > 0) {
    dma_tile(0, 0);
    if (ntk > 1) {
      dma_tile(1, 1);
      // tile 0's loads; tile 1's XI + WI may still be in flight
      if constexpr (XI + WI == 8) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
      else asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
      static_assert(XI + WI == 8 || XI + WI == 4, "add the matching wait");
    } else {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    load_frag(0, smem, 0);
  }
  for (int t = 0; t < ntk; t++) {
    const char* st = smem + (t & 1) * STAGE;
    load_frag(1, st, 1);
    mma(0);
    __builtin_amdgcn_sched_barrier(0);
    load_frag(0, st, 2);
    mma(1);
    __builtin_amdgcn_sched_barrier(0);
    load_frag(1, st, 3);
    mma(0);
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (t + 2 < ntk) dma_tile(t + 2, t & 1);
    if (t + 1 < ntk) load_frag(0, smem + ((t + 1) & 1) * STAGE, 0);
    mma(1);
    __builtin_amdgcn_sched_barrier(0);
  }

  // ---- store: register group rg of acc[i][j] is out[m = .. + 32j + lq][n = .. + 32i + 8rg + 4lh .. +3] ----------------------
#pragma unroll
  for (int j = 0; j < MJ; j++) {
    const long long m = m0 + (TM / WM) * wm + 32 * j + lq;
    if (m >= a.M) continue;
    T* orow = (T*)a.out + (long long)blockIdx.y * a.bso + m * a.ldo;
#pragma unroll
    for (int i = 0; i < NI; i++)
#pragma unroll
      for (int rg = 0; rg < 4; rg++) {
        const long long n = n0 + (TN / WN) * wn + 32 * i + 8 * rg + 4 * lh;
        if (n < a.N) {  // N is a multiple of 4 on this route
          f32x4 v;
#pragma unroll
          for (int e = 0; e < 4; e++) v[e] = acc[i][j][4 * rg + e];
          *(typename G::out4*)(orow + n) = G::cvt(v);
        }
      }
  }
}

// ---- 16-bit tensors with an operand stored contraction-major (op::matmul's other transpose flags) -------------------------
// out[m][n] = sum_k x(m,k) w(n,k) + bias[n] with x(m,k) = XT ? x[k*ldx + m] : x[m*ldx + k] and w(n,k) = WT ? w[k*ldw + n] :
// w[n*ldw + k]: the operands of op::matmul(a, b, transA, transB) as they lie in memory (reference
// src/Operation/OpLinalg.cpp:107-150 hands its flags to the GEMM; no transposed copy is made here either).
// Same tiles, workgroup order, stages and pipeline as linear_mfma_kernel.  What differs is the tile of a contraction-major
// operand and how fragments are read:
//  * such a tile is 64 k-rows of its 128 or 256 columns, kept as sub-tiles of 128 columns (64 rows x 256 bytes, the
//    layout of the attention kernels' V tile: 16-byte chunk c of row r at slot c ^ f(r), f(r) = (r%4)*4 + (r/4)%4), and a
//    fragment of it comes through the LDS transpose load: two ds_read_b64_tr_b16 give a lane the k values
//    {4h..4h+3} and {8+4h..8+4h+3} of a 16-k step for its row (h = lane/32);
//  * the contraction index has to be permuted identically on both sides, so a row-major operand's fragment is read in
//    the same order, as two 8-byte pieces (chunks 2ks and 2ks+1 of the k-step, bytes 8h..8h+7 of each).
namespace lint {
__device__ __forceinline__ int swz(int row) { return ((row & 3) << 2) | ((row >> 2) & 3); }
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
}  // namespace lint

template <typename TR, int TM, int TN, bool XT, bool WT>
__global__ __launch_bounds__(512, 1) void linear_mfma_t_kernel(LinArgs a) {
  static_assert(XT || WT, "both operands row-major: linear_mfma_kernel");
  constexpr int WN = 4, WM = 2, NW = 8;
  constexpr int XTILE = TM * ROWB, STAGE = (TM + TN) * ROWB;  // bytes: 64 k of 2 bytes per row or column, either layout
  constexpr int XI = TM / NW / 8, WI = TN / NW / 8;           // load instructions per wavefront and tile, either layout
  constexpr int NI = TN / WN / 32, MJ = TM / WM / 32;
  constexpr int BK = 64, SUB = 64 * 256;                      // k per tile; bytes of a 128-column sub-tile
  typedef typename TR::elem T;
  typedef typename TR::vec8 vec8;
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lq = lane & 31, lh = lane >> 5;

  // workgroup -> tile: 4 x 8 tile blocks per XCD, as in linear_mfma_kernel
  const int tiles_m = (int)((a.M + TM - 1) / TM), tiles_n = (int)((a.N + TN - 1) / TN);
  const int super_n = (tiles_n + 7) / 8;
  const int nsuper = ((tiles_m + 3) / 4) * super_n;
  const int slot = blockIdx.x >> 3;
  const int super = (slot >> 5) * 8 + (blockIdx.x & 7);
  if (super >= nsuper) return;
  const int tm = (super / super_n) * 4 + ((slot & 31) >> 3);
  const int tn = (super % super_n) * 8 + (slot & 7);
  if (tm >= tiles_m || tn >= tiles_n) return;
  const long long m0 = (long long)tm * TM, n0 = (long long)tn * TN;

  // ---- global -> LDS -------------------------------------------------------------------------------------------------------
  // row-major operand: wavefront w moves rows (T/8)w .. of the tile, 8 rows (1 KB) per instruction, lane l fills (row l/8,
  // chunk slot l%8) with chunk (l%8) ^ ((row/2) % 8); rows past the end re-read the last row.
  // contraction-major operand: wavefront w moves k-rows 8w .. 8w+7 of every 128-column sub-tile, 4 rows (1 KB) per
  // instruction, lane l fills (row l/16, chunk slot l%16) with chunk (l%16) ^ f(row); columns past the end re-read the
  // last 8 valid ones (their products land in outputs that are not stored).
  const long long mlim = a.M - 1 - m0, nlim = a.N - 1 - n0;
  auto rm_off = [&](int row, long long lim, long long ld) __attribute__((always_inline)) {
    const int chunk = (lane & 7) ^ ((row >> 1) & 7);
    const long long r = row < lim ? row : lim;
    return (unsigned)((r * ld + 8 * chunk) * 2);
  };
  auto km_off = [&](int row, int sub, long long cols_left, long long ld) __attribute__((always_inline)) {  // cols_left: valid columns from the tile's first
    const int chunk = (lane & 15) ^ lint::swz(row);
    long long col = 128 * sub + 8 * chunk;
    col = col + 8 <= cols_left ? col : cols_left - 8;
    return (unsigned)(((long long)row * ld + col) * 2);
  };
  const T* xb = (const T*)a.x + (long long)blockIdx.y * a.bsx;
  const T* wb = (const T*)a.w + (long long)blockIdx.y * a.bsw;
  const char* xbase = (const char*)(XT ? xb + m0 : xb + m0 * a.ldx);
  const char* wbase = (const char*)(WT ? wb + n0 : wb + n0 * a.ldw);
  const unsigned smem_addr = (unsigned)(unsigned long)(lds_void_t*)smem;
  auto dma_issue = [&](const char* sbase, unsigned voff, unsigned lds_addr) __attribute__((always_inline)) {
    const char* p = sbase + voff;
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(p), "s"(lds_addr) : "memory", "m0");
  };
  auto dma_operand = [&](bool km, const char* base, long long ld, long long lim, int T_, int NINSTR, long long t, unsigned dst) __attribute__((always_inline)) {
    if (km) {
      const char* src = base + t * BK * ld * 2;  // 64 k-rows further
#pragma unroll
      for (int i = 0; i < NINSTR; i++) {
        const int sub = i >> 1, row = 8 * wave + 4 * (i & 1) + (lane >> 4);
        dma_issue(src, km_off(row, sub, lim + 1, ld), dst + sub * SUB + (8 * wave + 4 * (i & 1)) * 256);
      }
    } else {
      const char* src = base + t * ROWB;
#pragma unroll
      for (int i = 0; i < NINSTR; i++) {
        const int row = (T_ / NW) * wave + 8 * i + (lane >> 3);
        dma_issue(src, rm_off(row, lim, ld), dst + ((T_ / NW) * wave + 8 * i) * ROWB);
      }
    }
  };
  auto dma_tile = [&](int t, int stage) __attribute__((always_inline)) {
    const unsigned dst = smem_addr + stage * STAGE;
    dma_operand(XT, xbase, a.ldx, mlim, TM, XI, t, dst);
    dma_operand(WT, wbase, a.ldw, nlim, TN, WI, t, dst + XTILE);
  };

  // ---- fragments ---------------------------------------------------------------------------------------------------------------
  const int wn = wave % WN, wm = wave / WN;
  // row-major: (block, ks, piece p): row 32*block + lq, bytes 8lh .. 8lh+7 of chunk 2ks + p
  const unsigned rm_base = (unsigned)(lq * ROWB + 8 * lh + 16 * ((lq >> 1) & 7));
  // contraction-major: piece ld of k-step ks for the 32 columns 32*db .. of a sub-tile (see sdpa_prefill_d128.hip, V operand)
  unsigned km_base[2];
  {
    const int s = lane & 15, dhalf = (lane >> 4) & 1;
#pragma unroll
    for (int ld = 0; ld < 2; ld++) {
      const int row = 8 * ld + 4 * lh + (s >> 2);
      const int chunk = 2 * dhalf + ((s & 3) >> 1);
      km_base[ld] = (unsigned)(row * 256 + 16 * (chunk ^ lint::swz(row)) + 8 * (s & 1));
    }
  }
  // fragment of the 32 rows / columns starting at `first` of an operand's tile at `region`, k-step ks
  auto frag_of = [&](bool km, const char* region, int first, int ks) __attribute__((always_inline)) {
    if (km) {
      const char* sub = region + (first >> 7) * SUB + 16 * ks * 256;
      const unsigned db = (unsigned)((first & 127) >> 5);
      const lint::s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lint::lds_s16x4*)(sub + (km_base[0] ^ (64u * db))));
      const lint::s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lint::lds_s16x4*)(sub + (km_base[1] ^ (64u * db))));
      return __builtin_bit_cast(vec8, (lint::s16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    } else {
      const char* rows = region + first * ROWB;
      const lint::s16x4 lo = *(const lint::s16x4*)(rows + (rm_base ^ (unsigned)(32 * ks)));
      const lint::s16x4 hi = *(const lint::s16x4*)(rows + (rm_base ^ (unsigned)(32 * ks + 16)));
      return __builtin_bit_cast(vec8, (lint::s16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    }
  };

  f32x16 acc[NI][MJ];
#pragma unroll
  for (int i = 0; i < NI; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const long long n = n0 + (TN / WN) * wn + 32 * i + 8 * (r >> 2) + 4 * lh + (r & 3);
      const float b = (a.bias && n < a.N) ? (float)((const T*)a.bias)[n] : 0.f;
#pragma unroll
      for (int j = 0; j < MJ; j++) acc[i][j][r] = b;
    }

  vec8 fw[2][NI], fx[2][MJ];
  auto load_frag = [&](int buf, const char* st, int ks) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < NI; i++) fw[buf][i] = frag_of(WT, st + XTILE, (TN / WN) * wn + 32 * i, ks);
#pragma unroll
    for (int j = 0; j < MJ; j++) fx[buf][j] = frag_of(XT, st, (TM / WM) * wm + 32 * j, ks);
  };
  auto mma = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < NI; i++)
#pragma unroll
      for (int j = 0; j < MJ; j++) acc[i][j] = TR::mfma32(fw[buf][i], fx[buf][j], acc[i][j]);
  };

  // the pipeline of linear_mfma_kernel: fragments double-buffered in registers, one barrier per tile before its last k-step
  const int ntk = (int)(a.K / BK);
  if (ntk > 0) {
    dma_tile(0, 0);
    if (ntk > 1) {
      dma_tile(1, 1);
      if constexpr (XI + WI == 8) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
      else asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
      static_assert(XI + WI == 8 || XI + WI == 4, "add the matching wait");
    } else {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    load_frag(0, smem, 0);
  }
  for (int t = 0; t < ntk; t++) {
    const char* st = smem + (t & 1) * STAGE;
    load_frag(1, st, 1);
    mma(0);
    __builtin_amdgcn_sched_barrier(0);
    load_frag(0, st, 2);
    mma(1);
    __builtin_amdgcn_sched_barrier(0);
    load_frag(1, st, 3);
    mma(0);
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (t + 2 < ntk) dma_tile(t + 2, t & 1);
    if (t + 1 < ntk) load_frag(0, smem + ((t + 1) & 1) * STAGE, 0);
    mma(1);
    __builtin_amdgcn_sched_barrier(0);
  }

  // store: register group rg of acc[i][j] is out[m = .. + 32j + lq][n = .. + 32i + 8rg + 4lh .. +3]
#pragma unroll
  for (int j = 0; j < MJ; j++) {
    const long long m = m0 + (TM / WM) * wm + 32 * j + lq;
    if (m >= a.M) continue;
    T* orow = (T*)a.out + (long long)blockIdx.y * a.bso + m * a.ldo;
#pragma unroll
    for (int i = 0; i < NI; i++)
#pragma unroll
      for (int rg = 0; rg < 4; rg++) {
        const long long n = n0 + (TN / WN) * wn + 32 * i + 8 * rg + 4 * lh;
        if (n < a.N) {  // N is a multiple of 4 on this route
          f32x4 v;
#pragma unroll
          for (int e = 0; e < 4; e++) v[e] = acc[i][j][4 * rg + e];
          *(typename TR::vec4*)(orow + n) = __builtin_convertvector(v, typename TR::vec4);
        }
      }
  }
}

// ---- 16-bit tensors, 256 x 256 tiles: four wavefronts with 128 x 128 each and the tile's arithmetic as one hand-ordered stream
// Same tiles, LDS layout and direct loads as linear_mfma_kernel<TR, 256, 256>; what differs is who owns what, the matrix
// instruction and who orders the instructions.  The clock of these kernels is power-managed, so what a tile costs is
// energy rather than issue slots:
//  * a wavefront owns 128 x 128 of the tile (256 accumulator registers, in AGPRs: one wavefront per SIMD), so an operand
//    read from LDS feeds eight matrix instructions — LDS operand traffic is the second consumer after the matrix pipe;
//  * v_mfma_f32_16x16x32 instead of 32x32x16: with random operands the chip sustains 2.10 against 1.84 PFLOP/s of them;
//  * the body of a tile (accumulators from the bias, K loop, conversion into LDS) is a single asm statement
//    (linear256_loop.inc, written by gen_linear256_loop.py): the compiler's version of the loop requested the operands
//    of a k-step in one burst behind the matrix instructions and waited for them before the next, and put the tile
//    loads and the next operands between the barrier and the matrix instructions behind it;
//  * the output leaves through LDS as whole lines: written 8 bytes at a time the tile's stores took 16 % of the kernel
//    (every instruction touched 32 rows, 16 bytes each; the L2 takes a request per piece).
#include "linear256_loop.inc"

typedef unsigned u32x8 __attribute__((ext_vector_type(8)));

template <typename TR>
struct Lin256Body;
template <>
struct Lin256Body<BF16> {
  static __device__ __forceinline__ void run(f32x16 bias_lo, f32x16 bias_hi, u32x8 xoff, u32x8 woff, u32x4 raddr, u32x8 eaddr,
                                             unsigned long long xp, unsigned long long wp, unsigned m0base, unsigned left, unsigned adv) {
#define TT_LIN256_TEXT TT_LIN256_BODY_BF16
#include "linear256_stmt.inc"
#undef TT_LIN256_TEXT
  }
};
template <>
struct Lin256Body<F16> {
  static __device__ __forceinline__ void run(f32x16 bias_lo, f32x16 bias_hi, u32x8 xoff, u32x8 woff, u32x4 raddr, u32x8 eaddr,
                                             unsigned long long xp, unsigned long long wp, unsigned m0base, unsigned left, unsigned adv) {
#define TT_LIN256_TEXT TT_LIN256_BODY_F16
#include "linear256_stmt.inc"
#undef TT_LIN256_TEXT
  }
};

template <typename TR>
__global__ __launch_bounds__(256, 1) void linear256_kernel(LinArgs a) {
  constexpr int TM = 256, TN = 256;
  constexpr int XTILE = TM * ROWB;
  constexpr int STAGE = (TM + TN) * ROWB;
  typedef typename TR::elem T;
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lr = lane & 15, lg = lane >> 4;

  // workgroup -> tile: 4 x 8 tile blocks per XCD, as in linear_mfma_kernel
  const int tiles_m = (int)((a.M + TM - 1) / TM), tiles_n = (int)((a.N + TN - 1) / TN);
  const int super_n = (tiles_n + 7) / 8;
  const int nsuper = ((tiles_m + 3) / 4) * super_n;
  const int slot = blockIdx.x >> 3;
  const int super = (slot >> 5) * 8 + (blockIdx.x & 7);
  if (super >= nsuper) return;
  const int tm = (super / super_n) * 4 + ((slot & 31) >> 3);
  const int tn = (super % super_n) * 8 + (slot & 7);
  if (tm >= tiles_m || tn >= tiles_n) return;
  const long long m0 = (long long)tm * TM, n0 = (long long)tn * TN;

  // global -> LDS: wavefront v moves rows 64v .. 64v+63 of both tiles, 8 rows (1 KB) per instruction; lane l fills
  // (row l/8, chunk slot l%8) and fetches chunk (l%8) ^ ((row/2) % 8); rows past the end re-read the last row
  const long long mlim = a.M - 1 - m0, nlim = a.N - 1 - n0;
  u32x8 xoff, woff;
#pragma unroll
  for (int i = 0; i < 8; i++) {
    const int row = 64 * wave + 8 * i + (lane >> 3);
    const int chunk = (lane & 7) ^ ((row >> 1) & 7);
    xoff[i] = (unsigned)(((row < mlim ? row : mlim) * a.ldx + 8 * chunk) * 2);
    woff[i] = (unsigned)(((row < nlim ? row : nlim) * a.ldw + 8 * chunk) * 2);
  }
  // (the 64-bit products are formed on the vector ALUs; the loads want their base in scalar registers)
  auto uniform = [](const void* p) __attribute__((always_inline)) {
    const unsigned long long v = (unsigned long long)p;
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)v), hi = __builtin_amdgcn_readfirstlane((unsigned)(v >> 32));
    return (const char*)(((unsigned long long)hi << 32) | lo);
  };
  const char* xbase = uniform((const T*)a.x + m0 * a.ldx);
  const char* wbase = uniform((const T*)a.w + n0 * a.ldw);
  const unsigned smem_addr = (unsigned)(unsigned long)(lds_void_t*)smem;
  auto dma_tile = [&](long long t, int stage) __attribute__((always_inline)) {
    const char* xs = xbase + t * ROWB;
    const char* ws = wbase + t * ROWB;
    const unsigned dst = smem_addr + stage * STAGE + wave * 8192;
#pragma unroll
    for (int i = 0; i < 8; i++)
      asm volatile("s_mov_b32 m0, %2\n\ts_nop 3\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(xoff[i]), "s"(xs), "s"(dst + 1024 * i) : "memory", "m0");
#pragma unroll
    for (int i = 0; i < 8; i++)
      asm volatile("s_mov_b32 m0, %2\n\ts_nop 3\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(woff[i]), "s"(ws), "s"(dst + XTILE + 1024 * i) : "memory", "m0");
  };

  // this wavefront's part: n rows 128*wn .. of the w tile (A operand), m rows 128*wm .. of the x tile (B operand);
  // operand (block, s): row 16*block + lane%16, chunk 4*s + lane/16 at row*128 + 16 * (chunk ^ ((row/2) % 8))
  const int wn = wave & 1, wm = wave >> 1;
  const unsigned frag = (unsigned)(lr * ROWB + 16 * (lg ^ ((lr >> 1) & 7)));
  u32x4 raddr;
#pragma unroll
  for (int s = 0; s < 2; s++) {
    raddr[2 * s] = smem_addr + ((128 * wm * ROWB + frag) ^ (unsigned)(64 * s));
    raddr[2 * s + 1] = smem_addr + ((128 * wn * ROWB + frag) ^ (unsigned)(64 * s));
  }
  // block (i, j) leaves the lane with out[m = .. + 16j + lane%16][n = .. + 16i + 4(lane/16) .. +3]: 8 bytes of row 16j + lane%16
  // of the wavefront's quarter of LDS (rows of 256 bytes, the 16-byte chunks of row r at slot c ^ (r % 16))
  u32x8 eaddr;
#pragma unroll
  for (int i = 0; i < 8; i++) eaddr[i] = smem_addr + wave * 32768 + lr * 256 + 16 * ((2 * i + (lg >> 1)) ^ lr) + 8 * (lg & 1);
  // accumulators start from the bias (the reference writes the bias into C and accumulates onto it)
  f32x16 bias_lo, bias_hi;
#pragma unroll
  for (int i = 0; i < 8; i++)
#pragma unroll
    for (int e = 0; e < 4; e++) {
      const long long n = n0 + 128 * wn + 16 * i + 4 * lg + e;
      const float b = (a.bias && n < a.N) ? (float)((const T*)a.bias)[n] : 0.f;
      if (i < 4) bias_lo[4 * i + e] = b;
      else bias_hi[4 * (i - 4) + e] = b;
    }

  const long long ntk = a.K / 64;  // > 0 on this route
  dma_tile(0, 0);
  if (ntk > 1) {
    dma_tile(1, 1);
    asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
  } else {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  {
    // the loop's loads: k-tile min(t + 2, ntk - 1) while k-tile t is computed
    const long long first = ntk > 2 ? 2 : ntk - 1;
    Lin256Body<TR>::run(bias_lo, bias_hi, xoff, woff, raddr, eaddr, (unsigned long long)(xbase + first * ROWB),
                        (unsigned long long)(wbase + first * ROWB), smem_addr + wave * 8192, (unsigned)ntk,
                        ntk > 3 ? (unsigned)(ntk - 3) : 0u);
  }

  // 16 lanes read a row of the wavefront's quarter back and store its 256 bytes (a wavefront reads only what it wrote)
  const char* mine = smem + wave * 32768;
  const long long nbase = n0 + 128 * wn;
#pragma unroll 8
  for (int it = 0; it < 32; it++) {
    const int row = 4 * it + (lane >> 4);
    const int c = (lane & 15) ^ (row & 15);
    const u32x4 v = *(const u32x4*)(mine + row * 256 + 16 * (lane & 15));
    const long long m = m0 + 128 * wm + row, n = nbase + 8 * c;
    if (m < a.M) {
      T* dst = (T*)a.out + m * a.ldo + n;
      if (n + 8 <= a.N) {
        *(u32x4*)dst = v;
      } else if (n + 4 <= a.N) {  // N is a multiple of 4 on this route
        *(u32x2*)dst = u32x2{v[0], v[1]};
      }
    }
  }
}

// ---- few rows of x (a decode step's projections: M = the batch): the weight is read once at HBM speed ------------------
// With M <= 64 the layer is a stream over w (N*K elements) against 64 rows of x that stay in L2: a workgroup owns 32
// output columns and all rows of x; its four wavefronts take the 64-element k-blocks in turn (wavefront v: blocks v,
// v+4, ...) and add their partial sums through LDS at the end.  Every wavefront has a ring of three k-blocks of its own in
// LDS, filled by direct global->LDS loads (eight lanes fetch the 128 bytes of a row's k-block: whole cache lines) and
// read back as MFMA operands, 16-byte chunk c of row r at slot c ^ ((r/2) % 8) (conflict-free b128 reads).  No
// barriers inside the stream: a ring belongs to one wavefront.  out^T[n][m] accumulates with w as the A operand, so a
// lane ends up with four consecutive n of one row m: 8-byte stores.
template <int MB, int NB>
struct Skinny {
  static constexpr int WT = NB * 32 * 128;             // bytes of a weight tile: NB x 32 rows x 64 k
  static constexpr int STG = WT + MB * 32 * 128;       // ... plus the x tile
  static constexpr int NST = 4 * 3 * STG <= 160 * 1024 ? 3 : 2;  // k-blocks of a wavefront in LDS (what fits the CU's 160 KiB)
  static constexpr int LPB = 4 * NB + 4 * MB;          // load instructions per k-block
  static constexpr int LDS = 4 * NST * STG;
  static_assert(LDS >= 3 * MB * NB * 16 * 64 * 4, "the partial sums of three wavefronts reuse the rings");
};

// MB = 32-row blocks of x: 1 (M <= 32) or 2 (M <= 64).  NB = 32-column blocks of the output a workgroup owns: every x
// tile a wavefront fetches (from L2) serves NB weight tiles (from memory), so the bytes a CU takes in per weight byte
// fall from 1 + MB to 1 + MB / NB.  At M = 64 the kernel with NB = 1 is bound by what the L2s deliver (three bytes per
// weight byte).
template <typename TR, int MB, int NB>
__global__ __launch_bounds__(256) void linear_skinny_kernel(LinArgs a) {
  typedef typename TR::elem T;
  typedef typename TR::vec8 vec8;
  typedef Skinny<MB, NB> SK;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lq = lane & 31, lh = lane >> 5;
  const long long n0 = (long long)blockIdx.x * (32 * NB);
  char* ring = smem + wave * SK::NST * SK::STG;
  const unsigned ring_addr = (unsigned)(unsigned long)(lds_void_t*)ring;

  auto dma16 = [&](const char* sbase, unsigned voff, unsigned lds_addr) __attribute__((always_inline)) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 3\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(sbase), "s"(lds_addr) : "memory", "m0");
  };
  // this lane's part of a load instruction: row 8i + lane/8 of a tile, slot lane%8
  unsigned woff[NB][4], xoff[MB][4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int row = 8 * i + (lane >> 3);
    const unsigned chunk = (unsigned)((lane & 7) ^ ((row >> 1) & 7));
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
      const long long n = n0 + 32 * nb + row;  // columns past the end re-read the last weight row (not stored)
      woff[nb][i] = (unsigned)(((n < a.N ? n - n0 : a.N - 1 - n0) * a.ldw + 8 * chunk) * 2);
    }
#pragma unroll
    for (int mb = 0; mb < MB; mb++) {
      const int m = 32 * mb + row;
      xoff[mb][i] = (unsigned)(((m < a.M ? m : (int)(a.M - 1)) * a.ldx + 8 * chunk) * 2);
    }
  }
  const char* wbase = (const char*)((const T*)a.w + n0 * a.ldw);
  const char* xbase = (const char*)a.x;
  auto issue = [&](long long kb, int stage) __attribute__((always_inline)) {
    const unsigned at = ring_addr + stage * SK::STG;
    const char* wk = wbase + kb * 128;
    const char* xk = xbase + kb * 128;
#pragma unroll
    for (int nb = 0; nb < NB; nb++)
#pragma unroll
      for (int i = 0; i < 4; i++) dma16(wk, woff[nb][i], at + (32 * nb + 8 * i) * 128);
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
      for (int i = 0; i < 4; i++) dma16(xk, xoff[mb][i], at + SK::WT + (32 * mb + 8 * i) * 128);
  };
  // operand (j): row lq, chunk 4*lh + j
  unsigned rd[4];
#pragma unroll
  for (int j = 0; j < 4; j++) rd[j] = (unsigned)(lq * 128 + 16 * ((4 * lh + j) ^ ((lq >> 1) & 7)));

  f32x16 acc[NB][MB];
#pragma unroll
  for (int nb = 0; nb < NB; nb++)
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[nb][mb][r] = 0.f;
  const long long nkb = a.K / 64;
  const long long nb_ = nkb > wave ? (nkb - wave + 3) / 4 : 0;  // k-blocks of this wavefront: wave, wave + 4, ...
  constexpr int AHEAD = SK::NST - 1;                             // k-blocks in flight beyond the one in use
  for (int t = 0; t < AHEAD; t++)
    if (nb_ > t) issue(wave + 4 * t, t);
  int cur = 0;
  for (long long t = 0; t < nb_; t++) {
    const int nxt = cur == 0 ? SK::NST - 1 : cur - 1;  // (t + AHEAD) % NST
    if (t + AHEAD < nb_) issue(wave + 4 * (t + AHEAD), nxt);
    // block t has landed when only the loads of the blocks issued after it are outstanding
    const long long later = nb_ - 1 - t < AHEAD ? nb_ - 1 - t : AHEAD;
    if (later == 2) {
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * SK::LPB) : "memory");
    } else if (later == 1) {
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(SK::LPB) : "memory");
    } else {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    const char* wt = ring + cur * SK::STG;
    const char* xt = wt + SK::WT;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      vec8 xv[MB];
#pragma unroll
      for (int mb = 0; mb < MB; mb++) xv[mb] = *(const vec8*)(xt + mb * 32 * 128 + rd[j]);
#pragma unroll
      for (int nb = 0; nb < NB; nb++) {
        const vec8 wv = *(const vec8*)(wt + nb * 32 * 128 + rd[j]);
#pragma unroll
        for (int mb = 0; mb < MB; mb++) acc[nb][mb] = TR::mfma32(wv, xv[mb], acc[nb][mb]);
      }
    }
    cur = cur == SK::NST - 1 ? 0 : cur + 1;
  }
  __syncthreads();  // every ring is drained: the partial sums of wavefronts 1-3 take their place
  float* part = (float*)smem;
  if (wave > 0) {
#pragma unroll
    for (int nb = 0; nb < NB; nb++)
#pragma unroll
      for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int r = 0; r < 16; r++) part[((((wave - 1) * NB + nb) * MB + mb) * 16 + r) * 64 + lane] = acc[nb][mb][r];
  }
  __syncthreads();
  if (wave != 0) return;
#pragma unroll
  for (int nb = 0; nb < NB; nb++)
#pragma unroll
    for (int mb = 0; mb < MB; mb++) {
      const long long m = 32 * mb + lq;
#pragma unroll
      for (int rg = 0; rg < 4; rg++) {
        const long long n = n0 + 32 * nb + 8 * rg + 4 * lh;
        f32x4 v;
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const int r = 4 * rg + i;
          float sum = acc[nb][mb][r];
#pragma unroll
          for (int w = 0; w < 3; w++) sum += part[(((w * NB + nb) * MB + mb) * 16 + r) * 64 + lane];
          if (a.bias && n + i < a.N) sum += load_as_float((const T*)a.bias + n + i);
          v[i] = sum;
        }
        if (m < a.M && n < a.N) {  // N is a multiple of 4 on this route: a group of four is inside or outside
          *(typename TR::vec4*)((T*)a.out + m * a.ldo + n) = __builtin_convertvector(v, typename TR::vec4);
        }
      }
    }
}

template <typename TR, int MB, int NB>
int launch_skinny_mb(const LinArgs& a, hipStream_t stream) {
  static hipError_t state[kMaxDevices];
  static bool done[kMaxDevices];
  constexpr int lds = Skinny<MB, NB>::LDS;
  const hipError_t granted = grant_dynamic_lds((const void*)linear_skinny_kernel<TR, MB, NB>, lds, state, done);
  if (granted != hipSuccess) return (int)granted;
  const long long nwg = (a.N + 32 * NB - 1) / (32 * NB);
  if (nwg > 0x7fffffffLL) return TTSDPA_ERR_SHAPE;
  hipLaunchKernelGGL((linear_skinny_kernel<TR, MB, NB>), dim3((unsigned)nwg), dim3(256), lds, stream, a);
  return (int)hipGetLastError();
}

// Two column blocks per workgroup once they still make a workgroup per CU (N >= 16384).  Weights beyond the last-level
// cache, bf16, K = 4096: N = 28672 (an MLP's up projection) 3.9 -> 4.4 TB/s at M <= 8, 3.4 -> 4.3 at M = 32, 2.8 -> 3.5 at
// M = 64; N = 6144 and 4096 (96 and 64 workgroups then) 3.0 -> 2.7 and 2.7 -> 2.4: those keep one block.
template <typename TR>
int launch_skinny(const LinArgs& a, hipStream_t stream) {
  if (a.N >= 16384) return a.M <= 32 ? launch_skinny_mb<TR, 1, 2>(a, stream) : launch_skinny_mb<TR, 2, 2>(a, stream);
  return a.M <= 32 ? launch_skinny_mb<TR, 1, 1>(a, stream) : launch_skinny_mb<TR, 2, 1>(a, stream);
}

// Any element type and shape: 64 x 64 output tile per workgroup, 4 x 4 outputs per lane, K in steps of 16 through LDS.
template <typename T>
__global__ __launch_bounds__(256) void linear_general_kernel(LinArgs a) {
  __shared__ float Xs[16][64 + 1], Ws[16][64 + 1];
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;
  const long long m0 = (long long)blockIdx.y * 64, n0 = (long long)blockIdx.x * 64;
  const T* x = (const T*)a.x + (long long)blockIdx.z * a.bsx;
  const T* w = (const T*)a.w + (long long)blockIdx.z * a.bsw;
  float acc[4][4];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const long long n = n0 + 4 * tx + j;
    const float b = (a.bias && n < a.N) ? load_as_float((const T*)a.bias + n) : 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++) acc[i][j] = b;
  }
  for (long long k0 = 0; k0 < a.K; k0 += 16) {
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int e = tid + 256 * i;
      const int row = e >> 4, kk = e & 15;
      const bool kin = k0 + kk < a.K;
      const long long xat = a.xt ? (k0 + kk) * a.ldx + m0 + row : (m0 + row) * a.ldx + k0 + kk;
      const long long wat = a.wt ? (k0 + kk) * a.ldw + n0 + row : (n0 + row) * a.ldw + k0 + kk;
      Xs[kk][row] = (kin && m0 + row < a.M) ? load_as_float(x + xat) : 0.f;
      Ws[kk][row] = (kin && n0 + row < a.N) ? load_as_float(w + wat) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 16; kk++) {
      float xv[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; i++) xv[i] = Xs[kk][4 * ty + i], wv[i] = Ws[kk][4 * tx + i];
#pragma unroll
      for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = fmaf(xv[i], wv[j], acc[i][j]);
    }
  }
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const long long m = m0 + 4 * ty + i;
    if (m >= a.M) continue;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const long long n = n0 + 4 * tx + j;
      if (n < a.N) store_from_float((T*)a.out + (long long)blockIdx.z * a.bso + m * a.ldo + n, acc[i][j]);
    }
  }
}

// dst[c, r] = src[r, c] for src [R, C] with row stride ld; dst dense [C, R].  64 x 64 tiles through LDS, 16 bytes per
// global access where the row lengths allow it (VECOK: ld and R multiples of 16 bytes, both pointers 16-byte aligned).
template <typename T, bool VECOK>
__global__ __launch_bounds__(256) void transpose_kernel(const T* src, T* dst, long long R, long long C, long long ld) {
  constexpr int VEC = 16 / sizeof(T);
  constexpr int PITCH = 64 + VEC;  // rows stay 16-byte aligned
  typedef T vecT __attribute__((ext_vector_type(VEC)));
  __shared__ __attribute__((aligned(16))) T tile[64][PITCH];
  const long long r0 = (long long)blockIdx.y * 64, c0 = (long long)blockIdx.x * 64;
  constexpr int CPR = 64 / VEC;  // 16-byte chunks per tile row
#pragma unroll
  for (int i = 0; i < 64 * CPR / 256; i++) {
    const int chunk = threadIdx.x + 256 * i;
    const int row = chunk / CPR, cc = (chunk % CPR) * VEC;
    const long long r = r0 + row, c = c0 + cc;
    if (r >= R) continue;
    if (VECOK && c + VEC <= C) {
      *(vecT*)&tile[row][cc] = *(const vecT*)(src + r * ld + c);
    } else {
#pragma unroll
      for (int e = 0; e < VEC; e++)
        if (c + e < C) tile[row][cc + e] = src[r * ld + c + e];
    }
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 64 * CPR / 256; i++) {
    const int chunk = threadIdx.x + 256 * i;
    const int orow = chunk / CPR, oc = (chunk % CPR) * VEC;  // output row = source column; first of VEC source rows
    const long long c = c0 + orow, r = r0 + oc;
    if (c >= C) continue;
    if (VECOK && r + VEC <= R) {
      vecT v;
#pragma unroll
      for (int e = 0; e < VEC; e++) v[e] = tile[oc + e][orow];
      *(vecT*)(dst + c * R + r) = v;
    } else {
#pragma unroll
      for (int e = 0; e < VEC; e++)
        if (r + e < R) dst[c * R + r + e] = tile[oc + e][orow];
    }
  }
}

template <typename T>
int launch_transpose(const void* src, void* dst, long long R, long long C, long long ld, hipStream_t stream) {
  if ((R + 63) / 64 > 65535 || (C + 63) / 64 > 0x7fffffffLL) return TTSDPA_ERR_SHAPE;
  dim3 grid((unsigned)((C + 63) / 64), (unsigned)((R + 63) / 64));
  constexpr long long VEC = 16 / sizeof(T);
  const bool vecok = ld % VEC == 0 && R % VEC == 0 && ((uintptr_t)src % 16) == 0 && ((uintptr_t)dst % 16) == 0;
  if (vecok) {
    hipLaunchKernelGGL((transpose_kernel<T, true>), grid, dim3(256), 0, stream, (const T*)src, (T*)dst, R, C, ld);
  } else {
    hipLaunchKernelGGL((transpose_kernel<T, false>), grid, dim3(256), 0, stream, (const T*)src, (T*)dst, R, C, ld);
  }
  return (int)hipGetLastError();
}

bool aligned(const void* p, size_t n) { return ((uintptr_t)p % n) == 0; }

int check(int dtype, const void* x, const void* w, const void* out, long long M, long long N, long long K, long long ldx,
          long long ldw, long long ldo, int* route) {
  if (dtype != TTSDPA_F32 && dtype != TTSDPA_F16 && dtype != TTSDPA_BF16) return TTSDPA_ERR_DTYPE;
  if (M < 0 || N < 0 || K < 0) return TTSDPA_ERR_SHAPE;
  *route = TTLINEAR_ROUTE_NONE;
  if (M == 0 || N == 0) return TTSDPA_OK;
  if (!out || (K > 0 && (!x || !w))) return TTSDPA_ERR_NULL;
  if (ldx < K || ldw < K || ldo < N) return TTSDPA_ERR_STRIDE;
  const size_t esz = dtype == TTSDPA_F32 ? 4 : 2;
  if (!aligned(x, esz) || !aligned(w, esz) || !aligned(out, esz)) return TTSDPA_ERR_STRIDE;
  if ((M + 63) / 64 > 65535 || (N + 63) / 64 > 0x7fffffffLL) return TTSDPA_ERR_SHAPE;
  const long long kpc = 16 / (long long)esz;  // elements per 16 bytes
  const bool mfma = K > 0 && K % (8 * kpc) == 0 && N % 4 == 0 && ldx % kpc == 0 && ldw % kpc == 0 && ldo % 4 == 0 &&
                    aligned(x, 16) && aligned(w, 16) && aligned(out, 4 * esz) &&
                    ldx < (1 << 21) && ldw < (1 << 21);  // 256 rows are addressed with 32-bit byte offsets
  *route = mfma ? TTLINEAR_ROUTE_MFMA : TTLINEAR_ROUTE_GENERAL;
  return TTSDPA_OK;
}

template <typename TR, int TM, int TN, int WN, int WM>
int launch_mfma_tile(const LinArgs& a, hipStream_t stream, unsigned entries = 1) {
  constexpr int lds = 2 * (TM + TN) * ROWB;
  static hipError_t state[kMaxDevices];
  static bool done[kMaxDevices];
  const hipError_t granted = grant_dynamic_lds((const void*)linear_mfma_kernel<TR, TM, TN, WN, WM>, lds, state, done);
  if (granted != hipSuccess) return (int)granted;
  const long long tiles_m = (a.M + TM - 1) / TM, tiles_n = (a.N + TN - 1) / TN;
  const long long nsuper = ((tiles_m + 3) / 4) * ((tiles_n + 7) / 8);
  const long long nwg = (nsuper + 7) / 8 * 8 * 32;
  if (nwg > 0x7fffffffLL) return TTSDPA_ERR_SHAPE;
  hipLaunchKernelGGL((linear_mfma_kernel<TR, TM, TN, WN, WM>), dim3((unsigned)nwg, entries), dim3(WN * WM * 64), lds, stream, a);
  return (int)hipGetLastError();
}

template <typename TR, int T_, bool XT, bool WT>
int launch_mfma_t_tile(const LinArgs& a, hipStream_t stream) {
  constexpr int lds = 2 * (T_ + T_) * ROWB;
  static hipError_t state[kMaxDevices];
  static bool done[kMaxDevices];
  const hipError_t granted = grant_dynamic_lds((const void*)linear_mfma_t_kernel<TR, T_, T_, XT, WT>, lds, state, done);
  if (granted != hipSuccess) return (int)granted;
  const long long tiles_m = (a.M + T_ - 1) / T_, tiles_n = (a.N + T_ - 1) / T_;
  const long long nsuper = ((tiles_m + 3) / 4) * ((tiles_n + 7) / 8);
  const long long nwg = (nsuper + 7) / 8 * 8 * 32;
  if (nwg > 0x7fffffffLL) return TTSDPA_ERR_SHAPE;
  hipLaunchKernelGGL((linear_mfma_t_kernel<TR, T_, T_, XT, WT>), dim3((unsigned)nwg), dim3(512), lds, stream, a);
  return (int)hipGetLastError();
}

// 16-bit operands read as they lie in memory (a.xt / a.wt: stored contraction-major)
template <typename TR>
int launch_mfma_t(const LinArgs& a, hipStream_t stream) {
  // 256 x 256 tiles once they fill the chip, unless their last round over the 256 CUs would be under 85 % full: then four
  // times as many 128 x 128 tiles (weight gradient of the QKV projection, 384 large tiles: 878 -> 936 TFLOP/s; its input
  // gradient, 512 large tiles, runs 1063 against 795 on the small ones)
  const long long n256 = ((a.M + 255) / 256) * ((a.N + 255) / 256);
  const bool big = n256 >= 256 && n256 * 100 >= (n256 + 255) / 256 * 256 * 85;
  if (a.xt && a.wt) return big ? launch_mfma_t_tile<TR, 256, true, true>(a, stream) : launch_mfma_t_tile<TR, 128, true, true>(a, stream);
  if (a.xt) return big ? launch_mfma_t_tile<TR, 256, true, false>(a, stream) : launch_mfma_t_tile<TR, 128, true, false>(a, stream);
  return big ? launch_mfma_t_tile<TR, 256, false, true>(a, stream) : launch_mfma_t_tile<TR, 128, false, true>(a, stream);
}

template <typename TR>
int launch_linear256(const LinArgs& a, hipStream_t stream) {
  constexpr int lds = 2 * (256 + 256) * ROWB;
  static hipError_t state[kMaxDevices];
  static bool done[kMaxDevices];
  const hipError_t granted = grant_dynamic_lds((const void*)linear256_kernel<TR>, lds, state, done);
  if (granted != hipSuccess) return (int)granted;
  const long long tiles_m = (a.M + 255) / 256, tiles_n = (a.N + 255) / 256;
  const long long nsuper = ((tiles_m + 3) / 4) * ((tiles_n + 7) / 8);
  const long long nwg = (nsuper + 7) / 8 * 8 * 32;
  if (nwg > 0x7fffffffLL) return TTSDPA_ERR_SHAPE;
  hipLaunchKernelGGL((linear256_kernel<TR>), dim3((unsigned)nwg), dim3(256), lds, stream, a);
  return (int)hipGetLastError();
}

template <typename TR>
int launch_mfma(const LinArgs& a, hipStream_t stream) {
  // 256 x 256 tiles once they fill the 256 CUs; smaller problems get four times as many 128 x 128 tiles
  const long long big = ((a.M + 255) / 256) * ((a.N + 255) / 256);
  // (four wavefronts with 128 x 128 each — accumulators in AGPRs, half the LDS operand reads — measured 2-10 % slower
  // than eight with 64 x 128: one wavefront per SIMD hides too little)
  if constexpr (!std::is_same<TR, F32>::value) {
    // 16-bit tensors: the hand-ordered kernel
    // and it stores 16 bytes at a time
    if (big >= 256 && a.ldo % 8 == 0 && ((uintptr_t)a.out & 15) == 0) return launch_linear256<TR>(a, stream);
  }
  return big >= 256 ? launch_mfma_tile<TR, 256, 256, 4, 2>(a, stream) : launch_mfma_tile<TR, 128, 128, 4, 2>(a, stream);
}

template <typename T>
int launch_general_linear(const LinArgs& a, hipStream_t stream, unsigned entries = 1) {
  dim3 grid((unsigned)((a.N + 63) / 64), (unsigned)((a.M + 63) / 64), entries);
  hipLaunchKernelGGL((linear_general_kernel<T>), grid, dim3(256), 0, stream, a);
  return (int)hipGetLastError();
}

}  // namespace
}  // namespace ttsdpa

using namespace ttsdpa;

extern "C" {

int ttlinear_plan(int dtype, const void* x, const void* w, const void* bias, const void* out, int64_t M, int64_t N,
                  int64_t K, int64_t ldx, int64_t ldw, int64_t ldo, int* route) {
  (void)bias;
  int r = TTLINEAR_ROUTE_NONE;
  const int rc = check(dtype, x, w, out, M, N, K, ldx, ldw, ldo, &r);
  if (rc == TTSDPA_OK && route) *route = r;
  return rc;
}

int ttlinear_forward(int dtype, const void* x, const void* w, const void* bias, void* out, int64_t M, int64_t N,
                     int64_t K, int64_t ldx, int64_t ldw, int64_t ldo, void* stream) {
  int route = TTLINEAR_ROUTE_NONE;
  const int rc = check(dtype, x, w, out, M, N, K, ldx, ldw, ldo, &route);
  if (rc != TTSDPA_OK || route == TTLINEAR_ROUTE_NONE) return rc;
  const size_t esz = dtype == TTSDPA_F32 ? 4 : 2;
  if (bias && !aligned(bias, esz)) return TTSDPA_ERR_STRIDE;
  LinArgs a{x, w, bias, out, M, N, K, ldx, ldw, ldo};
  hipStream_t s = (hipStream_t)stream;
  if (route == TTLINEAR_ROUTE_MFMA) {
    // a handful of rows (a decode step): stream the weight once instead of tiling for reuse
    if (dtype != TTSDPA_F32 && M <= 64 && N >= 64) return dtype == TTSDPA_F16 ? launch_skinny<F16>(a, s) : launch_skinny<BF16>(a, s);
    return dtype == TTSDPA_F32 ? launch_mfma<F32>(a, s) : dtype == TTSDPA_F16 ? launch_mfma<F16>(a, s) : launch_mfma<BF16>(a, s);
  }
  switch (dtype) {
    case TTSDPA_F32: return launch_general_linear<float>(a, s);
    case TTSDPA_F16: return launch_general_linear<_Float16>(a, s);
    default: return launch_general_linear<__bf16>(a, s);
  }
}

// Bytes of the dense transposed copies the MFMA route of ttlinear_matmul makes: a as [M, K] when it is stored [K, M],
// b as [N, K] when it is stored [K, N]; each rounded up to 256 bytes.
static size_t matmul_copy_bytes(int dtype, int64_t rows, int64_t K) {
  const size_t esz = dtype == TTSDPA_F32 ? 4 : 2;
  return ((size_t)rows * (size_t)K * esz + 255) / 256 * 256;
}

size_t ttlinear_matmul_workspace_bytes(int dtype, int64_t M, int64_t N, int64_t K, int trans_a, int trans_b) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  return (trans_a ? matmul_copy_bytes(dtype, M, K) : 0) + (!trans_b ? matmul_copy_bytes(dtype, N, K) : 0);
}

int ttlinear_matmul(int dtype, const void* a, const void* b, const void* bias, void* out, int64_t M, int64_t N, int64_t K,
                    int trans_a, int trans_b, int64_t lda, int64_t ldb, int64_t ldo, void* workspace,
                    size_t workspace_bytes, void* stream) {
  if (!trans_a && trans_b) return ttlinear_forward(dtype, a, b, bias, out, M, N, K, lda, ldb, ldo, stream);
  if (dtype != TTSDPA_F32 && dtype != TTSDPA_F16 && dtype != TTSDPA_BF16) return TTSDPA_ERR_DTYPE;
  if (M < 0 || N < 0 || K < 0) return TTSDPA_ERR_SHAPE;
  if (M == 0 || N == 0) return TTSDPA_OK;
  if (!out || (K > 0 && (!a || !b))) return TTSDPA_ERR_NULL;
  if (lda < (trans_a ? M : K) || ldb < (trans_b ? K : N) || ldo < N) return TTSDPA_ERR_STRIDE;
  const size_t esz = dtype == TTSDPA_F32 ? 4 : 2;
  if (!aligned(a, esz) || !aligned(b, esz) || !aligned(out, esz) || (bias && !aligned(bias, esz))) return TTSDPA_ERR_STRIDE;
  if ((M + 63) / 64 > 65535 || (N + 63) / 64 > 0x7fffffffLL) return TTSDPA_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;

  // 16-bit tensors: the matrix-core kernel that reads contraction-major operands in place (no copies, no scratch)
  if (dtype != TTSDPA_F32 && K > 0 && K % 64 == 0 && N % 4 == 0 && ldo % 4 == 0 && aligned(out, 8)) {
    auto in_place = [](const void* p, bool contraction_major, int64_t rows, int64_t ld) {
      if (!aligned(p, 16) || ld % 8 != 0) return false;
      // a tile's rows are addressed with 32-bit byte offsets: 64 k-rows of a contraction-major operand, 256 rows otherwise
      return contraction_major ? (rows % 8 == 0 && ld < (1 << 24)) : ld < (1 << 21);
    };
    if (in_place(a, trans_a, M, lda) && in_place(b, !trans_b, N, ldb)) {
      LinArgs g{a, b, bias, out, M, N, K, lda, ldb, ldo, trans_a ? 1 : 0, trans_b ? 0 : 1};
      return dtype == TTSDPA_F16 ? launch_mfma_t<F16>(g, s) : launch_mfma_t<BF16>(g, s);
    }
  }

  // MFMA route: dense row-major copies of the operands that are stored contraction-major, then the x . w^T kernel
  const size_t need = ttlinear_matmul_workspace_bytes(dtype, M, N, K, trans_a, trans_b);
  if (K > 0 && workspace && workspace_bytes >= need && aligned(workspace, 256)) {
    const void* x = a;
    const void* w = b;
    long long ldx = lda, ldw = ldb;
    char* ws = (char*)workspace;
    int route = TTLINEAR_ROUTE_NONE;
    const void* xprobe = trans_a ? (const void*)ws : a;
    const void* wprobe = !trans_b ? (const void*)(ws + (trans_a ? matmul_copy_bytes(dtype, M, K) : 0)) : b;
    if (check(dtype, xprobe, wprobe, out, M, N, K, trans_a ? K : lda, !trans_b ? K : ldb, ldo, &route) == TTSDPA_OK &&
        route == TTLINEAR_ROUTE_MFMA) {
      int rc = 0;
      if (trans_a) {  // a is [K, M]
        rc = dtype == TTSDPA_F32 ? launch_transpose<float>(a, ws, K, M, lda, s) : launch_transpose<uint16_t>(a, ws, K, M, lda, s);
        if (rc != 0) return rc;
        x = ws, ldx = K;
        ws += matmul_copy_bytes(dtype, M, K);
      }
      if (!trans_b) {  // b is [K, N]
        rc = dtype == TTSDPA_F32 ? launch_transpose<float>(b, ws, K, N, ldb, s) : launch_transpose<uint16_t>(b, ws, K, N, ldb, s);
        if (rc != 0) return rc;
        w = ws, ldw = K;
      }
      return ttlinear_forward(dtype, x, w, bias, out, M, N, K, ldx, ldw, ldo, stream);
    }
  }
  LinArgs g{a, b, bias, out, M, N, K, lda, ldb, ldo, trans_a ? 1 : 0, trans_b ? 0 : 1};
  switch (dtype) {
    case TTSDPA_F32: return launch_general_linear<float>(g, s);
    case TTSDPA_F16: return launch_general_linear<_Float16>(g, s);
    default: return launch_general_linear<__bf16>(g, s);
  }
}

int ttlinear_matmul_batched(int dtype, const void* a, const void* b, const void* bias, void* out, int64_t M, int64_t N,
                            int64_t K, int trans_a, int trans_b, int64_t lda, int64_t ldb, int64_t ldo, int nbatch_dims,
                            const int64_t* batch_shape, const int64_t* a_batch_stride, const int64_t* b_batch_stride,
                            int64_t out_batch_stride, void* workspace, size_t workspace_bytes, void* stream) {
  if (dtype != TTSDPA_F32 && dtype != TTSDPA_F16 && dtype != TTSDPA_BF16) return TTSDPA_ERR_DTYPE;
  if (nbatch_dims < 0 || nbatch_dims > TTLINEAR_MAX_BATCH_DIMS) return TTSDPA_ERR_SHAPE;
  if (nbatch_dims > 0 && (!batch_shape || !a_batch_stride || !b_batch_stride)) return TTSDPA_ERR_NULL;
  long long entries = 1;
  for (int d = 0; d < nbatch_dims; d++) {
    if (batch_shape[d] < 0 || a_batch_stride[d] < 0 || b_batch_stride[d] < 0) return TTSDPA_ERR_SHAPE;
    entries *= batch_shape[d];
  }
  if (out_batch_stride < 0) return TTSDPA_ERR_STRIDE;
  const size_t esz = dtype == TTSDPA_F32 ? 4 : 2;
  auto offsets = [&](long long i, long long* ao, long long* bo) {
    // offsets of entry i: the reference's index walk from the innermost batch dimension outwards
    long long rest = i;
    *ao = 0, *bo = 0;
    for (int d = nbatch_dims - 1; d >= 0; d--) {
      const long long idx = rest % batch_shape[d];
      rest /= batch_shape[d];
      *ao += idx * a_batch_stride[d];
      *bo += idx * b_batch_stride[d];
    }
  };
  // One grid for all entries (the reference's strided-batched product, src/Operation/OpLinalg.cpp:113-150) when the
  // entries' offsets are a multiple of the entry index in both operands (no broadcast pattern that breaks the stride)
  // and an entry is small enough that a launch each would be launch-bound; x . w^T on the tiled matrix-core kernel when
  // the layout allows, every other flag pair on the vector-ALU kernel, which reads the operands in place.
  if (entries > 1 && entries <= 65535 && M > 0 && N > 0 && K > 0 && a && b && out && (double)M * N * K <= (double)(1 << 27)) {
    long long sa = 0, sb = 0;
    offsets(1, &sa, &sb);
    bool uniform = true;
    for (long long i = 2; i < entries && uniform; i++) {
      long long ao, bo;
      offsets(i, &ao, &bo);
      uniform = ao == i * sa && bo == i * sb;
    }
    if (uniform && lda >= (trans_a ? M : K) && ldb >= (trans_b ? K : N) && ldo >= N && aligned(a, esz) && aligned(b, esz) &&
        aligned(out, esz) && (!bias || aligned(bias, esz)) && (M + 63) / 64 <= 65535) {
      hipStream_t s = (hipStream_t)stream;
      LinArgs g{a, b, bias, out, M, N, K, lda, ldb, ldo, trans_a ? 1 : 0, trans_b ? 0 : 1};
      g.bsx = sa, g.bsw = sb, g.bso = out_batch_stride;
      int route = TTLINEAR_ROUTE_NONE;
      const long long kpc = 16 / (long long)esz;
      if (!trans_a && trans_b && check(dtype, a, b, out, M, N, K, lda, ldb, ldo, &route) == TTSDPA_OK && route == TTLINEAR_ROUTE_MFMA &&
          sa % kpc == 0 && sb % kpc == 0 && out_batch_stride % 4 == 0 && !(dtype != TTSDPA_F32 && M <= 64 && N >= 64)) {
        g.xt = g.wt = 0;
        switch (dtype) {
          case TTSDPA_F32: return launch_mfma_tile<F32, 128, 128, 4, 2>(g, s, (unsigned)entries);
          case TTSDPA_F16: return launch_mfma_tile<F16, 128, 128, 4, 2>(g, s, (unsigned)entries);
          default: return launch_mfma_tile<BF16, 128, 128, 4, 2>(g, s, (unsigned)entries);
        }
      }
      switch (dtype) {
        case TTSDPA_F32: return launch_general_linear<float>(g, s, (unsigned)entries);
        case TTSDPA_F16: return launch_general_linear<_Float16>(g, s, (unsigned)entries);
        default: return launch_general_linear<__bf16>(g, s, (unsigned)entries);
      }
    }
  }
  for (long long i = 0; i < entries; i++) {
    // offsets of entry i: the reference's index walk from the innermost batch dimension outwards
    long long ao = 0, bo = 0, rest = i;
    for (int d = nbatch_dims - 1; d >= 0; d--) {
      const long long idx = rest % batch_shape[d];
      rest /= batch_shape[d];
      ao += idx * a_batch_stride[d];
      bo += idx * b_batch_stride[d];
    }
    const int rc = ttlinear_matmul(dtype, a ? (const char*)a + ao * esz : nullptr, b ? (const char*)b + bo * esz : nullptr, bias,
                                   out ? (char*)out + i * out_batch_stride * esz : nullptr, M, N, K, trans_a, trans_b, lda, ldb,
                                   ldo, workspace, workspace_bytes, stream);
    if (rc != 0) return rc;
  }
  return TTSDPA_OK;
}

}  // extern "C"
