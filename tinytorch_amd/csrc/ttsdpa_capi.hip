// C ABI of the attention library (declarations and contract: include/ttsdpa.h).
// Validates a call, picks the kernel family, and enqueues it on the caller's stream.  Nothing here allocates device
// memory, synchronises, throws or aborts.

#include <math.h>
#include <string.h>

#include "../../include/ttsdpa.h"
#include "sdpa_common.h"

using namespace ttsdpa;

namespace {

bool dense_last_ok(const int64_t* st, int align) { return st[0] % align == 0 && st[1] % align == 0 && st[2] % align == 0; }

bool ptr_aligned(const void* p, size_t a) { return ((uintptr_t)p % a) == 0; }

// The causal mode a call reduces to.  Bottom-right alignment with one query row hides nothing; without per-batch key
// counts and with S <= L its offset is 0, which is the top-left aligned mask.
int effective_causal(const ttsdpa_params* p) {
  if (p->causal != TTSDPA_CAUSAL_BOTTOM_RIGHT) return p->causal;
  if (p->L == 1) return TTSDPA_CAUSAL_NONE;
  if (!p->kv_len && p->S <= p->L) return TTSDPA_CAUSAL_TOP_LEFT;
  return TTSDPA_CAUSAL_BOTTOM_RIGHT;
}

// Groups of four consecutive keys of the mask (starting at multiples of 4) can be read with one aligned load.
bool mask_vec4_ok(const ttsdpa_params* p) {
  if (p->mask_kind != TTSDPA_MASK_BOOL && p->mask_kind != TTSDPA_MASK_ADD) return false;
  const size_t mesz = p->mask_kind == TTSDPA_MASK_BOOL ? 1 : (p->dtype == TTSDPA_F32 ? 4 : 2);
  return p->mask_stride[3] == 1 && p->mask_stride[0] % 4 == 0 && p->mask_stride[1] % 4 == 0 && p->mask_stride[2] % 4 == 0 &&
         ptr_aligned(p->mask, 4 * mesz);
}

// Validation shared by every entry point; fills the kernel argument block.
int validate(const ttsdpa_params* p, KArgs* a) {
  if (!p) return TTSDPA_ERR_NULL;
  if (p->struct_size != sizeof(ttsdpa_params)) return TTSDPA_ERR_ABI;
  if (p->dtype != TTSDPA_F32 && p->dtype != TTSDPA_F16 && p->dtype != TTSDPA_BF16) return TTSDPA_ERR_DTYPE;
  if (p->B < 0 || p->Hq < 1 || p->Hkv < 1 || p->L < 0 || p->S < 0 || p->D < 1 || p->D > 256) return TTSDPA_ERR_SHAPE;
  if (p->Hq % p->Hkv != 0) return TTSDPA_ERR_SHAPE;
  if (p->mask_kind < TTSDPA_MASK_NONE || p->mask_kind > TTSDPA_MASK_ADD) return TTSDPA_ERR_MASK;
  if (p->causal < TTSDPA_CAUSAL_NONE || p->causal > TTSDPA_CAUSAL_BOTTOM_RIGHT) return TTSDPA_ERR_MASK;
  if (p->mask_kind != TTSDPA_MASK_NONE && p->causal) return TTSDPA_ERR_MASK;  // reference FuncNNLayer.h:242
  const bool empty_out = p->B == 0 || p->L == 0;
  if (!empty_out) {
    if (!p->q || !p->out) return TTSDPA_ERR_NULL;
    if (p->S > 0 && (!p->k || !p->v)) return TTSDPA_ERR_NULL;
    if (p->mask_kind != TTSDPA_MASK_NONE && !p->mask) return TTSDPA_ERR_NULL;
  }
  for (int i = 0; i < 3; i++) {
    if (p->q_stride[i] < 0 || p->k_stride[i] < 0 || p->v_stride[i] < 0 || p->o_stride[i] < 0) return TTSDPA_ERR_STRIDE;
  }
  if (p->q_stride[2] < p->D && p->L > 1) return TTSDPA_ERR_STRIDE;
  if (p->o_stride[2] < p->D && p->L > 1) return TTSDPA_ERR_STRIDE;
  if ((p->k_stride[2] < p->D || p->v_stride[2] < p->D) && p->S > 1) return TTSDPA_ERR_STRIDE;
  const size_t esz = p->dtype == TTSDPA_F32 ? 4 : 2;
  if (!ptr_aligned(p->q, esz) || !ptr_aligned(p->k, esz) || !ptr_aligned(p->v, esz) || !ptr_aligned(p->out, esz))
    return TTSDPA_ERR_STRIDE;
  for (int i = 0; i < 4; i++) {
    if (p->mask_kind != TTSDPA_MASK_NONE && p->mask_stride[i] < 0) return TTSDPA_ERR_STRIDE;
    a->ms[i] = p->mask_kind != TTSDPA_MASK_NONE ? p->mask_stride[i] : 0;
  }
  if (p->mask_kind == TTSDPA_MASK_ADD && !ptr_aligned(p->mask, esz)) return TTSDPA_ERR_STRIDE;
  a->mask_vec4 = mask_vec4_ok(p) ? 1 : 0;
  a->single_tiles = 0;
  a->pack_L = 0, a->kv_splits = 1, a->kv_chunk = 0, a->ws = nullptr;
  if (p->kv_len && !ptr_aligned(p->kv_len, 4)) return TTSDPA_ERR_STRIDE;
  a->kv_len = p->kv_len;
  a->block_table = p->block_table, a->page_shift = 0, a->bt_stride = p->block_table_stride;
  if (p->block_table) {
    if (!ptr_aligned(p->block_table, 4) || p->block_table_stride < 0) return TTSDPA_ERR_STRIDE;
    if (p->page_size < 1 || (p->page_size & (p->page_size - 1)) != 0) return TTSDPA_ERR_SHAPE;
    while ((1 << a->page_shift) < p->page_size) a->page_shift++;
    if ((long long)p->block_table_stride * p->page_size < p->S && p->B > 1) return TTSDPA_ERR_STRIDE;  // tables would overlap
  }
  a->q = p->q, a->k = p->k, a->v = p->v, a->out = p->out, a->mask = p->mask;
  a->B = p->B, a->Hq = p->Hq, a->Hkv = p->Hkv, a->L = p->L, a->S = p->S, a->D = p->D;
  a->G = p->Hq / p->Hkv;
  a->causal = effective_causal(p) != TTSDPA_CAUSAL_NONE ? 1 : 0;
  a->causal_br = effective_causal(p) == TTSDPA_CAUSAL_BOTTOM_RIGHT ? 1 : 0;
  a->mask_kind = p->mask_kind;
  a->scale = p->scale;
  for (int i = 0; i < 3; i++) {
    a->qs[i] = p->q_stride[i], a->ks[i] = p->k_stride[i], a->vs[i] = p->v_stride[i], a->os[i] = p->o_stride[i];
  }
  return TTSDPA_OK;
}

// The MFMA prefill kernels stage key tiles of up to 64 rows: over a paged cache a tile must lie in one page.
constexpr int kPrefillMinPage = 64;

// 16-bit tensors the MFMA kernels can read with 16-byte loads and write with 8-byte stores.
bool fast_layout_ok(const ttsdpa_params* p, bool masks_ok = false, bool pages_ok = false) {
  if (p->block_table && !pages_ok) return false;
  if (p->dtype != TTSDPA_F16 && p->dtype != TTSDPA_BF16) return false;
  if (p->mask_kind != TTSDPA_MASK_NONE && !masks_ok) return false;
  if (!(p->scale > 0.f) || !isfinite(p->scale)) return false;  // the row maximum is taken on unscaled scores
  if (!dense_last_ok(p->q_stride, 8) || !dense_last_ok(p->k_stride, 8) || !dense_last_ok(p->v_stride, 8) ||
      !dense_last_ok(p->o_stride, 8))
    return false;
  return ptr_aligned(p->q, 16) && ptr_aligned(p->k, 16) && ptr_aligned(p->v, 16) && ptr_aligned(p->out, 16);
}

// The 4-wavefront and fp32 kernels read an attnMask four keys at a time: aligned groups, whole groups only.
bool simple_mask_ok(const ttsdpa_params* p) {
  return p->mask_kind == TTSDPA_MASK_NONE || (mask_vec4_ok(p) && p->S % 4 == 0 && !p->kv_len);
}

// fp32 tensors the fp32 MFMA kernel can read and write with 16-byte accesses.
bool f32_prefill_ok(const ttsdpa_params* p) {
  if (p->dtype != TTSDPA_F32 || (p->block_table && p->page_size < kPrefillMinPage) || !simple_mask_ok(p)) return false;
  if (p->D < 4 || p->D > 128 || p->D % 4 != 0) return false;  // 64 and 128; other multiples of 4 on the next one up with zero columns
  if (!(p->scale > 0.f) || !isfinite(p->scale) || p->S < 1 || p->L < 1) return false;
  if (!dense_last_ok(p->q_stride, 4) || !dense_last_ok(p->k_stride, 4) || !dense_last_ok(p->v_stride, 4) ||
      !dense_last_ok(p->o_stride, 4))
    return false;
  return ptr_aligned(p->q, 16) && ptr_aligned(p->k, 16) && ptr_aligned(p->v, 16) && ptr_aligned(p->out, 16);
}

bool pipelined_ok(const ttsdpa_params* p) {
  // the kernel addresses the 64 rows of a K / V tile and the 256 rows of a Q tile with 32-bit byte offsets
  return p->D == 128 && p->L > 128 && p->k_stride[2] < (1 << 24) && p->v_stride[2] < (1 << 24) && p->q_stride[2] < (1 << 22);
}

// Shapes whose row tiles the pipelined kernels divide among workgroups by keys (plan_pipelined_splits): `units` 256-row
// tiles in all, `keys` = what a row can see (under a top-left aligned causal mask no more than there are rows).
bool split_shape(const ttsdpa_params* p, long long* units, long long* keys) {
  *units = (long long)p->B * p->Hq * ((p->L + 255) / 256);
  *keys = effective_causal(p) == TTSDPA_CAUSAL_TOP_LEFT && p->L < p->S ? p->L : p->S;
  if (p->mask_kind != TTSDPA_MASK_NONE || p->block_table || *units > 128 || *keys < 2048) return false;
  return *units <= 64 || (p->causal && *keys >= 4096);
}

// A Bool attnMask the pipelined kernels apply inside their instruction streams (bool_mask_streams_ok on the kernels' side).
bool bool_mask_streams_param_ok(const ttsdpa_params* p) {
  return p->mask_kind == TTSDPA_MASK_BOOL && !p->causal && mask_vec4_ok(p) && p->S % 4 == 0 && !p->kv_len && !p->block_table &&
         (long long)(p->L - 1) * p->mask_stride[2] + 8 < (1ll << 32);
}

// The pipelined kernel at head_dim 64: no pages, and of attnMasks only Bool masks its streams can apply.  Against the 4-wavefront kernel (128-row tiles, keys
// divided among workgroups when the heads are not grouped) it measured level or up to 30 % faster from 512 query rows
// on; shorter calls take it when they fill half of the chip's CUs, or when their keys are split (16 heads x 256 rows on
// 32768 keys: 0.56 ms on the 4-wavefront kernel, which cannot split grouped heads).
bool pipelined64_ok(const ttsdpa_params* p) {
  if (p->D != 64 || p->L <= 128 || p->block_table) return false;
  if (p->mask_kind != TTSDPA_MASK_NONE && !bool_mask_streams_param_ok(p)) return false;
  if (!(p->k_stride[2] < (1 << 24) && p->v_stride[2] < (1 << 24) && p->q_stride[2] < (1 << 22))) return false;
  const long long tiles = (p->L + 255) / 256;
  if ((long long)p->B * p->Hq * (p->causal ? (tiles + 1) / 2 : tiles) >= 128) return true;
  long long units, keys;
  return p->L >= 512 || split_shape(p, &units, &keys);
}

// Few query rows per head against many keys on the 4-wavefront kernel: the G heads of a KV head share one row tile
// (dense q / out make [B,Hq,L,D] a [B,Hkv,G*L,D] tensor), so K/V are streamed once per KV head instead of once per
// query head and the tile is not mostly padding.
bool pack_heads_ok(const ttsdpa_params* p) {
  const int G = p->Hq / p->Hkv;
  if (pipelined_ok(p) || G < 2 || p->mask_kind != TTSDPA_MASK_NONE || p->L > 64 || p->S < 256) return false;
  if (p->dtype == TTSDPA_F32 && !f32_prefill_ok(p)) return false;
  return p->q_stride[1] == (int64_t)p->L * p->q_stride[2] && p->o_stride[1] == (int64_t)p->L * p->o_stride[2];
}

void pack_heads(KArgs* a) {
  a->pack_L = a->L;
  a->L = a->L * a->G, a->Hq = a->Hkv;
  a->qs[1] *= a->G, a->os[1] *= a->G;
  a->G = 1;
}

// Key splits of a short-L call on the 4-wavefront kernel (one query head per KV head, possibly after packing): when
// batch x heads x row tiles leave most of the 256 CUs idle, the keys are divided among several workgroups whose
// partial results the decode path's merge kernel combines.  Needs head_dim 64 or 128 (the merge kernel's) and scratch.
struct SplitPlan {
  int splits, chunk;
  size_t ws_bytes;
};
SplitPlan plan_prefill_splits(const ttsdpa_params* p, const KArgs& a /* after packing */) {
  SplitPlan s{1, 0, 0};
  if (a.G != 1 || (a.D != 64 && a.D != 128) || p->mask_kind != TTSDPA_MASK_NONE || pipelined_ok(p)) return s;
  const long long wgs = (long long)a.B * a.Hq * ((a.L + 127) / 128);
  long long want = (2 * 256 + wgs - 1) / wgs;  // aim for two workgroups per CU
  const long long most = a.S / 512;            // at least 8 key tiles per split
  if (want > most) want = most;
  if (want > 64) want = 64;                    // the merge kernel's limit
  if (want < 2) return s;
  int chunk = (int)((a.S + want - 1) / want);
  chunk = (chunk + 63) / 64 * 64;
  s.splits = (a.S + chunk - 1) / chunk;
  s.chunk = chunk;
  if (s.splits < 2) return SplitPlan{1, 0, 0};
  s.ws_bytes = (size_t)a.B * a.Hq * s.splits * a.L * (a.D + 2) * sizeof(float);
  return s;
}


// Key splits for the pipelined kernels (head_dim 128 and 64): a call with a quarter as many 256-row tiles as the chip has CUs, or
// fewer (a chunk of one sequence's rows against a long cache, a few heads of a tensor-parallel share), leaves most CUs
// without work.  Its row tiles then share their keys among workgroups of `chunk` keys (a multiple of 256: four key
// tiles, so the kernel's stages keep their constants), enough for two workgroups per CU, and the
// kernel's merge kernel combines the records.  The records cost: with 65-128 row tiles the split pays only under a
// causal mask on 4096 keys or more (4 heads x 8192 rows +32 %, one KV head's share of 2 x 4096 rows +7 %; without a mask
// -9 %, 2048 keys -18 %); with 64 and fewer it measured 1.1x to 5x (32 heads x 512 rows on 8192 keys 1.5x).
SplitPlan plan_pipelined_splits(const ttsdpa_params* p) {
  SplitPlan s{1, 0, 0};
  long long units, keys;
  if (p->dtype == TTSDPA_F32 || !(pipelined_ok(p) || pipelined64_ok(p)) || !split_shape(p, &units, &keys)) return s;
  long long want = (512 + units - 1) / units;
  const long long most = keys / 512;  // at least 8 key tiles per split
  if (want > most) want = most;
  if (want > 64) want = 64;           // the merge kernel's limit
  if (want < 2) return s;
  long long chunk = (keys + want - 1) / want;
  chunk = (chunk + 255) / 256 * 256;
  s.splits = (int)((keys + chunk - 1) / chunk);
  s.chunk = (int)chunk;
  if (s.splits < 2) return SplitPlan{1, 0, 0};
  s.ws_bytes = (size_t)p->B * p->Hq * s.splits * p->L * (p->D + 2) * sizeof(float);
  return s;
}

bool prefill_ok(const ttsdpa_params* p) {
  if (f32_prefill_ok(p)) return true;
  // the pipelined head_dim-128 kernel takes any attnMask; the 4-wavefront kernel those it can read four keys at a time
  // head sizes between the 4-wavefront kernel's (32, 64, 96, 128, 192, 256) run on the next one up with zero columns
  const bool mfma_head_dim = p->D >= 8 && p->D <= 256 && p->D % 8 == 0;
  if (p->block_table && p->page_size < kPrefillMinPage) return false;
  // the 16-bit kernels address the rows of a K / V tile with 32-bit byte offsets (the fp32 kernel returned above does not)
  const bool tile_offsets_ok = p->k_stride[2] < (1 << 24) && p->v_stride[2] < (1 << 24);
  return fast_layout_ok(p, true, true) && mfma_head_dim && p->S >= 1 && p->L >= 1 && tile_offsets_ok &&
         (pipelined_ok(p) || simple_mask_ok(p));
}

bool decode_ok(const ttsdpa_params* p) {
  // a top-left aligned causal mask leaves a few keys per row: not the streaming kernel's case
  // head_dim 64 and 128; other multiples of 8 up to 128 on the next one up with zero columns
  if (!fast_layout_ok(p, false, true) || p->D < 8 || p->D > 128 || p->D % 8 != 0 || effective_causal(p) == TTSDPA_CAUSAL_TOP_LEFT ||
      p->S < 1 || p->L < 1)
    return false;
  if (p->block_table && p->page_size < 32) return false;  // a 32-key block of a wavefront must lie in one page
  return (long long)p->L * (p->Hq / p->Hkv) <= kDecodeMaxRows;
}

int pick_route(const ttsdpa_params* p) {
  if (p->B == 0 || p->L == 0) return TTSDPA_ROUTE_NONE;
  if (p->S == 0) return TTSDPA_ROUTE_ZERO;
  // Few query rows against many keys: streaming the cache once for the whole head group beats a 128-row tile.
  if (decode_ok(p) && p->S >= 256) {
    // 9-16 rows per KV head: the streaming kernel does P.V on the vector ALUs and measures 5.5 TB/s there; the
    // 4-wavefront MFMA kernel with packed heads and split keys 5.85 TB/s, when the call allows it
    const long long rows = (long long)p->L * (p->Hq / p->Hkv);
    // (head_dim 64 / 128: the zero-column variants of that kernel do not split their keys)
    if (rows > 8 && (p->D == 64 || p->D == 128) && prefill_ok(p) && !pipelined_ok(p) && (p->Hq == p->Hkv || pack_heads_ok(p)))
      return TTSDPA_ROUTE_PREFILL;
    return TTSDPA_ROUTE_DECODE;
  }
  if (prefill_ok(p) && p->L >= 16) return TTSDPA_ROUTE_PREFILL;
  if (decode_ok(p)) return TTSDPA_ROUTE_DECODE;
  if (prefill_ok(p)) return TTSDPA_ROUTE_PREFILL;
  return TTSDPA_ROUTE_GENERAL;
}

// ---- backward ---------------------------------------------------------------------------------------------------------
int validate_backward(const ttsdpa_backward_params* p, BwdArgs* a) {
  if (!p) return TTSDPA_ERR_NULL;
  if (p->struct_size != sizeof(ttsdpa_backward_params)) return TTSDPA_ERR_ABI;
  int rc = validate(&p->fwd, &a->f);
  if (rc != TTSDPA_OK) return rc;
  const ttsdpa_params* f = &p->fwd;
  if (f->block_table) return TTSDPA_ERR_UNSUPPORTED;
  const size_t esz = f->dtype == TTSDPA_F32 ? 4 : 2;
  if (f->B > 0 && f->L > 0 && (!p->dout || !p->dq)) return TTSDPA_ERR_NULL;
  if (f->B > 0 && f->S > 0 && (!p->dk || !p->dv || !f->k || !f->v)) return TTSDPA_ERR_NULL;
  if (!ptr_aligned(p->dout, esz) || !ptr_aligned(p->dq, esz) || !ptr_aligned(p->dk, esz) || !ptr_aligned(p->dv, esz))
    return TTSDPA_ERR_STRIDE;
  for (int i = 0; i < 3; i++) {
    if (p->dout_stride[i] < 0 || p->dq_stride[i] < 0 || p->dk_stride[i] < 0 || p->dv_stride[i] < 0) return TTSDPA_ERR_STRIDE;
    a->dos[i] = p->dout_stride[i], a->dqs[i] = p->dq_stride[i], a->dks[i] = p->dk_stride[i], a->dvs[i] = p->dv_stride[i];
  }
  if ((p->dout_stride[2] < f->D || p->dq_stride[2] < f->D) && f->L > 1) return TTSDPA_ERR_STRIDE;
  if ((p->dk_stride[2] < f->D || p->dv_stride[2] < f->D) && f->S > 1) return TTSDPA_ERR_STRIDE;
  a->dout = p->dout, a->dq = p->dq, a->dk = p->dk, a->dv = p->dv, a->stats = nullptr, a->partial = nullptr, a->dkv_splits = 1, a->dq_partial = nullptr, a->dq_splits = 1, a->dkv_round = 0;
  return TTSDPA_OK;
}

// The MFMA backward kernels: 16-bit tensors they can read and write with 16-byte / 8-byte accesses, head_dim 64 or
// 128, attnMasks the forward's 4-wavefront kernel takes (keys readable four at a time, no kv_len beside them).
bool backward_mfma_ok(const ttsdpa_backward_params* p) {
  const ttsdpa_params* f = &p->fwd;
  // head_dim 64 and 128; other multiples of 8 up to 128 on the register-staged kernels of the next one up (zero columns)
  if (!fast_layout_ok(f, true) || !simple_mask_ok(f) || f->D < 8 || f->D > 128 || f->D % 8 != 0 || f->L < 1 || f->S < 1) return false;
  if (!dense_last_ok(p->dout_stride, 8) || !dense_last_ok(p->dq_stride, 8) || !dense_last_ok(p->dk_stride, 8) ||
      !dense_last_ok(p->dv_stride, 8))
    return false;
  // the head_dim-128 dk/dv kernel addresses the rows of a tile with 32-bit byte offsets from the tile's first row
  if (f->D == 128 && (f->q_stride[2] >= (1 << 24) || f->k_stride[2] >= (1 << 24) || f->v_stride[2] >= (1 << 24) ||
                      p->dout_stride[2] >= (1 << 24)))
    return false;
  return ptr_aligned(p->dout, 16) && ptr_aligned(p->dq, 16) && ptr_aligned(p->dk, 16) && ptr_aligned(p->dv, 16);
}

// The fp32 matrix-core backward kernels: fp32 tensors with 16-byte aligned rows, head_dim 64 or 128, attnMasks as for
// the 16-bit pair.
bool backward_f32_ok(const ttsdpa_backward_params* p) {
  const ttsdpa_params* f = &p->fwd;
  if (f->dtype != TTSDPA_F32 || f->block_table || !simple_mask_ok(f) || f->D < 4 || f->D > 128 || f->D % 4 != 0) return false;
  if (!(f->scale > 0.f) || !isfinite(f->scale) || f->L < 1 || f->S < 1) return false;  // the row maximum is taken on unscaled scores
  if (!dense_last_ok(f->q_stride, 4) || !dense_last_ok(f->k_stride, 4) || !dense_last_ok(f->v_stride, 4) ||
      !dense_last_ok(f->o_stride, 4) || !dense_last_ok(p->dout_stride, 4) || !dense_last_ok(p->dq_stride, 4) ||
      !dense_last_ok(p->dk_stride, 4) || !dense_last_ok(p->dv_stride, 4))
    return false;
  return ptr_aligned(f->q, 16) && ptr_aligned(f->k, 16) && ptr_aligned(f->v, 16) && ptr_aligned(f->out, 16) &&
         ptr_aligned(p->dout, 16) && ptr_aligned(p->dq, 16) && ptr_aligned(p->dk, 16) && ptr_aligned(p->dv, 16);
}

int pick_backward_route(const ttsdpa_backward_params* p) {
  const ttsdpa_params* f = &p->fwd;
  if (f->B == 0 || (f->L == 0 && f->S == 0)) return TTSDPA_ROUTE_NONE;
  return backward_mfma_ok(p) || backward_f32_ok(p) ? TTSDPA_ROUTE_PREFILL : TTSDPA_ROUTE_GENERAL;
}

size_t backward_stats_bytes(const ttsdpa_backward_params* p) {
  return (size_t)p->fwd.B * p->fwd.Hq * p->fwd.L * 2 * sizeof(float);
}

// Scratch layout: the statistics, then (matrix-core pairs with a split query stream) the partial dk / dv, 256-byte aligned.
int dkv_splits_of(const ttsdpa_backward_params* p) {
  const ttsdpa_params* f = &p->fwd;
  if (pick_backward_route(p) != TTSDPA_ROUTE_PREFILL) return 1;
  if (f->D != 64 && f->D != 128) return 1;  // the zero-column variants do not split (their records are laid out for 64 / 128)
  const int groups = f->dtype != TTSDPA_F32 && f->D == 128 && f->mask_kind == TTSDPA_MASK_NONE ? 2 : 1;
  const int per_cu = f->D == 64 && f->mask_kind == TTSDPA_MASK_NONE ? 2 : 1;
  return backward_dkv_splits(f->B, f->Hkv, f->Hq, f->L, f->S, effective_causal(f) != TTSDPA_CAUSAL_NONE, groups, per_cu);
}
// ... then (matrix-core pairs whose dq kernel splits its key ranges) the partial dq records, 256-byte aligned.
int dq_splits_of(const ttsdpa_backward_params* p) {
  const ttsdpa_params* f = &p->fwd;
  if (pick_backward_route(p) != TTSDPA_ROUTE_PREFILL) return 1;
  if (f->D != 64 && f->D != 128) return 1;
  const int slots = f->dtype == TTSDPA_F32 && f->D == 128 ? 256 : 512;
  return backward_dq_splits(f->B, f->Hq, f->L, f->S, effective_causal(f) != TTSDPA_CAUSAL_NONE, slots);
}
size_t backward_partial_offset(const ttsdpa_backward_params* p) { return (backward_stats_bytes(p) + 255) & ~(size_t)255; }
size_t backward_dq_partial_offset(const ttsdpa_backward_params* p) {
  const int n = dkv_splits_of(p);
  if (n == 1) return backward_partial_offset(p);
  const size_t end = backward_partial_offset(p) + (size_t)n * 2 * p->fwd.B * p->fwd.Hkv * p->fwd.S * p->fwd.D * sizeof(float);
  return (end + 255) & ~(size_t)255;
}
size_t backward_scratch_bytes(const ttsdpa_backward_params* p) {
  const int n = dkv_splits_of(p), nq = dq_splits_of(p);
  if (nq > 1)
    return backward_dq_partial_offset(p) + (size_t)nq * p->fwd.B * p->fwd.Hq * p->fwd.L * (p->fwd.D + 2) * sizeof(float);
  if (n == 1) return backward_stats_bytes(p);
  return backward_partial_offset(p) + (size_t)n * 2 * p->fwd.B * p->fwd.Hkv * p->fwd.S * p->fwd.D * sizeof(float);
}

int check_grid(long long nwg) { return nwg > 0x7fffffffLL ? TTSDPA_ERR_SHAPE : TTSDPA_OK; }

// Scratch of ttsdpa_decode_static: the split-KV partial records of one decode call.  Every GPU the library runs on holds
// its own copy of this array, at its own address, until the process ends.  In host code the array's name is only a
// handle for hipGetSymbolAddress: kernels and memory calls get the address that call returns, never the name.
constexpr size_t kStaticScratchBytes = TTSDPA_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// Address of the current device's copy of `scratch`, looked up once per device (with that device current) and kept.
// Safe from several host threads: the worst case is two identical look-ups.
int static_scratch_of_current_device(void** out) {
  static void* ptr[kMaxDevices];
  static bool done[kMaxDevices];
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= kMaxDevices) return (int)hipErrorInvalidDevice;
  if (!__atomic_load_n(&done[dev], __ATOMIC_ACQUIRE)) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (!p) return (int)hipErrorInvalidSymbol;
    __atomic_store_n(&ptr[dev], p, __ATOMIC_RELAXED);
    __atomic_store_n(&done[dev], true, __ATOMIC_RELEASE);
  }
  *out = __atomic_load_n(&ptr[dev], __ATOMIC_RELAXED);
  return TTSDPA_OK;
}

}  // namespace

extern "C" {

int ttsdpa_abi_version(void) { return TTSDPA_ABI_VERSION; }

const char* ttsdpa_status_string(int status) {
  switch (status) {
    case TTSDPA_OK: return "ok";
    case TTSDPA_ERR_NULL: return "required pointer is NULL";
    case TTSDPA_ERR_DTYPE: return "unsupported dtype";
    case TTSDPA_ERR_SHAPE: return "invalid or unsupported shape";
    case TTSDPA_ERR_STRIDE: return "unsupported stride or alignment";
    case TTSDPA_ERR_MASK: return "invalid mask arguments";
    case TTSDPA_ERR_WORKSPACE: return "workspace missing or too small";
    case TTSDPA_ERR_UNSUPPORTED: return "arguments outside this kernel's domain";
    case TTSDPA_ERR_ABI: return "ttsdpa_params.struct_size mismatch";
    case TTSDPA_ERR_STATIC_SCRATCH: return "call needs more scratch than the library's static buffer holds (TTSDPA_STATIC_SCRATCH_BYTES)";
    default: return status > 0 ? hipGetErrorString((hipError_t)status) : "unknown status";
  }
}

void ttsdpa_params_init(ttsdpa_params* p, int dtype, int B, int Hq, int Hkv, int L, int S, int D) {
  memset(p, 0, sizeof(*p));
  p->struct_size = sizeof(*p);
  p->dtype = dtype;
  p->B = B, p->Hq = Hq, p->Hkv = Hkv, p->L = L, p->S = S, p->D = D;
  p->q_stride[0] = (int64_t)Hq * L * D, p->q_stride[1] = (int64_t)L * D, p->q_stride[2] = D;
  p->k_stride[0] = (int64_t)Hkv * S * D, p->k_stride[1] = (int64_t)S * D, p->k_stride[2] = D;
  p->v_stride[0] = p->k_stride[0], p->v_stride[1] = p->k_stride[1], p->v_stride[2] = D;
  p->o_stride[0] = p->q_stride[0], p->o_stride[1] = p->q_stride[1], p->o_stride[2] = D;
  p->scale = D > 0 ? 1.f / sqrtf((float)D) : 1.f;
  p->causal = 0;
  p->mask_kind = TTSDPA_MASK_NONE;
  p->mask = nullptr;
  p->mask_stride[0] = 0, p->mask_stride[1] = 0, p->mask_stride[2] = S, p->mask_stride[3] = 1;
  p->kv_len = nullptr;
  p->block_table = nullptr, p->page_size = 0, p->block_table_stride = 0;
}

int ttsdpa_plan(const ttsdpa_params* p, int* route) {
  KArgs a;
  int rc = validate(p, &a);
  if (rc != TTSDPA_OK) return rc;
  if (route) *route = pick_route(p);
  return TTSDPA_OK;
}

size_t ttsdpa_workspace_bytes(const ttsdpa_params* p) {
  KArgs a;
  if (validate(p, &a) != TTSDPA_OK) return 0;
  if (p->B == 0 || p->L == 0 || p->S == 0) return 0;
  // enough for ttsdpa_forward's route and for an explicit ttsdpa_decode of the same call
  size_t need = decode_ok(p) ? plan_decode(a).ws_bytes : 0;
  if (pick_route(p) == TTSDPA_ROUTE_PREFILL) {
    if (pack_heads_ok(p)) pack_heads(&a);
    size_t split = plan_prefill_splits(p, a).ws_bytes;
    need = split > need ? split : need;
    split = plan_pipelined_splits(p).ws_bytes;
    need = split > need ? split : need;
  }
  return need;
}

int ttsdpa_general(const ttsdpa_params* p, void* stream) {
  KArgs a;
  int rc = validate(p, &a);
  if (rc != TTSDPA_OK) return rc;
  if (p->B == 0 || p->L == 0) return TTSDPA_OK;
  if (p->S == 0) return launch_zero(a, p->dtype, (hipStream_t)stream);
  if ((rc = check_grid((long long)a.B * a.Hq * ((a.L + 63) / 64))) != TTSDPA_OK) return rc;
  return launch_general(a, p->dtype, (hipStream_t)stream);
}

// ttsdpa_prefill with optional scratch: with it, a short-L call may divide its keys among workgroups.
static int prefill_impl(const ttsdpa_params* p, void* workspace, size_t workspace_bytes, void* stream) {
  KArgs a;
  int rc = validate(p, &a);
  if (rc != TTSDPA_OK) return rc;
  if (p->B == 0 || p->L == 0) return TTSDPA_OK;
  if (!prefill_ok(p)) return TTSDPA_ERR_UNSUPPORTED;
  if ((rc = check_grid((long long)a.B * a.Hq * ((a.L + 127) / 128))) != TTSDPA_OK) return rc;
  // head_dim 128 with enough rows to fill 256-row workgroups takes the software-pipelined kernel (its tile loads
  // address 64 rows with 32-bit byte offsets)
  if (p->dtype != TTSDPA_F32 && pipelined_ok(p)) {
    const SplitPlan sp = plan_pipelined_splits(p);
    if (sp.splits > 1 && workspace && workspace_bytes >= sp.ws_bytes && ptr_aligned(workspace, 16)) {
      a.kv_splits = sp.splits, a.kv_chunk = sp.chunk, a.ws = (float*)workspace;
      if ((rc = check_grid((long long)a.B * a.Hq * ((a.L + 255) / 256 + 8) * sp.splits)) != TTSDPA_OK) return rc;
      return launch_prefill_d128(a, p->dtype, (hipStream_t)stream);  // the kernel and the merge of its records
    }
    a.kv_splits = 1, a.kv_chunk = 0, a.ws = nullptr;
    return launch_prefill_d128(a, p->dtype, (hipStream_t)stream);
  }
  if (p->dtype != TTSDPA_F32 && pipelined64_ok(p)) {
    const SplitPlan sp = plan_pipelined_splits(p);
    if (sp.splits > 1 && workspace && workspace_bytes >= sp.ws_bytes && ptr_aligned(workspace, 16))
      a.kv_splits = sp.splits, a.kv_chunk = sp.chunk, a.ws = (float*)workspace;
    else
      a.kv_splits = 1, a.kv_chunk = 0, a.ws = nullptr;
    return launch_prefill_d64(a, p->dtype, (hipStream_t)stream);  // with splits: the kernel and the merge of its records
  }
  auto launch = [&](const KArgs& k) {
    return p->dtype == TTSDPA_F32 ? launch_prefill_f32(k, (hipStream_t)stream) : launch_prefill(k, p->dtype, (hipStream_t)stream);
  };
  if (pack_heads_ok(p)) pack_heads(&a);
  a.kv_splits = 1, a.kv_chunk = 0, a.ws = nullptr;
  const SplitPlan sp = plan_prefill_splits(p, a);
  if (sp.splits > 1 && workspace && workspace_bytes >= sp.ws_bytes && ptr_aligned(workspace, 16) && p->S > 0) {
    a.kv_splits = sp.splits, a.kv_chunk = sp.chunk, a.ws = (float*)workspace;
    if ((rc = check_grid((long long)a.B * a.Hq * ((a.L + 127) / 128) * sp.splits)) != TTSDPA_OK) return rc;
    rc = launch(a);
    if (rc != 0) return rc;
    return launch_merge(a, p->dtype, sp.splits, a.ws, (hipStream_t)stream);
  }
  return launch(a);
}

int ttsdpa_prefill(const ttsdpa_params* p, void* stream) { return prefill_impl(p, nullptr, 0, stream); }

int ttsdpa_decode(const ttsdpa_params* p, void* workspace, size_t workspace_bytes, void* stream) {
  KArgs a;
  int rc = validate(p, &a);
  if (rc != TTSDPA_OK) return rc;
  if (p->B == 0 || p->L == 0) return TTSDPA_OK;
  if (!decode_ok(p)) return TTSDPA_ERR_UNSUPPORTED;
  DecodePlan pl = plan_decode(a);
  if (pl.ws_bytes > 0 && (!workspace || workspace_bytes < pl.ws_bytes || !ptr_aligned(workspace, 16)))
    return TTSDPA_ERR_WORKSPACE;
  if ((rc = check_grid((long long)a.B * a.Hkv * pl.splits)) != TTSDPA_OK) return rc;
  return launch_decode(a, p->dtype, workspace, (hipStream_t)stream);
}

int ttsdpa_decode_static(const ttsdpa_params* p, void* stream) {
  KArgs a;
  int rc = validate(p, &a);
  if (rc != TTSDPA_OK) return rc;
  if (p->B == 0 || p->L == 0) return TTSDPA_OK;
  if (!decode_ok(p)) return TTSDPA_ERR_UNSUPPORTED;
  const DecodePlan pl = plan_decode(a);
  if (pl.ws_bytes > kStaticScratchBytes) return TTSDPA_ERR_STATIC_SCRATCH;
  if ((rc = check_grid((long long)a.B * a.Hkv * pl.splits)) != TTSDPA_OK) return rc;
  void* ws = nullptr;
  if ((rc = static_scratch_of_current_device(&ws)) != TTSDPA_OK) return rc;
  // Nothing in the records has to start at zero: every split writes its whole record (an empty split a weight of
  // zero) before the merge kernel, later on the same stream, reads it.
  return launch_decode(a, p->dtype, ws, (hipStream_t)stream);
}

int ttsdpa_forward(const ttsdpa_params* p, void* workspace, size_t workspace_bytes, void* stream) {
  KArgs a;
  int rc = validate(p, &a);
  if (rc != TTSDPA_OK) return rc;
  switch (pick_route(p)) {
    case TTSDPA_ROUTE_NONE: return TTSDPA_OK;
    case TTSDPA_ROUTE_ZERO: return launch_zero(a, p->dtype, (hipStream_t)stream);
    case TTSDPA_ROUTE_DECODE: return ttsdpa_decode(p, workspace, workspace_bytes, stream);
    case TTSDPA_ROUTE_PREFILL: return prefill_impl(p, workspace, workspace_bytes, stream);
    default: return ttsdpa_general(p, stream);
  }
}

void ttsdpa_backward_params_init(ttsdpa_backward_params* p, int dtype, int B, int Hq, int Hkv, int L, int S, int D) {
  memset(p, 0, sizeof(*p));
  p->struct_size = sizeof(*p);
  ttsdpa_params_init(&p->fwd, dtype, B, Hq, Hkv, L, S, D);
  for (int i = 0; i < 3; i++) {
    p->dout_stride[i] = p->dq_stride[i] = p->fwd.q_stride[i];
    p->dk_stride[i] = p->dv_stride[i] = p->fwd.k_stride[i];
  }
}

int ttsdpa_backward_plan(const ttsdpa_backward_params* p, int* route) {
  BwdArgs a;
  int rc = validate_backward(p, &a);
  if (rc != TTSDPA_OK) return rc;
  if (route) *route = pick_backward_route(p);
  return TTSDPA_OK;
}

size_t ttsdpa_backward_workspace_bytes(const ttsdpa_backward_params* p) {
  BwdArgs a;
  if (validate_backward(p, &a) != TTSDPA_OK) return 0;
  return backward_scratch_bytes(p);
}

int ttsdpa_backward(const ttsdpa_backward_params* p, void* workspace, size_t workspace_bytes, void* stream) {
  BwdArgs a;
  int rc = validate_backward(p, &a);
  if (rc != TTSDPA_OK) return rc;
  const int route = pick_backward_route(p);
  if (route == TTSDPA_ROUTE_NONE) return TTSDPA_OK;
  const size_t need = backward_scratch_bytes(p);
  if (need > 0 && (!workspace || workspace_bytes < need || !ptr_aligned(workspace, 16))) return TTSDPA_ERR_WORKSPACE;
  a.stats = (float*)workspace;
  a.dkv_splits = dkv_splits_of(p);
  a.partial = a.dkv_splits > 1 ? (float*)((char*)workspace + backward_partial_offset(p)) : nullptr;
  a.dq_splits = dq_splits_of(p);
  a.dq_partial = a.dq_splits > 1 ? (float*)((char*)workspace + backward_dq_partial_offset(p)) : nullptr;
  if (route == TTSDPA_ROUTE_PREFILL) {
    const long long g1 = (long long)a.f.B * a.f.Hq * ((a.f.L + 127) / 128) * a.dq_splits, g2 = (long long)a.f.B * a.f.Hkv * ((a.f.S + 127) / 128);
    if (check_grid(g1) != TTSDPA_OK || check_grid(g2) != TTSDPA_OK) return TTSDPA_ERR_SHAPE;
    if (p->fwd.dtype == TTSDPA_F32) return launch_backward_f32(a, (hipStream_t)stream);
    return launch_backward_mfma(a, p->fwd.dtype, (hipStream_t)stream);
  }
  {  // the vector-ALU pair: 64 rows per workgroup up to head_dim 128, 32 beyond
    const int rows = a.f.D <= 128 ? 64 : 32;
    const long long g1 = (long long)a.f.B * a.f.Hq * ((a.f.L + rows - 1) / rows), g2 = (long long)a.f.B * a.f.Hkv * ((a.f.S + rows - 1) / rows);
    if (check_grid(g1) != TTSDPA_OK || check_grid(g2) != TTSDPA_OK) return TTSDPA_ERR_SHAPE;
  }
  return launch_backward_general(a, p->fwd.dtype, (hipStream_t)stream);
}

void ttsdpa_kv_append_params_init(ttsdpa_kv_append_params* p, int dtype, int B, int Hkv, int Smax, int Lnew, int D) {
  memset(p, 0, sizeof(*p));
  p->struct_size = sizeof(*p);
  p->dtype = dtype;
  p->B = B, p->Hkv = Hkv, p->Smax = Smax, p->Lnew = Lnew, p->D = D;
  p->kc_stride[0] = (int64_t)Hkv * Smax * D, p->kc_stride[1] = (int64_t)Smax * D, p->kc_stride[2] = D;
  p->kn_stride[0] = (int64_t)Hkv * Lnew * D, p->kn_stride[1] = (int64_t)Lnew * D, p->kn_stride[2] = D;
  for (int i = 0; i < 3; i++) p->vc_stride[i] = p->kc_stride[i], p->vn_stride[i] = p->kn_stride[i];
}

int ttsdpa_kv_append(const ttsdpa_kv_append_params* p, void* stream) {
  if (!p) return TTSDPA_ERR_NULL;
  if (p->struct_size != sizeof(ttsdpa_kv_append_params)) return TTSDPA_ERR_ABI;
  if (p->dtype != TTSDPA_F32 && p->dtype != TTSDPA_F16 && p->dtype != TTSDPA_BF16) return TTSDPA_ERR_DTYPE;
  if (p->B < 0 || p->Hkv < 1 || p->Smax < 0 || p->Lnew < 0 || p->D < 1) return TTSDPA_ERR_SHAPE;
  if (p->B == 0 || p->Lnew == 0 || p->Smax == 0) return TTSDPA_OK;
  if (!p->k_cache || !p->v_cache || !p->k_new || !p->v_new) return TTSDPA_ERR_NULL;
  const size_t esz = p->dtype == TTSDPA_F32 ? 4 : 2;
  if (!ptr_aligned(p->k_cache, esz) || !ptr_aligned(p->v_cache, esz) || !ptr_aligned(p->k_new, esz) ||
      !ptr_aligned(p->v_new, esz) || (p->positions && !ptr_aligned(p->positions, 4)))
    return TTSDPA_ERR_STRIDE;
  KvAppendArgs a;
  for (int i = 0; i < 3; i++) {
    if (p->kc_stride[i] < 0 || p->vc_stride[i] < 0 || p->kn_stride[i] < 0 || p->vn_stride[i] < 0) return TTSDPA_ERR_STRIDE;
    a.kcs[i] = p->kc_stride[i], a.vcs[i] = p->vc_stride[i], a.kns[i] = p->kn_stride[i], a.vns[i] = p->vn_stride[i];
  }
  if ((p->kc_stride[2] < p->D || p->vc_stride[2] < p->D) && p->Smax > 1) return TTSDPA_ERR_STRIDE;
  if ((p->kn_stride[2] < p->D || p->vn_stride[2] < p->D) && p->Lnew > 1) return TTSDPA_ERR_STRIDE;
  a.kc = p->k_cache, a.vc = p->v_cache, a.kn = p->k_new, a.vn = p->v_new, a.positions = p->positions;
  a.block_table = p->block_table, a.page_shift = 0, a.bt_stride = p->block_table_stride;
  if (p->block_table) {
    if (!ptr_aligned(p->block_table, 4) || p->block_table_stride < 0) return TTSDPA_ERR_STRIDE;
    if (p->page_size < 1 || (p->page_size & (p->page_size - 1)) != 0) return TTSDPA_ERR_SHAPE;
    while ((1 << a.page_shift) < p->page_size) a.page_shift++;
  }
  a.B = p->B, a.Hkv = p->Hkv, a.Smax = p->Smax, a.Lnew = p->Lnew, a.D = p->D, a.position = p->position, a.esz = (int)esz;
  return launch_kv_append(a, (hipStream_t)stream);
}

}  // extern "C"
