/*
 * ttsdpa — scaled-dot-product attention for AMD MI355X (gfx950), C ABI.
 *
 * This is the device boundary behind TinyTorch's attention call
 *     tinytorch::function::sdpAttention(query, key, value, isCausal, attnMask, dropoutP, scale)
 * (reference src/Function/FuncNNLayer.h:298-302; forward composite at :231-266).  In the reference that call expands
 * to ~11 generic device ops (transpose, batched GEMM, scale, mask build, broadcast add, softmax, GEMM; reference
 * src/Operation/OpLinalgCuda.cuh:239-293, src/Operation/OpNNLayerCuda.cuh:36-145,359-380,
 * src/Tensor/TensorIterator.cuh:72-161, src/Operation/OpTransformCuda.cuh:79,193).  Here the whole forward is one
 * entry point; the GPU slot of the {device, dtype} dispatch table (reference src/Tensor/Dispatch.h:32-48) binds to it.
 *
 * Conventions (they follow the reference's device ops, src/Utils/CUDAUtils.h:36-83 and src/Tensor/TensorImpl.cpp:234-241):
 *   - plain device pointers and sizes, no framework types; tensors are row-major with unit stride on the last
 *     (head_dim) axis and caller-given element strides on batch / head / sequence, so KV-cache views and
 *     grouped-query layouts pass without copies;
 *   - work is enqueued on the caller's HIP stream and the call returns without synchronising;
 *   - the library never allocates or frees device memory: the output and the decode workspace are the caller's;
 *   - no exceptions, no abort: every entry point returns a status.  0 = enqueued; negative = the arguments are
 *     outside what the library handles (nothing was launched, the caller may take another route);
 *     positive = a hipError_t from the runtime.
 */
#ifndef TTSDPA_H
#define TTSDPA_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TTSDPA_ABI_VERSION 7

/* Element types; numbering is the reference's DType enum (reference src/Tensor/DType.h:20-28). */
enum ttsdpa_dtype { TTSDPA_F32 = 0, TTSDPA_F16 = 1, TTSDPA_BF16 = 2 };

/* Kind of attnMask (reference src/Function/FuncNNLayer.h:249-256). */
enum ttsdpa_mask_kind {
  TTSDPA_MASK_NONE = 0,
  TTSDPA_MASK_BOOL = 1, /* uint8, 0 = key hidden (bias -inf), non-zero = visible */
  TTSDPA_MASK_ADD = 2   /* additive bias, same element type as q */
};

enum ttsdpa_status {
  TTSDPA_OK = 0,
  TTSDPA_ERR_NULL = -1,        /* a required pointer is NULL */
  TTSDPA_ERR_DTYPE = -2,       /* dtype not one of ttsdpa_dtype */
  TTSDPA_ERR_SHAPE = -3,       /* negative size, Hq not a multiple of Hkv, head_dim unsupported */
  TTSDPA_ERR_STRIDE = -4,      /* stride / pointer alignment the kernels cannot use */
  TTSDPA_ERR_MASK = -5,        /* mask_kind invalid, or causal together with a mask (the reference asserts) */
  TTSDPA_ERR_WORKSPACE = -6,   /* workspace NULL or smaller than ttsdpa_workspace_bytes() */
  TTSDPA_ERR_UNSUPPORTED = -7, /* valid call, but not for the kernel asked for (e.g. ttsdpa_decode with L > limit) */
  TTSDPA_ERR_ABI = -8,         /* struct_size does not match this library */
  TTSDPA_ERR_STATIC_SCRATCH = -9 /* ttsdpa_decode_static: the call needs more than TTSDPA_STATIC_SCRATCH_BYTES of scratch */
};

/* Which kernel a call maps to (ttsdpa_plan). */
enum ttsdpa_causal {
  TTSDPA_CAUSAL_NONE = 0,
  TTSDPA_CAUSAL_TOP_LEFT = 1,    /* the reference's isCausal */
  TTSDPA_CAUSAL_BOTTOM_RIGHT = 2 /* queries are the last L positions of the key sequence */
};

enum ttsdpa_route {
  TTSDPA_ROUTE_NONE = 0,    /* nothing to launch (an empty output) */
  TTSDPA_ROUTE_GENERAL = 1, /* any dtype / head_dim / mask / per-batch key counts; fp32 arithmetic on the vector ALUs */
  TTSDPA_ROUTE_PREFILL = 2, /* MFMA flash-attention forward: fp16/bf16 with any head_dim that is a multiple of 8 up to 256 (attnMasks readable four keys at a time; any attnMask at head_dim 128 with L > 128); fp32 with any head_dim that is a multiple of 4 up to 128 */
  TTSDPA_ROUTE_DECODE = 3,  /* fp16/bf16, head_dim a multiple of 8 up to 128, few query rows against a long KV cache: split-KV streaming */
  TTSDPA_ROUTE_ZERO = 4     /* S == 0: the reference's empty contraction yields zeros */
};

/*
 * One attention call.  Shapes follow the reference op: q [B,Hq,L,D], k and v [B,Hkv,S,D], out [B,Hq,L,D].
 * Query head h reads KV head h / (Hq/Hkv) — what op::repeatInterleave(k, Hq/Hkv, 1) (reference
 * src/Operation/OpTransformCpu.h:399-442) or the 5-D matmul broadcast (src/Operation/OpLinalg.cpp:205-223) feeds
 * the reference; Hkv == Hq is plain multi-head attention.
 * Strides are in elements: {batch, head, sequence}; the head_dim stride is 1.  A dense tensor [B,H,N,D] has
 * {H*N*D, N*D, D}.
 * causal (ttsdpa_causal): TTSDPA_CAUSAL_TOP_LEFT is the reference's isCausal — key j is visible to query i iff
 * j <= i (tril(ones(L,S),0), reference src/Function/FuncNNLayer.h:241-247); a decode step with L == 1 must therefore
 * not pass it.  TTSDPA_CAUSAL_BOTTOM_RIGHT aligns the diagonal with the end of the keys instead: the L queries are the
 * last L positions of a sequence of S_b keys (S_b = kv_len[b] when given, else S), key j is visible to query i iff
 * j <= i + max(0, S_b - L).  It is what the reference computes when handed the Bool mask tril(ones(L,S), S-L), and
 * what a chunked prefill or a multi-token decode step against a KV cache needs; for L == S the two coincide.
 * mask: NULL, or an attnMask of any shape that broadcasts to [B,Hq,L,S] — the reference adds it to the scores with
 * a broadcasting add (src/Function/FuncNNLayer.h:249-260).  mask_stride gives its element strides along
 * {batch, head, query row, key}; an axis the mask does not have, or has with size 1, gets stride 0.  A dense
 * [L,S] mask is {0, 0, S, 1} (what ttsdpa_params_init fills), a per-batch key-padding mask [B,1,1,S] is {S, 0, 0, 1}.
 * scale multiplies q.k^T before the bias; the reference default is 1/sqrt(D).
 */
typedef struct ttsdpa_params {
  uint32_t struct_size; /* sizeof(ttsdpa_params) */
  int32_t dtype;        /* ttsdpa_dtype of q, k, v, out */
  const void* q;
  const void* k;
  const void* v;
  void* out;
  int32_t B, Hq, Hkv, L, S, D;
  int64_t q_stride[3];
  int64_t k_stride[3];
  int64_t v_stride[3];
  int64_t o_stride[3];
  float scale;
  int32_t causal;    /* ttsdpa_causal */
  int32_t mask_kind; /* ttsdpa_mask_kind */
  const void* mask;
  int64_t mask_stride[4]; /* elements: batch, head, query row, key; 0 broadcasts the axis */
  /* Per-batch number of valid keys, int32[B] in device memory, or NULL (all S keys valid).  With a preallocated cache
   * [B,Hkv,Smax,D] pass S = Smax and the filled lengths here: batch b attends to keys 0 .. min(kv_len[b], S) - 1, the
   * result the reference gives on K/V grown to that length with op::concat (reference
   * src/Operation/OpTransform.cpp:306-357).  A length of 0 yields zeros (the reference's empty contraction).
   * Served by the decode kernel, the pipelined head_dim-128 prefill kernel and the general kernel. */
  const int32_t* kv_len;
  /* Paged KV cache (optional; no counterpart in the reference).  block_table != NULL: k and v point to page pools
   * [num_pages, Hkv, page_size, D] and k_stride / v_stride are {page, head, row} strides; key j of batch b is row
   * j % page_size of page block_table[b * block_table_stride + j / page_size] (int32, device memory).  S is the
   * logical capacity: the table holds at least ceil(S / page_size) entries per batch entry, of which those below
   * ceil(kv_len[b] / page_size) are read.  page_size must be a power of two; the decode kernel takes pages of 32 rows
   * or more and the MFMA prefill kernels pages of 64 rows or more, smaller pages go to the general kernel. */
  const int32_t* block_table;
  int32_t page_size;
  int32_t block_table_stride;
} ttsdpa_params;

/* Library identification.  No counterpart in the reference (its device ops are linked statically). */
int ttsdpa_abi_version(void);
const char* ttsdpa_status_string(int status);

/* Fill *p for dense tensors: sizes, dense strides, scale = 1/sqrt(D) (reference src/Function/FuncNNLayer.h:235),
 * no mask, not causal, mask strides of a dense [L,S] mask.  Pointers are left NULL. */
void ttsdpa_params_init(ttsdpa_params* p, int dtype, int B, int Hq, int Hkv, int L, int S, int D);

/* Validate *p and report the kernel ttsdpa_forward would pick (enum ttsdpa_route) in *route.  Launches nothing and
 * needs no GPU.  Plays the role of the reference's shape checks before a device op (src/Operation/OpLinalg.cpp:62-89). */
int ttsdpa_plan(const ttsdpa_params* p, int* route);

/* Bytes of device scratch ttsdpa_forward / ttsdpa_decode use for *p (0 for calls that need none): the split-KV
 * partials of the decode route, and of calls on the prefill route whose keys are divided among workgroups (few query
 * rows, or few 256-row tiles of head_dim 128 against many keys).
 * The decode route refuses to run with less (TTSDPA_ERR_WORKSPACE); the prefill route then runs unsplit.
 * The reference's precedent for op-owned device scratch is src/Operation/OpNNLayerCuda.cuh:415. */
size_t ttsdpa_workspace_bytes(const ttsdpa_params* p);

/* The whole of FuncSDPAttention::forward (reference src/Function/FuncNNLayer.h:231-266, dropoutP == 0) on the GPU:
 * out = softmax(q.k^T * scale + bias) . v, enqueued on `stream` (a hipStream_t; NULL = the default stream).
 * Chooses the route of ttsdpa_plan. */
int ttsdpa_forward(const ttsdpa_params* p, void* workspace, size_t workspace_bytes, void* stream);

/* The three kernels individually (same contract; TTSDPA_ERR_UNSUPPORTED when *p is outside the kernel's domain).
 * ttsdpa_prefill replaces the reference's GEMM -> scale -> bias -> softmax -> GEMM chain for training/prefill shapes
 * (16-bit tensors on the 16-bit matrix cores with fp32 accumulation, fp32 tensors on the fp32 matrix cores);
 * ttsdpa_decode replaces it for one (or a few) query rows against a long contiguous KV cache;
 * ttsdpa_general covers everything else the reference op accepts (other head sizes, unaligned rows, masks on fp32 or short inputs). */
int ttsdpa_prefill(const ttsdpa_params* p, void* stream);
int ttsdpa_decode(const ttsdpa_params* p, void* workspace, size_t workspace_bytes, void* stream);

/* ttsdpa_decode for callers that cannot allocate (code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc).  No counterpart in the reference.  Same kernels and results as ttsdpa_decode, but the split-KV
 * partial records live in a buffer of TTSDPA_STATIC_SCRATCH_BYTES that is part of the library's device image (each GPU
 * the library runs on holds one until the process ends), so the call takes no workspace and allocates nothing; a
 * call whose ttsdpa_workspace_bytes() exceeds that size is refused with TTSDPA_ERR_STATIC_SCRATCH and launches
 * nothing.  The first call on a device looks the buffer's address up (make it outside graph capture).  All calls on
 * one GPU share the buffer: calls that may overlap on that GPU (different streams, several host threads) race on
 * it; calls on one stream are ordered and safe. */
#define TTSDPA_STATIC_SCRATCH_BYTES (2u << 20)
int ttsdpa_decode_static(const ttsdpa_params* p, void* stream);
int ttsdpa_general(const ttsdpa_params* p, void* stream);

/*
 * Backward of the attention call.  The reference declares it and stops there: FuncSDPAttention::backward is
 * NOT_IMPLEMENTED() (reference src/Function/FuncNNLayer.h:267), as is FuncMatmul::backward (src/Function/FuncLinalg.h:20),
 * so a model that attends cannot be trained with it.  This entry point is what that backward would call: for the
 * forward call `fwd` (same tensors, mask, causal mode and scale; fwd.out is the forward's result and is READ here) and
 * the upstream gradient dout [B,Hq,L,D] it writes dq [B,Hq,L,D], dk and dv [B,Hkv,S,D] — the chain rule through
 * matmul -> scale -> bias -> softmax -> matmul (src/Function/FuncNNLayer.h:237-265), with the reference's own softmax
 * backward step (src/Operation/OpNNLayerCpu.h:79-109).  dk / dv sum over the query heads of a KV head; rows of dk / dv
 * at or beyond kv_len[b] are written as zeros.  Gradients have the element type of the inputs; strides are in elements
 * {batch, head, sequence}, head_dim stride 1.  Paged caches (fwd.block_table) are not differentiated:
 * TTSDPA_ERR_UNSUPPORTED.  A query row whose keys are all hidden gets dq = 0 and adds nothing to dk / dv.
 * Scratch: ttsdpa_backward_workspace_bytes() bytes of device memory (per-row softmax statistics, and fp32 partial
 * gradients where a kernel needs them); TTSDPA_ERR_WORKSPACE with less.  No allocation, no synchronisation; results
 * do not depend on timing (no atomics).
 */
typedef struct ttsdpa_backward_params {
  uint32_t struct_size; /* sizeof(ttsdpa_backward_params) */
  uint32_t reserved;    /* 0 */
  ttsdpa_params fwd;
  const void* dout;
  void* dq;
  void* dk;
  void* dv;
  int64_t dout_stride[3];
  int64_t dq_stride[3];
  int64_t dk_stride[3];
  int64_t dv_stride[3];
} ttsdpa_backward_params;

/* Fill *p for dense tensors (ttsdpa_params_init for fwd, dense gradient strides); pointers NULL. */
void ttsdpa_backward_params_init(ttsdpa_backward_params* p, int dtype, int B, int Hq, int Hkv, int L, int S, int D);
/* Validate and report the kernels ttsdpa_backward would use: TTSDPA_ROUTE_PREFILL = the MFMA backward kernels
 * (fp16 / bf16 with head_dim a multiple of 8 up to 128, fp32 — on the fp32 matrix cores — with head_dim a multiple of 4
 * up to 128; 16-byte aligned rows; an attnMask must have contiguous, 4-aligned keys), TTSDPA_ROUTE_GENERAL = the
 * vector-ALU kernels, TTSDPA_ROUTE_NONE = nothing to compute.  Needs no GPU. */
int ttsdpa_backward_plan(const ttsdpa_backward_params* p, int* route);
size_t ttsdpa_backward_workspace_bytes(const ttsdpa_backward_params* p);
int ttsdpa_backward(const ttsdpa_backward_params* p, void* workspace, size_t workspace_bytes, void* stream);

/*
 * KV-cache append.  The reference has no KV cache: a caller that generates token by token grows K and V with
 * op::concat on the sequence axis (reference src/Operation/OpTransform.cpp:306-357), an O(S) copy per token.  Here the
 * caller preallocates k_cache / v_cache [B,Hkv,Smax,D] and this call writes the Lnew new rows of every (batch, kv head)
 * at rows pos .. pos+Lnew-1, where pos = positions[b] (int32[B], device memory) or `position` when positions is NULL.
 * Rows that would land at or beyond Smax are dropped.  Strides are in elements {batch, head, sequence}; head_dim stride
 * is 1.  Enqueued on `stream`; no allocation, no synchronisation.  The matching attention call passes the caches with
 * S = Smax and ttsdpa_params.kv_len = positions + Lnew.
 */
typedef struct ttsdpa_kv_append_params {
  uint32_t struct_size; /* sizeof(ttsdpa_kv_append_params) */
  int32_t dtype;        /* ttsdpa_dtype of all four tensors */
  void* k_cache;
  void* v_cache;
  const void* k_new;
  const void* v_new;
  int32_t B, Hkv, Smax, Lnew, D;
  int32_t position;
  int64_t kc_stride[3];
  int64_t vc_stride[3];
  int64_t kn_stride[3];
  int64_t vn_stride[3];
  const int32_t* positions;
  /* Paged caches: block_table != NULL makes k_cache / v_cache page pools [num_pages, Hkv, page_size, D] with
   * kc_stride / vc_stride = {page, head, row}; row pos of batch b goes to row pos % page_size of page
   * block_table[b * block_table_stride + pos / page_size].  Smax is the logical capacity per batch entry. */
  const int32_t* block_table;
  int32_t page_size;
  int32_t block_table_stride;
} ttsdpa_kv_append_params;

/* Fill *p for dense tensors (cache [B,Hkv,Smax,D], new rows [B,Hkv,Lnew,D]); pointers NULL, position 0. */
void ttsdpa_kv_append_params_init(ttsdpa_kv_append_params* p, int dtype, int B, int Hkv, int Smax, int Lnew, int D);
int ttsdpa_kv_append(const ttsdpa_kv_append_params* p, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TTSDPA_H */
