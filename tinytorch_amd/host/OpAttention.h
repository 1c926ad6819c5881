// Tensor-level attention op, declared and registered the way the reference adds a fused op (DEFINE_OP +
// REGISTER_OP_IMPL per {device, dtype}; precedent reference src/Operation/OpFused.h:14-32, OpFusedCuda.cu:11-22).
// The reference has no such op: its FuncSDPAttention::forward composes ~11 generic ops
// (src/Function/FuncNNLayer.h:231-266).  Here the GPU slot of the table holds one implementation that hands the
// whole forward to the C ABI of include/ttsdpa.h.  The CPU slot is deliberately empty: a CPU tensor reaching this op
// fails loudly through the dispatcher instead of taking another route.
#pragma once

#include "Dispatch.h"

namespace tinytorch::op {

// query [B,Hq,L,D] (or [Hq,L,D]); key/value [B,Hkv,S,D] with Hq a multiple of Hkv (query head h reads KV head
// h / (Hq/Hkv); Hkv == Hq is the reference's layout).  isCausal is top-left aligned, exclusive with attnMask.
// attnMask: undefined, Bool [L,S] (false = hidden) or the query dtype [L,S] (added to the scores).
// dropoutP must be 0.  Returns [B,Hq,L,D] in the query dtype, or an undefined Tensor after a failed ASSERT.
using SdpAttentionOpFn = Tensor (*)(const Tensor& query, const Tensor& key, const Tensor& value, bool isCausal,
                                    const Tensor& attnMask, float dropoutP, float scale);

DEFINE_OP(sdpAttention, SdpAttentionOpFn)

// Gradients {dQuery, dKey, dValue} of op::sdpAttention(query, key, value, isCausal, attnMask, 0, scale) for the upstream
// gradient gradOut; `out` is that call's result.  dKey / dValue have the shapes of key / value (grouped heads are
// summed).  The reference stops at NOT_IMPLEMENTED here (src/Function/FuncNNLayer.h:267).  Empty vector after a failed
// ASSERT.
using SdpAttentionBackwardOpFn = std::vector<Tensor> (*)(const Tensor& gradOut, const Tensor& query, const Tensor& key,
                                                         const Tensor& value, const Tensor& out, bool isCausal,
                                                         const Tensor& attnMask, float scale);
DEFINE_OP(sdpAttentionBackward, SdpAttentionBackwardOpFn)

// KV cache (no counterpart in the reference, whose callers would grow K/V with op::concat on the sequence axis,
// src/Operation/OpTransform.cpp:306-357, copying the whole history per generated token).
// kvCacheAppend writes kNew/vNew [B,Hkv,Lnew,D] into the preallocated caches [B,Hkv,Smax,D] in place, at rows
// positions[b] .. +Lnew-1 (positions: Int32 [B] on the device; undefined = `position` for every batch entry); rows
// that do not fit are dropped.  sdpAttentionCached attends query [B,Hq,L,D] to the first kvLens[b] rows of the caches
// (kvLens: Int32 [B] on the device), no mask.  isCausal here means: the L query rows are the last L positions of each
// batch entry's kvLens[b] keys (their K/V already appended) and row i sees the keys up to its own position,
// kvLens[b] - L + i — a chunk of a prompt, or several speculated tokens; one new token (L == 1) sees every key either way.
// blockTable (Int32 [B, n] on the device, or undefined): the caches are page pools [pages,Hkv,pageSize,D] and key j of
// batch entry b is row j % pageSize of page blockTable[b][j / pageSize]; pageSize is a power of two.
using KvCacheAppendOpFn = void (*)(const Tensor& kCache, const Tensor& vCache, const Tensor& kNew, const Tensor& vNew,
                                   const Tensor& positions, int32_t position, const Tensor& blockTable);
using SdpAttentionCachedOpFn = Tensor (*)(const Tensor& query, const Tensor& kCache, const Tensor& vCache,
                                          const Tensor& kvLens, bool isCausal, float scale, const Tensor& blockTable);
DEFINE_OP(kvCacheAppend, KvCacheAppendOpFn)
DEFINE_OP(sdpAttentionCached, SdpAttentionCachedOpFn)

void registerAttentionGpu();
STATIC_CALL(registerAttentionGpu);

}  // namespace tinytorch::op
