#include "OpAttention.h"

#include <hip/hip_runtime.h>

#include "../../include/ttsdpa.h"
#include "Function.h"

namespace tinytorch::op {

namespace {

int dtypeCode(DType t) {
  switch (t) {
    case DType::Float32: return TTSDPA_F32;
    case DType::Float16: return TTSDPA_F16;
    default: return TTSDPA_BF16;
  }
}

// Checks the arguments of an attention call and fills *p for dense tensors (pointers of q, k, v and the mask; p->out
// is left to the caller).  false after a failed precondition.
bool fillAttentionParams(ttsdpa_params* pp, const Tensor& query, const Tensor& key, const Tensor& value, bool isCausal,
                         const Tensor& attnMask, float dropoutP, float scale) {
  ttsdpa_params& p = *pp;
  ASSERT(query.defined() && key.defined() && value.defined());
  ASSERT(query.dim() == key.dim() && key.dim() == value.dim() && (query.dim() == 4 || query.dim() == 3));
  ASSERT(key.dtype() == query.dtype() && value.dtype() == query.dtype());
  ASSERT(key.device() == query.device() && value.device() == query.device());
  ASSERT(dropoutP == 0.f);  // the fused path has no dropout (the reference's composite passes p through inverted)
  ASSERT(!(isCausal && attnMask.defined()));  // reference src/Function/FuncNNLayer.h:242
  if (query.dim() != key.dim() || dropoutP != 0.f || (isCausal && attnMask.defined())) return false;

  const int nd = static_cast<int>(query.dim());
  const int B = nd == 4 ? static_cast<int>(query.size(0)) : 1;
  const int Hq = static_cast<int>(query.size(-3)), Hkv = static_cast<int>(key.size(-3));
  const int L = static_cast<int>(query.size(-2)), S = static_cast<int>(key.size(-2));
  const int D = static_cast<int>(query.size(-1));
  ASSERT(key.shape() == value.shape() && key.size(-1) == D && Hkv >= 1 && Hq % Hkv == 0);
  ASSERT(nd == 3 || key.size(0) == B);
  if (key.shape() != value.shape() || key.size(-1) != D || Hkv < 1 || Hq % Hkv != 0) return false;

  ttsdpa_params_init(&p, dtypeCode(query.dtype()), B, Hq, Hkv, L, S, D);
  p.q = query.rawPtr(), p.k = key.rawPtr(), p.v = value.rawPtr();
  p.scale = scale;
  p.causal = isCausal ? TTSDPA_CAUSAL_TOP_LEFT : TTSDPA_CAUSAL_NONE;  // the reference's alignment
  if (attnMask.defined()) {
    ASSERT(attnMask.device() == query.device());
    ASSERT(attnMask.dtype() == DType::Bool || attnMask.dtype() == query.dtype());
    // Any shape that broadcasts to [B,Hq,L,S], as the reference's broadcasting add of the bias accepts
    // (src/Function/FuncNNLayer.h:249-260): right-align the mask's axes, size-1 and missing axes get stride 0.
    const int md = static_cast<int>(attnMask.dim());
    ASSERT(md >= 1 && md <= 4);
    if (md < 1 || md > 4) return false;
    const int64_t target[4] = {B, Hq, L, S};
    int64_t dense = 1;
    for (int i = 3; i >= 0; i--) {
      const int mi = i - (4 - md);
      const int64_t n = mi >= 0 ? attnMask.size(mi) : 1;
      ASSERT(n == target[i] || n == 1);
      if (n != target[i] && n != 1) return false;
      p.mask_stride[i] = n == 1 ? 0 : dense;
      dense *= n;
    }
    p.mask_kind = attnMask.dtype() == DType::Bool ? TTSDPA_MASK_BOOL : TTSDPA_MASK_ADD;
    p.mask = attnMask.rawPtr();
  }
  return true;
}

// GPU entry of op::sdpAttention for every floating dtype: one enqueue on the thread's current stream, output and
// scratch from the caching allocator, no host synchronisation.
Tensor sdpAttentionGpuImpl(const Tensor& query, const Tensor& key, const Tensor& value, bool isCausal,
                           const Tensor& attnMask, float dropoutP, float scale) {
  ttsdpa_params p;
  if (!fillAttentionParams(&p, query, key, value, isCausal, attnMask, dropoutP, scale)) return {};
  Tensor out = Tensor::empty(query.shape(), query.options().noGrad());
  p.out = out.rawPtr();
  const DeviceIndex dev = query.device().index;
  HIP_CHECK(hipSetDevice(dev));
  const size_t wsBytes = ttsdpa_workspace_bytes(&p);
  std::shared_ptr<Storage> ws;  // returned to the allocator's cache on scope exit; the stream orders its reuse
  if (wsBytes) ws = std::make_shared<Storage>(wsBytes, query.device());
  const int rc = ttsdpa_forward(&p, ws ? ws->data() : nullptr, wsBytes, getCurrentStream(dev));
  if (rc != TTSDPA_OK) {
    LOGE("ttsdpa_forward failed: %d (%s)", rc, ttsdpa_status_string(rc));
    ASSERT(rc == TTSDPA_OK);
    return {};
  }
  return out;
}

// GPU entry of op::sdpAttentionBackward: {dq, dk, dv} for the forward call with the same arguments, whose result is
// `out`.  One enqueue of two kernels on the thread's current stream; gradients and scratch from the caching allocator.
std::vector<Tensor> sdpAttentionBackwardGpuImpl(const Tensor& gradOut, const Tensor& query, const Tensor& key,
                                                const Tensor& value, const Tensor& out, bool isCausal,
                                                const Tensor& attnMask, float scale) {
  ttsdpa_backward_params bp;
  ASSERT(gradOut.defined() && out.defined());
  if (!gradOut.defined() || !out.defined()) return {};
  if (!fillAttentionParams(&bp.fwd, query, key, value, isCausal, attnMask, 0.f, scale)) return {};
  ASSERT(gradOut.shape() == query.shape() && out.shape() == query.shape());
  ASSERT(gradOut.dtype() == query.dtype() && out.dtype() == query.dtype());
  ASSERT(gradOut.device() == query.device() && out.device() == query.device());
  if (gradOut.shape() != query.shape() || out.shape() != query.shape() || gradOut.dtype() != query.dtype() ||
      out.dtype() != query.dtype())
    return {};
  const ttsdpa_params fwd = bp.fwd;
  ttsdpa_backward_params_init(&bp, fwd.dtype, fwd.B, fwd.Hq, fwd.Hkv, fwd.L, fwd.S, fwd.D);
  bp.fwd = fwd;
  bp.fwd.out = out.rawPtr();
  Tensor dq = Tensor::empty(query.shape(), query.options().noGrad());
  Tensor dk = Tensor::empty(key.shape(), key.options().noGrad());
  Tensor dv = Tensor::empty(value.shape(), value.options().noGrad());
  bp.dout = gradOut.rawPtr(), bp.dq = dq.rawPtr(), bp.dk = dk.rawPtr(), bp.dv = dv.rawPtr();
  const DeviceIndex dev = query.device().index;
  HIP_CHECK(hipSetDevice(dev));
  const size_t wsBytes = ttsdpa_backward_workspace_bytes(&bp);
  std::shared_ptr<Storage> ws;
  if (wsBytes) ws = std::make_shared<Storage>(wsBytes, query.device());
  const int rc = ttsdpa_backward(&bp, ws ? ws->data() : nullptr, wsBytes, getCurrentStream(dev));
  if (rc != TTSDPA_OK) {
    LOGE("ttsdpa_backward failed: %d (%s)", rc, ttsdpa_status_string(rc));
    ASSERT(rc == TTSDPA_OK);
    return {};
  }
  return {dq, dk, dv};
}

// Fills the block-table fields of a parameter struct; false after a failed precondition.
template <typename P>
bool setBlockTable(P& p, const Tensor& blockTable, const Tensor& pool, int64_t B) {
  ASSERT(blockTable.dtype() == DType::Int32 && blockTable.dim() == 2 && blockTable.size(0) == B &&
         blockTable.device() == pool.device());
  if (blockTable.dtype() != DType::Int32 || blockTable.dim() != 2 || blockTable.size(0) != B) return false;
  p.block_table = static_cast<const int32_t*>(blockTable.rawPtr());
  p.page_size = static_cast<int32_t>(pool.size(2));
  p.block_table_stride = static_cast<int32_t>(blockTable.size(1));
  return true;
}

void kvCacheAppendGpuImpl(const Tensor& kCache, const Tensor& vCache, const Tensor& kNew, const Tensor& vNew,
                          const Tensor& positions, int32_t position, const Tensor& blockTable) {
  ASSERT(kCache.defined() && vCache.defined() && kNew.defined() && vNew.defined());
  ASSERT(kCache.dim() == 4 && kNew.dim() == 4 && kCache.shape() == vCache.shape() && kNew.shape() == vNew.shape());
  const bool paged = blockTable.defined();
  ASSERT((paged || kNew.size(0) == kCache.size(0)) && kNew.size(1) == kCache.size(1) && kNew.size(3) == kCache.size(3));
  ASSERT(vCache.dtype() == kCache.dtype() && kNew.dtype() == kCache.dtype() && vNew.dtype() == kCache.dtype());
  ASSERT(vCache.device() == kCache.device() && kNew.device() == kCache.device() && vNew.device() == kCache.device());
  if (kCache.dim() != 4 || kNew.dim() != 4 || kCache.shape() != vCache.shape() || kNew.shape() != vNew.shape()) return;
  if ((!paged && kNew.size(0) != kCache.size(0)) || kNew.size(1) != kCache.size(1) || kNew.size(3) != kCache.size(3)) return;
  const int64_t B = kNew.size(0);
  const int64_t capacity = paged && blockTable.dim() == 2 ? blockTable.size(1) * kCache.size(2) : kCache.size(2);
  ttsdpa_kv_append_params p;
  ttsdpa_kv_append_params_init(&p, dtypeCode(kCache.dtype()), static_cast<int>(B), static_cast<int>(kCache.size(1)),
                               static_cast<int>(capacity), static_cast<int>(kNew.size(2)),
                               static_cast<int>(kCache.size(3)));
  if (paged) {  // the pool's strides are {page, head, row}
    p.kc_stride[0] = p.vc_stride[0] = kCache.size(1) * kCache.size(2) * kCache.size(3);
    p.kc_stride[1] = p.vc_stride[1] = kCache.size(2) * kCache.size(3);
    if (!setBlockTable(p, blockTable, kCache, B)) return;
  }
  p.k_cache = kCache.rawPtr(), p.v_cache = vCache.rawPtr(), p.k_new = kNew.rawPtr(), p.v_new = vNew.rawPtr();
  p.position = position;
  if (positions.defined()) {
    ASSERT(positions.dtype() == DType::Int32 && positions.numel() == B && positions.device() == kCache.device());
    if (positions.dtype() != DType::Int32 || positions.numel() != B) return;
    p.positions = static_cast<const int32_t*>(positions.rawPtr());
  }
  const DeviceIndex dev = kCache.device().index;
  HIP_CHECK(hipSetDevice(dev));
  const int rc = ttsdpa_kv_append(&p, getCurrentStream(dev));
  if (rc != TTSDPA_OK) {
    LOGE("ttsdpa_kv_append failed: %d (%s)", rc, ttsdpa_status_string(rc));
    ASSERT(rc == TTSDPA_OK);
  }
}

Tensor sdpAttentionCachedGpuImpl(const Tensor& query, const Tensor& kCache, const Tensor& vCache, const Tensor& kvLens,
                                 bool isCausal, float scale, const Tensor& blockTable) {
  const bool paged = blockTable.defined();
  ASSERT(query.defined() && kCache.defined() && vCache.defined() && kvLens.defined());
  ASSERT(query.dim() == 4 && kCache.dim() == 4 && kCache.shape() == vCache.shape());
  ASSERT((paged || kCache.size(0) == query.size(0)) && kCache.size(3) == query.size(3) && query.size(1) % kCache.size(1) == 0);
  ASSERT(kCache.dtype() == query.dtype() && vCache.dtype() == query.dtype());
  ASSERT(kvLens.dtype() == DType::Int32 && kvLens.numel() == query.size(0) && kvLens.device() == query.device());
  if (query.dim() != 4 || kCache.dim() != 4 || kCache.shape() != vCache.shape() || (!paged && kCache.size(0) != query.size(0)) ||
      kCache.size(3) != query.size(3) || query.size(1) % kCache.size(1) != 0 || kvLens.dtype() != DType::Int32 ||
      kvLens.numel() != query.size(0))
    return {};
  ttsdpa_params p;
  ttsdpa_params_init(&p, dtypeCode(query.dtype()), static_cast<int>(query.size(0)), static_cast<int>(query.size(1)),
                     static_cast<int>(kCache.size(1)), static_cast<int>(query.size(2)),
                     static_cast<int>(paged && blockTable.dim() == 2 ? blockTable.size(1) * kCache.size(2) : kCache.size(2)),
                     static_cast<int>(query.size(3)));
  if (paged) {  // the pool's strides are {page, head, row}
    p.k_stride[0] = p.v_stride[0] = kCache.size(1) * kCache.size(2) * kCache.size(3);
    p.k_stride[1] = p.v_stride[1] = kCache.size(2) * kCache.size(3);
    if (!setBlockTable(p, blockTable, kCache, query.size(0))) return {};
  }
  Tensor out = Tensor::empty(query.shape(), query.options().noGrad());
  p.q = query.rawPtr(), p.k = kCache.rawPtr(), p.v = vCache.rawPtr(), p.out = out.rawPtr();
  p.scale = scale;
  p.causal = isCausal ? TTSDPA_CAUSAL_BOTTOM_RIGHT : TTSDPA_CAUSAL_NONE;
  p.kv_len = static_cast<const int32_t*>(kvLens.rawPtr());
  const DeviceIndex dev = query.device().index;
  HIP_CHECK(hipSetDevice(dev));
  const size_t wsBytes = ttsdpa_workspace_bytes(&p);
  std::shared_ptr<Storage> ws;
  if (wsBytes) ws = std::make_shared<Storage>(wsBytes, query.device());
  const int rc = ttsdpa_forward(&p, ws ? ws->data() : nullptr, wsBytes, getCurrentStream(dev));
  if (rc != TTSDPA_OK) {
    LOGE("ttsdpa_forward failed: %d (%s)", rc, ttsdpa_status_string(rc));
    ASSERT(rc == TTSDPA_OK);
    return {};
  }
  return out;
}

}  // namespace

void registerAttentionGpu() {
  REGISTER_OP_IMPL(sdpAttention, GPU, Float32, &sdpAttentionGpuImpl);
  REGISTER_OP_IMPL(sdpAttention, GPU, Float16, &sdpAttentionGpuImpl);
  REGISTER_OP_IMPL(sdpAttention, GPU, BFloat16, &sdpAttentionGpuImpl);
  REGISTER_OP_IMPL(sdpAttentionBackward, GPU, Float32, &sdpAttentionBackwardGpuImpl);
  REGISTER_OP_IMPL(sdpAttentionBackward, GPU, Float16, &sdpAttentionBackwardGpuImpl);
  REGISTER_OP_IMPL(sdpAttentionBackward, GPU, BFloat16, &sdpAttentionBackwardGpuImpl);
  REGISTER_OP_IMPL(kvCacheAppend, GPU, Float32, &kvCacheAppendGpuImpl);
  REGISTER_OP_IMPL(kvCacheAppend, GPU, Float16, &kvCacheAppendGpuImpl);
  REGISTER_OP_IMPL(kvCacheAppend, GPU, BFloat16, &kvCacheAppendGpuImpl);
  REGISTER_OP_IMPL(sdpAttentionCached, GPU, Float32, &sdpAttentionCachedGpuImpl);
  REGISTER_OP_IMPL(sdpAttentionCached, GPU, Float16, &sdpAttentionCachedGpuImpl);
  REGISTER_OP_IMPL(sdpAttentionCached, GPU, BFloat16, &sdpAttentionCachedGpuImpl);
}

}  // namespace tinytorch::op
