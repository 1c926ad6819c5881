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

// GPU entry of op::sdpAttention for every floating dtype: one enqueue on the thread's current stream, output and
// scratch from the caching allocator, no host synchronisation.
Tensor sdpAttentionGpuImpl(const Tensor& query, const Tensor& key, const Tensor& value, bool isCausal,
                           const Tensor& attnMask, float dropoutP, float scale) {
  ASSERT(query.defined() && key.defined() && value.defined());
  ASSERT(query.dim() == key.dim() && key.dim() == value.dim() && (query.dim() == 4 || query.dim() == 3));
  ASSERT(key.dtype() == query.dtype() && value.dtype() == query.dtype());
  ASSERT(key.device() == query.device() && value.device() == query.device());
  ASSERT(dropoutP == 0.f);  // the fused path has no dropout (the reference's composite passes p through inverted)
  ASSERT(!(isCausal && attnMask.defined()));  // reference src/Function/FuncNNLayer.h:242
  if (query.dim() != key.dim() || dropoutP != 0.f || (isCausal && attnMask.defined())) return {};

  const int nd = static_cast<int>(query.dim());
  const int B = nd == 4 ? static_cast<int>(query.size(0)) : 1;
  const int Hq = static_cast<int>(query.size(-3)), Hkv = static_cast<int>(key.size(-3));
  const int L = static_cast<int>(query.size(-2)), S = static_cast<int>(key.size(-2));
  const int D = static_cast<int>(query.size(-1));
  ASSERT(key.shape() == value.shape() && key.size(-1) == D && Hkv >= 1 && Hq % Hkv == 0);
  ASSERT(nd == 3 || key.size(0) == B);
  if (key.shape() != value.shape() || key.size(-1) != D || Hkv < 1 || Hq % Hkv != 0) return {};

  ttsdpa_params p;
  ttsdpa_params_init(&p, dtypeCode(query.dtype()), B, Hq, Hkv, L, S, D);
  Tensor out = Tensor::empty(query.shape(), query.options().noGrad());
  p.q = query.rawPtr(), p.k = key.rawPtr(), p.v = value.rawPtr(), p.out = out.rawPtr();
  p.scale = scale;
  p.causal = isCausal ? 1 : 0;
  if (attnMask.defined()) {
    ASSERT(attnMask.device() == query.device());
    ASSERT(attnMask.dtype() == DType::Bool || attnMask.dtype() == query.dtype());
    // Any shape that broadcasts to [B,Hq,L,S], as the reference's broadcasting add of the bias accepts
    // (src/Function/FuncNNLayer.h:249-260): right-align the mask's axes, size-1 and missing axes get stride 0.
    const int md = static_cast<int>(attnMask.dim());
    ASSERT(md >= 1 && md <= 4);
    if (md < 1 || md > 4) return {};
    const int64_t target[4] = {B, Hq, L, S};
    int64_t dense = 1;
    for (int i = 3; i >= 0; i--) {
      const int mi = i - (4 - md);
      const int64_t n = mi >= 0 ? attnMask.size(mi) : 1;
      ASSERT(n == target[i] || n == 1);
      if (n != target[i] && n != 1) return {};
      p.mask_stride[i] = n == 1 ? 0 : dense;
      dense *= n;
    }
    p.mask_kind = attnMask.dtype() == DType::Bool ? TTSDPA_MASK_BOOL : TTSDPA_MASK_ADD;
    p.mask = attnMask.rawPtr();
  }

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

}  // namespace

void registerAttentionGpu() {
  REGISTER_OP_IMPL(sdpAttention, GPU, Float32, &sdpAttentionGpuImpl);
  REGISTER_OP_IMPL(sdpAttention, GPU, Float16, &sdpAttentionGpuImpl);
  REGISTER_OP_IMPL(sdpAttention, GPU, BFloat16, &sdpAttentionGpuImpl);
}

}  // namespace tinytorch::op
