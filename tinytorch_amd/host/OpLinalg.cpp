#include "OpLinalg.h"

#include "../../include/ttlinear.h"
#include "Function.h"
#include "Macros.h"

namespace tinytorch::op {

namespace {

// The other transpose flag pairs of op::matmul for 2-D operands (reference src/Operation/OpLinalgCpu.h:119-150): a is
// [M, K], or [K, M] with transA; b is [K, N], or [N, K] with transB.  The first operand may carry leading batch axes when
// it is not transposed (they are part of M).
Tensor matmulFlagsGpuImpl(const Tensor& a, const Tensor& b, bool transA, bool transB, const Tensor& bias) {
  ASSERT(a.dim() >= 2 && b.dim() == 2 && (!transA || a.dim() == 2));
  ASSERT(b.dtype() == a.dtype() && b.device() == a.device());
  if (a.dim() < 2 || b.dim() != 2 || (transA && a.dim() != 2) || b.dtype() != a.dtype()) return {};
  const int64_t K = transA ? a.size(0) : a.size(-1);
  const int64_t N = transB ? b.size(0) : b.size(1);
  ASSERT((transB ? b.size(1) : b.size(0)) == K);
  if ((transB ? b.size(1) : b.size(0)) != K) return {};
  if (bias.defined()) {
    ASSERT(bias.dim() == 1 && bias.size(0) == N && bias.dtype() == a.dtype());
    if (bias.dim() != 1 || bias.size(0) != N || bias.dtype() != a.dtype()) return {};
  }
  std::vector<int64_t> shape;
  int64_t M = 1;
  if (transA) {
    M = a.size(1);
    shape = {M, N};
  } else {
    shape = a.shape();
    shape.back() = N;
    for (size_t i = 0; i + 1 < shape.size(); i++) M *= shape[i];
  }
  Tensor out = Tensor::empty(shape, a.options().noGrad());
  const int dtype = a.dtype() == DType::Float32 ? TTSDPA_F32 : a.dtype() == DType::Float16 ? TTSDPA_F16 : TTSDPA_BF16;
  const DeviceIndex dev = a.device().index;
  HIP_CHECK(hipSetDevice(dev));
  const size_t wsBytes = ttlinear_matmul_workspace_bytes(dtype, M, N, K, transA, transB);
  std::shared_ptr<Storage> ws;  // back to the allocator's cache on scope exit; the stream orders its reuse
  if (wsBytes) ws = std::make_shared<Storage>(wsBytes, a.device());
  const int rc = ttlinear_matmul(dtype, a.rawPtr(), b.rawPtr(), bias.defined() ? bias.rawPtr() : nullptr, out.rawPtr(), M, N, K,
                                 transA, transB, transA ? M : K, transB ? K : N, N, ws ? ws->data() : nullptr, wsBytes,
                                 getCurrentStream(dev));
  if (rc != TTSDPA_OK) {
    LOGE("ttlinear_matmul failed: %d (%s)", rc, ttsdpa_status_string(rc));
    ASSERT(rc == TTSDPA_OK);
    return {};
  }
  return out;
}

// op::matmul in its general form (reference src/Operation/OpLinalg.cpp:52-241): 1-D operands become a row / a column
// vector (their flags ignored), leading dimensions broadcast against each other, every batch entry is one 2-D product
// (ttlinear_matmul_batched), and the dimensions added for 1-D operands are dropped from a 2-D result.
Tensor matmulNdGpuImpl(const Tensor& a, const Tensor& b, bool transA, bool transB, const Tensor& bias) {
  ASSERT(a.dim() >= 1 && b.dim() >= 1 && b.dtype() == a.dtype() && b.device() == a.device());
  if (a.dim() < 1 || b.dim() < 1 || b.dtype() != a.dtype()) return {};
  std::vector<int64_t> sa = a.shape(), sb = b.shape();
  const bool prependA = sa.size() == 1, appendB = sb.size() == 1;
  if (prependA) sa.insert(sa.begin(), 1), transA = false;
  if (appendB) sb.push_back(1), transB = false;
  const int64_t m = transA ? sa.back() : sa[sa.size() - 2], k = transA ? sa[sa.size() - 2] : sa.back();
  const int64_t kb = transB ? sb.back() : sb[sb.size() - 2], n = transB ? sb[sb.size() - 2] : sb.back();
  ASSERT(k == kb && "matmul error: shape not aligned");
  if (k != kb) return {};
  if (bias.defined()) {
    ASSERT(bias.dim() == 1 && bias.size(0) == n && bias.dtype() == a.dtype());
    if (bias.dim() != 1 || bias.size(0) != n || bias.dtype() != a.dtype()) return {};
  }
  // batch dimensions, right-aligned; element strides of the dense operands, 0 where an operand is broadcast
  const size_t na = sa.size() - 2, nb = sb.size() - 2, nd = na > nb ? na : nb;
  ASSERT(nd <= TTLINEAR_MAX_BATCH_DIMS);
  if (nd > TTLINEAR_MAX_BATCH_DIMS) return {};
  std::vector<int64_t> batch(nd), strA(nd, 0), strB(nd, 0);
  int64_t runA = sa[sa.size() - 2] * sa.back(), runB = sb[sb.size() - 2] * sb.back();
  for (size_t r = 0; r < nd; r++) {  // r counts from the innermost batch dimension
    const int64_t da = r < na ? sa[na - 1 - r] : 1, db = r < nb ? sb[nb - 1 - r] : 1;
    ASSERT((da == db || da == 1 || db == 1) && "matmul error: shape not aligned");
    if (da != db && da != 1 && db != 1) return {};
    batch[nd - 1 - r] = da > db ? da : db;
    if (r < na) {
      strA[nd - 1 - r] = da > 1 ? runA : 0;
      runA *= da;
    }
    if (r < nb) {
      strB[nd - 1 - r] = db > 1 ? runB : 0;
      runB *= db;
    }
  }
  // A 1-D second operand against a first operand with batch dimensions: the reference reshapes the [..., m, 1] result to
  // {m} (src/Operation/OpLinalg.cpp:196-200, :232-238), which its element count does not fit.  No result shape is defined:
  // refused, as the Python mirror does.
  ASSERT(!(appendB && nd > 0) && "matmul error: a 1-D second operand against a batched first operand has no result shape");
  if (appendB && nd > 0) return {};
  std::vector<int64_t> shape = batch;
  shape.push_back(m);
  shape.push_back(n);
  Tensor out = Tensor::empty(shape, a.options().noGrad());
  const int dtype = a.dtype() == DType::Float32 ? TTSDPA_F32 : a.dtype() == DType::Float16 ? TTSDPA_F16 : TTSDPA_BF16;
  const DeviceIndex dev = a.device().index;
  HIP_CHECK(hipSetDevice(dev));
  const size_t wsBytes = ttlinear_matmul_workspace_bytes(dtype, m, n, k, transA, transB);
  std::shared_ptr<Storage> ws;
  if (wsBytes) ws = std::make_shared<Storage>(wsBytes, a.device());
  const int rc = ttlinear_matmul_batched(dtype, a.rawPtr(), b.rawPtr(), bias.defined() ? bias.rawPtr() : nullptr, out.rawPtr(), m, n,
                                         k, transA, transB, sa.back(), sb.back(), n, (int)nd, batch.data(), strA.data(),
                                         strB.data(), m * n, ws ? ws->data() : nullptr, wsBytes, getCurrentStream(dev));
  if (rc != TTSDPA_OK) {
    LOGE("ttlinear_matmul_batched failed: %d (%s)", rc, ttsdpa_status_string(rc));
    ASSERT(rc == TTSDPA_OK);
    return {};
  }
  if (nd == 0) {  // reference :221-239
    if (appendB)
      out.reshape_(prependA ? std::vector<int64_t>{} : std::vector<int64_t>{m});
    else if (prependA)
      out.reshape_({n});
  }
  return out;
}

Tensor matmulGpuImpl(const Tensor& a, const Tensor& b, bool transA, bool transB, const Tensor& bias) {
  ASSERT(a.defined() && b.defined());
  if (!a.defined() || !b.defined()) return {};
  // a second operand with batch dimensions, a transposed first operand with them, or a 1-D operand: the general form
  if (b.dim() != 2 || a.dim() < 2 || (transA && a.dim() != 2)) return matmulNdGpuImpl(a, b, transA, transB, bias);
  if (transA || !transB) return matmulFlagsGpuImpl(a, b, transA, transB, bias);
  ASSERT(a.dim() >= 1 && b.dim() == 2 && a.size(-1) == b.size(1));
  ASSERT(b.dtype() == a.dtype() && b.device() == a.device());
  if (!a.defined() || !b.defined() || transA || !transB || a.dim() < 1 || b.dim() != 2 || a.size(-1) != b.size(1) ||
      b.dtype() != a.dtype())
    return {};
  const int64_t K = b.size(1), N = b.size(0);
  if (bias.defined()) {
    ASSERT(bias.dim() == 1 && bias.size(0) == N && bias.dtype() == a.dtype());  // reference src/Operation/OpLinalg.cpp:262
    if (bias.dim() != 1 || bias.size(0) != N || bias.dtype() != a.dtype()) return {};
  }
  std::vector<int64_t> shape = a.shape();
  shape.back() = N;
  int64_t M = 1;
  for (size_t i = 0; i + 1 < shape.size(); i++) M *= shape[i];
  Tensor out = Tensor::empty(shape, a.options().noGrad());
  const int dtype = a.dtype() == DType::Float32 ? TTSDPA_F32 : a.dtype() == DType::Float16 ? TTSDPA_F16 : TTSDPA_BF16;
  const DeviceIndex dev = a.device().index;
  HIP_CHECK(hipSetDevice(dev));
  const int rc = ttlinear_forward(dtype, a.rawPtr(), b.rawPtr(), bias.defined() ? bias.rawPtr() : nullptr, out.rawPtr(), M, N, K,
                                  K, K, N, getCurrentStream(dev));
  if (rc != TTSDPA_OK) {
    LOGE("ttlinear_forward failed: %d (%s)", rc, ttsdpa_status_string(rc));
    ASSERT(rc == TTSDPA_OK);
    return {};
  }
  return out;
}

}  // namespace

void registerLinalgGpu() {
  REGISTER_OP_IMPL(matmul, GPU, Float32, &matmulGpuImpl);
  REGISTER_OP_IMPL(matmul, GPU, Float16, &matmulGpuImpl);
  REGISTER_OP_IMPL(matmul, GPU, BFloat16, &matmulGpuImpl);
}

}  // namespace tinytorch::op
