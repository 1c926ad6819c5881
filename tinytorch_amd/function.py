"""Host-side mirror of TinyTorch's attention interface for torch device tensors.

``sdpAttention`` keeps the name, argument order, defaults and error behaviour of
``tinytorch::function::sdpAttention`` (reference src/Function/FuncNNLayer.h:298-302) and of
``FuncSDPAttention::forward`` (:231-266); the work itself is one call through the C ABI of include/ttsdpa.h.
torch is only the owner of device memory and of the current stream here.
"""
import ctypes
import math

import torch

from . import _capi

_DTYPES = {torch.float32: _capi.F32, torch.float16: _capi.F16, torch.bfloat16: _capi.BF16}


def _workspace(device, nbytes):
    """Device scratch of one call, taken from torch's caching allocator as the reference's ops take theirs from its own
    (src/Operation/OpNNLayerCuda.cuh:415).  A buffer per call, not one kept per device: the allocator orders reuse by
    stream and keeps allocations made under graph capture in the graph's pool, so a captured call keeps its scratch for
    every replay and calls on different streams never share partial results."""
    return torch.empty(max(int(nbytes), 16), dtype=torch.uint8, device=device)


def _strides3(t):
    assert t.stride(-1) == 1 or t.size(-1) == 1
    return (t.stride(0), t.stride(1), t.stride(2))


_CAUSAL_ALIGN = {"top-left": _capi.CAUSAL_TOP_LEFT, "bottom-right": _capi.CAUSAL_BOTTOM_RIGHT}


def _check_block_table(name, blockTable, B, device):
    if blockTable.dtype != torch.int32 or blockTable.dim() != 2 or blockTable.shape[0] != B \
            or blockTable.stride(1) != 1 or blockTable.device != device:
        raise ValueError("%s: blockTable must be an int32 [B, pages per entry] tensor on the device of the tensors" % name)


def build_params(query, key, value, out, isCausal=False, attnMask=None, scale=None, kvLens=None, causalAlign="top-left",
                 blockTable=None):
    """Fill a ttsdpa_params for 4-D tensors [B,H,N,D] (with blockTable: key/value are page pools [pages,Hkv,page,D])."""
    B, Hq, L, D = query.shape
    Bk, Hkv, S, Dk = key.shape
    if blockTable is not None:
        _check_block_table("sdpAttention", blockTable, B, query.device)
        page = S
        if page < 1 or page & (page - 1):
            raise ValueError("sdpAttention: the page size (%d rows) must be a power of two" % page)
        Bk, S = B, blockTable.shape[1] * page  # logical capacity per batch entry
    if value.shape != key.shape or Bk != B or Dk != D:
        raise ValueError("sdpAttention: key/value shape %s / %s do not match query %s"
                         % (tuple(key.shape), tuple(value.shape), tuple(query.shape)))
    if Hkv < 1 or Hq % Hkv != 0:
        raise ValueError("sdpAttention: %d query heads cannot share %d key/value heads" % (Hq, Hkv))
    if query.dtype not in _DTYPES or key.dtype != query.dtype or value.dtype != query.dtype:
        raise TypeError("sdpAttention: dtype must be one of float32/float16/bfloat16 and equal for q, k, v")
    p = _capi.make_params(_DTYPES[query.dtype], B, Hq, Hkv, L, S, D)
    p.q, p.k, p.v, p.out = query.data_ptr(), key.data_ptr(), value.data_ptr(), out.data_ptr()
    for name, t in (("q_stride", query), ("k_stride", key), ("v_stride", value), ("o_stride", out)):
        st = _strides3(t)
        for i in range(3):
            getattr(p, name)[i] = st[i]
    p.scale = float(scale) if scale is not None else 1.0 / math.sqrt(float(D))
    if causalAlign not in _CAUSAL_ALIGN:
        raise ValueError("sdpAttention: causalAlign must be 'top-left' or 'bottom-right'")
    p.causal = _CAUSAL_ALIGN[causalAlign] if isCausal else _capi.CAUSAL_NONE
    if attnMask is not None:
        if isCausal:
            raise ValueError("sdpAttention: isCausal and attnMask are exclusive")  # reference FuncNNLayer.h:242
        if attnMask.device != query.device:  # its address goes to the kernels as is: a host pointer would fault the GPU
            raise RuntimeError("sdpAttention: attnMask must live on the device of the tensors (got %s, tensors on %s)"
                               % (attnMask.device, query.device))
        if attnMask.dim() > 4:
            raise ValueError("sdpAttention: attnMask must broadcast to [B, H, L, S]")
        try:  # the reference adds the mask with a broadcasting add (FuncNNLayer.h:249-260)
            full = attnMask.expand(B, Hq, L, S)  # a view: broadcast axes get stride 0
        except RuntimeError:
            raise ValueError("sdpAttention: attnMask %s does not broadcast to [%d, %d, %d, %d]"
                             % (tuple(attnMask.shape), B, Hq, L, S))
        if attnMask.dtype == torch.bool:
            p.mask_kind = _capi.MASK_BOOL
        elif attnMask.dtype == query.dtype:
            p.mask_kind = _capi.MASK_ADD
        else:
            raise TypeError("sdpAttention: attnMask must be bool or of the query dtype")
        p.mask = attnMask.data_ptr()
        for i in range(4):
            p.mask_stride[i] = full.stride(i) if full.size(i) > 1 else 0
    if kvLens is not None:
        if kvLens.dtype != torch.int32 or kvLens.dim() != 1 or kvLens.numel() != B or not kvLens.is_contiguous():
            raise ValueError("sdpAttention: kvLens must be a contiguous int32 tensor of B entries")
        if kvLens.device != query.device:
            raise RuntimeError("sdpAttention: kvLens must live on the device of the tensors")
        p.kv_len = kvLens.data_ptr()
    if blockTable is not None:
        p.block_table = blockTable.data_ptr()
        p.page_size = key.shape[2]
        p.block_table_stride = blockTable.stride(0)
    return p


def sdpAttention(query, key, value, isCausal=False, attnMask=None, dropoutP=0.0, scale=None, kvLens=None,
                 causalAlign="top-left", blockTable=None):
    """out = softmax(query @ key^T * scale + bias) @ value on the GPU.

    query [B,Hq,L,D]; key/value [B,Hkv,S,D] with Hq a multiple of Hkv (query head h reads KV head h // (Hq//Hkv));
    returns [B,Hq,L,D] in the dtype of query.  isCausal is top-left aligned (key j visible iff j <= i), as in the
    reference; causalAlign="bottom-right" makes the L queries the last L positions of the keys instead (key j visible
    iff j <= i + S_b - L with S_b = kvLens[b] or S): a prompt chunk or several new tokens against a KV cache.
    kvLens (not in the reference, which has no KV cache): int32 [B] on the device; batch b attends to the first
    kvLens[b] keys only, so key/value may be preallocated caches [B,Hkv,Smax,D] filled by kvCacheAppend.
    blockTable (likewise not in the reference): int32 [B, n] on the device makes key/value page pools
    [pages,Hkv,pageSize,D]; key j of batch b is row j % pageSize of page blockTable[b, j // pageSize].
    """
    if dropoutP != 0.0:
        raise NotImplementedError("sdpAttention: dropoutP must be 0 on this path")
    if query.dim() != 4 or key.dim() != 4 or value.dim() != 4:
        raise ValueError("sdpAttention: expected 4-D tensors [B, H, N, D]")
    if not query.is_cuda:
        raise RuntimeError("tinytorch_amd.sdpAttention runs on the GPU only; got a %s tensor" % query.device)
    if key.device != query.device or value.device != query.device:
        raise RuntimeError("sdpAttention: q, k, v must live on the same device")
    fix = lambda t: t if (t.stride(-1) == 1 or t.size(-1) == 1) else t.contiguous()
    query, key, value = fix(query), fix(key), fix(value)
    out = torch.empty(query.shape, dtype=query.dtype, device=query.device)
    p = build_params(query, key, value, out, isCausal, attnMask, scale, kvLens, causalAlign, blockTable)
    L = _capi.lib()
    with torch.cuda.device(query.device):
        nbytes = L.ttsdpa_workspace_bytes(ctypes.byref(p))
        ws = _workspace(query.device, nbytes) if nbytes else None
        stream = torch.cuda.current_stream().cuda_stream
        rc = L.ttsdpa_forward(ctypes.byref(p), ws.data_ptr() if ws is not None else None, nbytes, stream)
    if rc != 0:
        raise RuntimeError("ttsdpa_forward failed: %d (%s)" % (rc, _capi.status_string(rc)))
    return out


def build_backward_params(query, key, value, out, gradOut, gradQuery, gradKey, gradValue, isCausal=False, attnMask=None,
                          scale=None, kvLens=None, causalAlign="top-left"):
    """Fill a ttsdpa_backward_params: the forward call of build_params plus the four gradient tensors."""
    bp = _capi.BackwardParams()
    bp.struct_size = ctypes.sizeof(_capi.BackwardParams)
    bp.fwd = build_params(query, key, value, out, isCausal, attnMask, scale, kvLens, causalAlign)
    bp.dout, bp.dq, bp.dk, bp.dv = gradOut.data_ptr(), gradQuery.data_ptr(), gradKey.data_ptr(), gradValue.data_ptr()
    for name, t in (("dout_stride", gradOut), ("dq_stride", gradQuery), ("dk_stride", gradKey), ("dv_stride", gradValue)):
        st = _strides3(t)
        for i in range(3):
            getattr(bp, name)[i] = st[i]
    return bp


def sdpAttentionBackward(gradOut, query, key, value, out, isCausal=False, attnMask=None, scale=None, kvLens=None,
                         causalAlign="top-left"):
    """(gradQuery, gradKey, gradValue) of sdpAttention(query, key, value, ...) for the upstream gradient gradOut.

    What FuncSDPAttention::backward would compute; the reference leaves it NOT_IMPLEMENTED (reference
    src/Function/FuncNNLayer.h:267).  `out` is the forward's result for the same arguments.  gradKey / gradValue have
    the shape of key / value: with grouped heads they sum over the query heads of a KV head; rows at or beyond
    kvLens[b] are zero.
    """
    if any(t.dim() != 4 for t in (gradOut, query, key, value, out)):
        raise ValueError("sdpAttentionBackward: expected 4-D tensors [B, H, N, D]")
    if not query.is_cuda:
        raise RuntimeError("tinytorch_amd.sdpAttentionBackward runs on the GPU only; got a %s tensor" % query.device)
    if any(t.device != query.device for t in (gradOut, key, value, out)):
        raise RuntimeError("sdpAttentionBackward: all tensors must live on the same device")
    if gradOut.shape != query.shape or out.shape != query.shape:
        raise ValueError("sdpAttentionBackward: gradOut %s and out %s must have the shape of query %s"
                         % (tuple(gradOut.shape), tuple(out.shape), tuple(query.shape)))
    if gradOut.dtype != query.dtype or out.dtype != query.dtype:
        raise TypeError("sdpAttentionBackward: gradOut and out must have the dtype of query")
    fix = lambda t: t if (t.stride(-1) == 1 or t.size(-1) == 1) else t.contiguous()
    gradOut, query, key, value, out = fix(gradOut), fix(query), fix(key), fix(value), fix(out)
    gq, gk, gv = torch.empty_like(query), torch.empty_like(key), torch.empty_like(value)
    if gq.stride(-1) != 1 or gk.stride(-1) != 1 or gv.stride(-1) != 1:
        gq, gk, gv = (torch.empty(t.shape, dtype=t.dtype, device=t.device) for t in (query, key, value))
    bp = build_backward_params(query, key, value, out, gradOut, gq, gk, gv, isCausal, attnMask, scale, kvLens, causalAlign)
    L = _capi.lib()
    with torch.cuda.device(query.device):
        nbytes = L.ttsdpa_backward_workspace_bytes(ctypes.byref(bp))
        ws = _workspace(query.device, nbytes) if nbytes else None
        stream = torch.cuda.current_stream().cuda_stream
        rc = L.ttsdpa_backward(ctypes.byref(bp), ws.data_ptr() if ws is not None else None, nbytes, stream)
    if rc != 0:
        raise RuntimeError("ttsdpa_backward failed: %d (%s)" % (rc, _capi.status_string(rc)))
    return gq, gk, gv


def kvCacheAppend(kCache, vCache, kNew, vNew, positions, blockTable=None):
    """Write kNew/vNew [B,Hkv,Lnew,D] into the caches [B,Hkv,Smax,D] at rows positions[b] .. positions[b]+Lnew-1.

    positions: int32 [B] device tensor, or an int used for every batch entry.  In place, on the current stream; rows
    that would land beyond Smax are dropped.  Replaces growing K/V with op::concat on the sequence axis (reference
    src/Operation/OpTransform.cpp:306-357), which copies the whole history per generated token.
    blockTable: int32 [B, n] makes the caches page pools [pages,Hkv,pageSize,D]; row pos of batch b lands in row
    pos % pageSize of page blockTable[b, pos // pageSize], and the capacity per batch entry is n * pageSize.
    """
    if kCache.dim() != 4 or kNew.dim() != 4 or vCache.shape != kCache.shape or vNew.shape != kNew.shape:
        raise ValueError("kvCacheAppend: expected caches [B,Hkv,Smax,D] and new rows [B,Hkv,Lnew,D]")
    B, Hkv, Smax, D = kCache.shape
    if blockTable is not None:
        B = kNew.shape[0]
        _check_block_table("kvCacheAppend", blockTable, B, kCache.device)
        page = Smax
        if page < 1 or page & (page - 1):
            raise ValueError("kvCacheAppend: the page size (%d rows) must be a power of two" % page)
        Smax = blockTable.shape[1] * page
    if kNew.shape[0] != B or kNew.shape[1] != Hkv or kNew.shape[3] != D:
        raise ValueError("kvCacheAppend: new rows %s do not match the cache %s" % (tuple(kNew.shape), tuple(kCache.shape)))
    if kCache.dtype not in _DTYPES or any(t.dtype != kCache.dtype for t in (vCache, kNew, vNew)):
        raise TypeError("kvCacheAppend: dtype must be one of float32/float16/bfloat16 and equal for all four tensors")
    if not kCache.is_cuda or any(t.device != kCache.device for t in (vCache, kNew, vNew)):
        raise RuntimeError("kvCacheAppend runs on the GPU only, all tensors on one device")
    for t in (kCache, vCache, kNew, vNew):
        if t.stride(-1) != 1 and t.size(-1) != 1:
            raise ValueError("kvCacheAppend: head_dim must be contiguous")
    p = _capi.KvAppendParams()
    L = _capi.lib()
    L.ttsdpa_kv_append_params_init(ctypes.byref(p), _DTYPES[kCache.dtype], B, Hkv, Smax, kNew.shape[2], D)
    p.k_cache, p.v_cache, p.k_new, p.v_new = kCache.data_ptr(), vCache.data_ptr(), kNew.data_ptr(), vNew.data_ptr()
    for name, t in (("kc_stride", kCache), ("vc_stride", vCache), ("kn_stride", kNew), ("vn_stride", vNew)):
        for i in range(3):
            getattr(p, name)[i] = t.stride(i)
    if isinstance(positions, int):
        p.position = positions
    else:
        if positions.dtype != torch.int32 or positions.numel() != B or not positions.is_contiguous() \
                or positions.device != kCache.device:
            raise ValueError("kvCacheAppend: positions must be a contiguous int32 device tensor of B entries")
        p.positions = positions.data_ptr()
    if blockTable is not None:
        p.block_table = blockTable.data_ptr()
        p.page_size = kCache.shape[2]
        p.block_table_stride = blockTable.stride(0)
    with torch.cuda.device(kCache.device):
        rc = L.ttsdpa_kv_append(ctypes.byref(p), torch.cuda.current_stream().cuda_stream)
    if rc != 0:
        raise RuntimeError("ttsdpa_kv_append failed: %d (%s)" % (rc, _capi.status_string(rc)))


# ---- the row-wise ops next to attention (include/ttfused.h) ---------------------------------------------------------

def _check_rowwise(name, *tensors):
    t0 = tensors[0]
    if t0.dtype not in _DTYPES:
        raise TypeError("%s: dtype must be one of float32/float16/bfloat16" % name)
    if not t0.is_cuda:
        raise RuntimeError("tinytorch_amd.%s runs on the GPU only; got a %s tensor" % (name, t0.device))
    for t in tensors[1:]:
        if t is not None and (t.dtype != t0.dtype or t.device != t0.device):
            raise TypeError("%s: all tensors must share dtype and device" % name)


def _launch(name, fn, device, *args):
    with torch.cuda.device(device):
        rc = fn(*args, torch.cuda.current_stream().cuda_stream)
    if rc != 0:
        raise RuntimeError("%s failed: %d (%s)" % (name, rc, _capi.status_string(rc)))


def rmsNorm(input, normalizedShape, weight=None, eps=1e-8):
    """input / sqrt(mean(input^2) + eps) * weight over the last axis (reference src/Function/FuncNNLayer.h:294-296;
    normalizedShape must be [input.shape[-1]] as in src/Operation/OpNNLayerCpu.h:183-184)."""
    _check_rowwise("rmsNorm", input, weight)
    dim = input.shape[-1]
    if list(normalizedShape) != [dim]:
        raise ValueError("rmsNorm: normalizedShape must be [%d]" % dim)
    if weight is not None and tuple(weight.shape) != (dim,):
        raise ValueError("rmsNorm: weight must have shape [%d]" % dim)
    x = input.contiguous()
    w = weight.contiguous() if weight is not None else None
    out = torch.empty_like(x)
    rows = x.numel() // dim if dim else 0
    _launch("ttfused_rms_norm", _capi.lib().ttfused_rms_norm, x.device, _DTYPES[x.dtype], x.data_ptr(),
            w.data_ptr() if w is not None else None, out.data_ptr(), rows, dim, float(eps))
    return out


def fusedAddRmsNorm(input, residual, weight, eps):
    """In place: residual += input; input = rmsNorm(residual) * weight (reference src/Function/FuncFused.h:32-34)."""
    _check_rowwise("fusedAddRmsNorm", input, residual, weight)
    if input.shape != residual.shape or not input.is_contiguous() or not residual.is_contiguous():
        raise ValueError("fusedAddRmsNorm: input and residual must be contiguous tensors of one shape")
    dim = input.shape[-1]
    if tuple(weight.shape) != (dim,):
        raise ValueError("fusedAddRmsNorm: weight must have shape [%d]" % dim)
    w = weight.contiguous()
    rows = input.numel() // dim if dim else 0
    _launch("ttfused_add_rms_norm", _capi.lib().ttfused_add_rms_norm, input.device, _DTYPES[input.dtype],
            input.data_ptr(), residual.data_ptr(), w.data_ptr(), rows, dim, float(eps))


def siluMul(x):
    """silu(x[..., :d]) * x[..., d:] with d = x.shape[-1] / 2 (reference src/Function/FuncFused.h:30)."""
    _check_rowwise("siluMul", x)
    if x.shape[-1] % 2 != 0:
        raise ValueError("siluMul: the last axis must be even")  # reference ASSERT, src/Operation/OpFusedCpu.h:17
    x = x.contiguous()
    d = x.shape[-1] // 2
    out = torch.empty(x.shape[:-1] + (d,), dtype=x.dtype, device=x.device)
    rows = x.numel() // (2 * d) if d else 0
    _launch("ttfused_silu_mul", _capi.lib().ttfused_silu_mul, x.device, _DTYPES[x.dtype], x.data_ptr(), out.data_ptr(),
            rows, d)
    return out


def _softmax(name, x, dim, log):
    _check_rowwise(name, x)
    if x.dim() == 0:
        raise ValueError("%s: expected at least one axis" % name)
    dim = dim % x.dim()
    x = x.contiguous()
    out = torch.empty_like(x)
    outer = 1
    for n in x.shape[:dim]:
        outer *= n
    inner = 1
    for n in x.shape[dim + 1:]:
        inner *= n
    _launch("ttfused_softmax", _capi.lib().ttfused_softmax, x.device, _DTYPES[x.dtype], x.data_ptr(), out.data_ptr(),
            outer, x.shape[dim], inner, int(log))
    return out


def softmax(x, dim=-1):
    """softmax along `dim` (reference src/Function/FuncActivation.h:91)."""
    return _softmax("softmax", x, dim, False)


def logSoftmax(x, dim=-1):
    """logSoftmax along `dim` (reference src/Function/FuncActivation.h:92)."""
    return _softmax("logSoftmax", x, dim, True)


def _softmax_backward(name, grad, output, dim, log):
    _check_rowwise(name, grad, output)
    if grad.shape != output.shape or grad.dim() == 0:
        raise ValueError("%s: grad %s and output %s must have the same shape" % (name, tuple(grad.shape), tuple(output.shape)))
    dim = dim % grad.dim()
    grad, output = grad.contiguous(), output.contiguous()
    out = torch.empty_like(grad)
    outer = 1
    for n in grad.shape[:dim]:
        outer *= n
    inner = 1
    for n in grad.shape[dim + 1:]:
        inner *= n
    _launch("ttfused_softmax_backward", _capi.lib().ttfused_softmax_backward, grad.device, _DTYPES[grad.dtype],
            grad.data_ptr(), output.data_ptr(), out.data_ptr(), outer, grad.shape[dim], inner, int(log))
    return out


def softmaxBackward(grad, output, dim=-1):
    """output * (grad - sum(output * grad)) along `dim` (reference op::softmaxBackward, src/Operation/OpNNLayerCpu.h:79-109)."""
    return _softmax_backward("softmaxBackward", grad, output, dim, False)


def logSoftmaxBackward(grad, output, dim=-1):
    """grad - exp(output) * sum(grad) along `dim` (reference op::logSoftmaxBackward, src/Operation/OpNNLayerCpu.h:123-150)."""
    return _softmax_backward("logSoftmaxBackward", grad, output, dim, True)


# ---- the linear layer (include/ttlinear.h) ------------------------------------------------------------------------------

def linear(input, weight, bias=None):
    """input [..., K] . weight [N, K]^T + bias [N] (reference src/Function/FuncNNLayer.h:270-272): fp32 accumulation
    starting from the bias, one rounding to the dtype of input."""
    _check_rowwise("linear", input, weight, bias)
    if weight.dim() != 2 or input.dim() < 1 or input.shape[-1] != weight.shape[1]:
        raise ValueError("linear: input [..., K] and weight [N, K] do not match: %s, %s"
                         % (tuple(input.shape), tuple(weight.shape)))
    N, K = weight.shape
    if bias is not None and tuple(bias.shape) != (N,):
        raise ValueError("linear: bias must have shape [%d]" % N)
    M = 1
    for n in input.shape[:-1]:
        M *= n
    x = input.reshape(M, K)
    if x.stride(-1) != 1 and K > 1:
        x = x.contiguous()
    w = weight if (weight.stride(-1) == 1 or K == 1) else weight.contiguous()
    b = bias.contiguous() if bias is not None else None
    out = torch.empty(M, N, dtype=input.dtype, device=input.device)
    _launch("ttlinear_forward", _capi.lib().ttlinear_forward, x.device, _DTYPES[x.dtype], x.data_ptr(), w.data_ptr(),
            b.data_ptr() if b is not None else None, out.data_ptr(), M, N, K,
            x.stride(0) if M > 1 else max(K, 1), w.stride(0) if N > 1 else max(K, 1), N)
    return out.reshape(input.shape[:-1] + (N,))


def matmul(a, b, transA=False, transB=False, bias=None):
    """op(a) . op(b) + bias with the reference's transpose flags and batch rules (op::matmul, reference
    src/Operation/OpLinalg.cpp:52-241): a is [..., M, K], or [..., K, M] with transA; b is [..., K, N], or [..., N, K]
    with transB; leading dimensions broadcast against each other (:84-89, :205-223).  A 1-D a is a row vector, a 1-D b
    a column vector (their transpose flags are ignored, :63-72), and the added dimension is dropped from the result.
    For 2-D operands (False, True) is the linear layer; (False, False) and (True, False) are what
    FuncLinear::backward calls for the input and the weight gradient (reference src/Function/FuncNNLayer.h:20-33)."""
    _check_rowwise("matmul", a, b, bias)
    if a.dim() == 0 or b.dim() == 0:
        raise ValueError("matmul: invalid shape")  # reference :54-57
    prepend_a, append_b = a.dim() == 1, b.dim() == 1
    if prepend_a:
        a, transA = a.unsqueeze(0), False
    if append_b:
        b, transB = b.unsqueeze(-1), False
    K, M = (a.shape[-2], a.shape[-1]) if transA else (a.shape[-1], a.shape[-2])
    Kb, N = (b.shape[-1], b.shape[-2]) if transB else (b.shape[-2], b.shape[-1])
    if K != Kb:
        raise ValueError("matmul: inner sizes differ: %s (transA=%s), %s (transB=%s)" % (tuple(a.shape), transA, tuple(b.shape), transB))
    if bias is not None and tuple(bias.shape) != (N,):
        raise ValueError("matmul: bias must have shape [%d]" % N)
    try:
        batch = tuple(torch.broadcast_shapes(a.shape[:-2], b.shape[:-2]))
    except RuntimeError:
        raise ValueError("matmul: batch dimensions %s and %s do not broadcast" % (tuple(a.shape[:-2]), tuple(b.shape[:-2])))
    if len(batch) > 8:
        raise ValueError("matmul: more than 8 batch dimensions")
    dense = lambda t: t if (t.stride(-1) == 1 or t.shape[-1] == 1) and (t.shape[-2] == 1 or t.stride(-2) >= max(t.shape[-1], 1)) else t.contiguous()
    a, b = dense(a), dense(b)
    bs = bias.contiguous() if bias is not None else None
    out = torch.empty(batch + (M, N), dtype=a.dtype, device=a.device)
    L = _capi.lib()
    nbytes = L.ttlinear_matmul_workspace_bytes(_DTYPES[a.dtype], M, N, K, int(transA), int(transB))
    ws = _workspace(a.device, nbytes) if nbytes else None
    lda = a.stride(-2) if a.shape[-2] > 1 else max(a.shape[-1], 1)
    ldb = b.stride(-2) if b.shape[-2] > 1 else max(b.shape[-1], 1)
    common = (_DTYPES[a.dtype], a.data_ptr(), b.data_ptr(), bs.data_ptr() if bs is not None else None, out.data_ptr(), M, N, K,
              int(transA), int(transB), lda, ldb, N)
    tail = (ws.data_ptr() if ws is not None else None, nbytes, torch.cuda.current_stream(a.device).cuda_stream)
    with torch.cuda.device(a.device):
        if not batch:
            rc = L.ttlinear_matmul(*common, *tail)
        else:
            ea = a.expand(batch + tuple(a.shape[-2:]))  # views: broadcast axes get stride 0
            eb = b.expand(batch + tuple(b.shape[-2:]))
            nb = len(batch)
            arr = ctypes.c_int64 * nb
            sa = arr(*[ea.stride(d) if batch[d] > 1 else 0 for d in range(nb)])
            sb = arr(*[eb.stride(d) if batch[d] > 1 else 0 for d in range(nb)])
            rc = L.ttlinear_matmul_batched(*common, nb, arr(*batch), sa, sb, M * N, *tail)
    if rc != 0:
        raise RuntimeError("ttlinear_matmul failed: %d (%s)" % (rc, _capi.status_string(rc)))
    # the added dimensions are dropped as the reference drops them (:221-239): for 2-D results only — with batch
    # dimensions a 1-D a keeps its row ([..., 1, N]) and a 1-D b has no defined result there (its reshape to [M] would not fit)
    if append_b:
        if batch and out.numel() != (1 if prepend_a else M):
            raise ValueError("matmul: a 1-D second operand against a batched first operand has no result shape in the reference")
        out = out.reshape(() if prepend_a else (M,))
    elif prepend_a and not batch:
        out = out.reshape(N)
    return out


def linearBackward(gradOut, input, weight, needBias=True):
    """(gradInput, gradWeight, gradBias) of linear(input, weight, bias) — FuncLinear::backward (reference
    src/Function/FuncNNLayer.h:20-33): grad . weight, grad^T . input, and the column sums of grad."""
    N, K = weight.shape
    g = gradOut.reshape(-1, N)
    x = input.reshape(-1, K)
    gi = matmul(g, weight, False, False).reshape(input.shape)
    gw = matmul(g, x, True, False)
    gb = g.float().sum(dim=0).to(g.dtype) if needBias else None   # the reference's op::sumOnDim(grad, 0)
    return gi, gw, gb
