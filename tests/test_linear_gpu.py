"""GPU parity of the linear layer (include/ttlinear.h) against the CPU oracle (the reference's gemm loop with the bias
as the starting value, oracle/fused_oracle.c) on identical seeded inputs.  Bars: fp32 max-abs-error <= 1e-4 * sqrt(K)
(sums of K unit-variance products; the summation order differs), fp16/bf16 <= 2e-2 relative to the result's scale
sqrt(K) (fp32 accumulation, one rounding)."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from gpu_util import to_device, to_host_f32
from tinytorch_amd import _capi, linear

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


def inputs(seed, stream, shape, dtype, mul=1.0):
    vals, bits = oracle.round_to(oracle.randn(seed, stream, shape, mul), dtype)
    return vals, to_device(vals, bits, dtype)


def route(xd, wd, od):
    r = ctypes.c_int(-1)
    M, K = xd.shape
    rc = _capi.lib().ttlinear_plan(_capi.BF16 if xd.dtype == torch.bfloat16 else _capi.F16 if xd.dtype == torch.float16 else _capi.F32,
                                   xd.data_ptr(), wd.data_ptr(), None, od.data_ptr(), M, wd.shape[0], K,
                                   xd.stride(0), wd.stride(0), od.stride(0), ctypes.byref(r))
    assert rc == 0
    return _capi.LINEAR_ROUTE_NAMES[r.value]


CASES = [
    # M, N, K, dtype, bias, route
    (256, 256, 64, "bf16", True, "mfma"),        # one tile, one k step
    (256, 512, 256, "f16", False, "mfma"),
    (300, 260, 192, "bf16", True, "mfma"),       # ragged in M and N
    (1, 4, 64, "bf16", True, "mfma"),            # a single row
    (1100, 2300, 128, "f16", True, "mfma"),      # more than one 4 x 8 block of tiles
    (64, 768, 1024, "bf16", False, "mfma"),
    (256, 256, 32, "f32", True, "mfma"),         # fp32 on the fp32 matrix cores: one tile, one k step
    (300, 260, 160, "f32", True, "mfma"),
    (1100, 520, 96, "f32", False, "mfma"),
    (1, 4096, 512, "bf16", True, "mfma"),        # a handful of rows: the weight-streaming kernel
    (7, 200, 128, "f16", False, "mfma"),         # ... a partial block of 32 columns
    (33, 96, 192, "bf16", True, "mfma"),         # ... two row blocks, the second nearly empty
    (64, 1536, 2048, "f16", True, "mfma"),
    (5, 16384, 256, "bf16", True, "mfma"),       # ... many columns: two column blocks per workgroup
    (40, 16420, 192, "f16", False, "mfma"),      # ... with both row blocks and a partial last pair of column blocks
    (64, 20000, 128, "bf16", True, "mfma"),
    (2, 3, 5, "f32", True, "general"),
    (70, 90, 100, "f32", True, "general"),
    (129, 65, 200, "bf16", True, "general"),     # K not a multiple of 64
    (64, 66, 128, "f16", False, "general"),      # N not a multiple of 4
    (33, 40, 0, "f32", True, "general"),         # empty contraction: the bias
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "M%dN%dK%d-%s-b%d-%s" % c)
def test_linear_against_oracle(case):
    M, N, K, dtype, has_bias, want = case
    say("linear", case)
    xh, xd = inputs(600 + M + K, 0, (M, K), dtype)
    wh, wd = inputs(600 + M + K, 1, (N, K), dtype)
    bh, bd = inputs(600 + M + K, 2, (N,), dtype) if has_bias else (None, None)
    exp = oracle.linear(xh, wh, bh, dtype)
    out = linear(xd, wd, bd)
    assert route(xd, wd, out) == want
    y = to_host_f32(out)
    assert y.shape == exp.shape and np.isfinite(y).all()
    scale = max(1.0, np.sqrt(K))
    tol = 1e-4 * scale if dtype == "f32" else 2e-2 * scale
    err = float(np.abs(y.astype(np.float64) - exp).max()) if y.size else 0.0
    say("   max-abs-err", err, "tol", tol)
    assert err <= tol


def test_reference_known_answer_and_views():
    """reference test/test_function.cpp:234-241 through the GPU; leading batch axes; strided views of x, w and out."""
    x = torch.tensor([[-0.3089, 0.5301, -0.0245], [1.5852, 0.8954, 0.7485]], device="cuda")
    w = torch.tensor([[0.8397, 1.7990, -0.2738], [-0.8910, -0.6746, 0.3419]], device="cuda")
    b = torch.tensor([-0.9601, -1.4163], device="cuda")
    assert abs(float(linear(x, w, b).sum()) - (-3.1661377)) < 1e-5
    xh, xd = inputs(1, 0, (2, 5, 70, 128), "bf16")
    wh, wd = inputs(1, 1, (96, 128), "bf16")
    exp = oracle.linear(xh.reshape(-1, 128), wh, None, "bf16").reshape(2, 5, 70, 96)
    assert np.abs(to_host_f32(linear(xd, wd)) - exp).max() <= 2e-2 * np.sqrt(128)
    # rows taken out of wider buffers (leading dimensions larger than K / N), through the C ABI
    xbuf = torch.zeros(300, 192 + 64, dtype=torch.bfloat16, device="cuda")
    wbuf = torch.zeros(260, 192 + 8, dtype=torch.bfloat16, device="cuda")
    obuf = torch.full((300, 260 + 12), -3.0, dtype=torch.bfloat16, device="cuda")
    xh, xd = inputs(2, 0, (300, 192), "bf16")
    wh, wd = inputs(2, 1, (260, 192), "bf16")
    xbuf[:, :192], wbuf[:, :192] = xd, wd
    rc = _capi.lib().ttlinear_forward(_capi.BF16, xbuf.data_ptr(), wbuf.data_ptr(), None, obuf.data_ptr(), 300, 260, 192,
                                      xbuf.stride(0), wbuf.stride(0), obuf.stride(0), torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert rc == 0
    assert np.abs(to_host_f32(obuf[:, :260]) - oracle.linear(xh, wh, None, "bf16")).max() <= 2e-2 * np.sqrt(192)
    assert bool((obuf[:, 260:] == -3.0).all())   # nothing written beyond N


def test_full_size_projection_properties():
    """The QKV projection of config 3's token batch (8192 tokens, hidden 4096 -> 6144): sampled outputs against fp64
    dot products, linearity in x, and the bias entering exactly once."""
    M, N, K = 8192, 6144, 4096
    gen = torch.Generator(device="cuda").manual_seed(3)
    x = torch.randn(M, K, device="cuda", generator=gen).bfloat16()
    w = (torch.randn(N, K, device="cuda", generator=gen) * K ** -0.5).bfloat16()
    b = torch.randn(N, device="cuda", generator=gen).bfloat16()
    y = linear(x, w, b)
    rows = torch.randint(0, M, (64,), device="cuda", generator=gen)
    cols = torch.randint(0, N, (64,), device="cuda", generator=gen)
    exact = (x[rows].double() * w[cols].double()).sum(-1) + b[cols].double()
    assert float((y[rows, cols].double() - exact).abs().max()) <= 2e-2
    y0 = linear(x, w)
    assert float((y.float() - y0.float() - b.float()[None, :]).abs().max()) <= 3e-2   # two roundings apart
    y2 = linear(x * 2, w)   # doubling x is exact in bf16
    assert torch.equal(y2.float(), y0.float() * 2)
    # the same projection in fp32 (full fp32 products): 1e-4 * sqrt(K) against fp64 on the sampled outputs
    xf, wf, bf = x.float(), w.float(), b.float()
    yf = linear(xf, wf, bf)
    assert float((yf[rows, cols].double() - exact).abs().max()) <= 1e-4 * np.sqrt(K)


MATMUL_CASES = [
    # M, N, K, transA, transB, dtype, bias
    (512, 384, 256, False, False, "bf16", False),   # input gradient of a linear layer: dy [M, N'] . w [N', K']
    (384, 256, 512, True, False, "bf16", False),    # weight gradient: dy^T . x
    (300, 260, 192, False, False, "f16", True),
    (260, 192, 320, True, False, "f16", False),
    (256, 128, 64, True, True, "bf16", True),
    (300, 260, 160, False, False, "f32", True),     # fp32 on the fp32 matrix cores after the copies
    (260, 96, 320, True, False, "f32", False),
    (70, 90, 100, False, False, "f32", True),       # shapes the MFMA kernel does not take: read in place
    (33, 47, 65, True, False, "bf16", True),
    (5, 3, 2, True, True, "f32", False),
    (64, 64, 64, False, True, "bf16", True),        # the linear layer's own form
    (296, 264, 192, False, False, "bf16", True),    # contraction-major b read in place, ragged 128-tiles
    (264, 200, 320, True, False, "f16", True),      # both operands contraction-major, ragged
    (136, 72, 64, True, True, "bf16", False),       # contraction-major a, row-major b
    (4088, 4088, 128, True, False, "bf16", False),  # 256 ragged 256 x 256 tiles, both operands contraction-major
    (4088, 4088, 64, False, False, "f16", True),    # the same tiles, row-major a
]


@pytest.mark.parametrize("case", MATMUL_CASES, ids=lambda c: "M%dN%dK%d-tA%d-tB%d-%s-b%d" % c)
def test_matmul_transpose_flags_against_oracle(case):
    from tinytorch_amd import matmul
    M, N, K, ta, tb, dtype, has_bias = case
    say("matmul", case)
    ah, ad = inputs(700 + M + K, 0, (K, M) if ta else (M, K), dtype)
    bh, bd = inputs(700 + M + K, 1, (N, K) if tb else (K, N), dtype)
    ch, cd = inputs(700 + M + K, 2, (N,), dtype) if has_bias else (None, None)
    exp = oracle.matmul(ah, bh, ta, tb, ch, dtype)
    y = to_host_f32(matmul(ad, bd, ta, tb, cd))
    assert y.shape == exp.shape and np.isfinite(y).all()
    scale = max(1.0, np.sqrt(K))
    tol = 1e-4 * scale if dtype == "f32" else 2e-2 * scale
    err = float(np.abs(y.astype(np.float64) - exp).max())
    say("   max-abs-err", err, "tol", tol)
    assert err <= tol
    # without scratch the operands are read in place on the vector ALUs: the same result to the same bar
    L = _capi.lib()
    out = torch.empty(M, N, dtype=ad.dtype, device="cuda")
    code = {"f32": _capi.F32, "f16": _capi.F16, "bf16": _capi.BF16}[dtype]
    rc = L.ttlinear_matmul(code, ad.data_ptr(), bd.data_ptr(), cd.data_ptr() if cd is not None else None, out.data_ptr(),
                           M, N, K, int(ta), int(tb), ad.stride(0), bd.stride(0), N, None, 0, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert rc == 0
    assert float(np.abs(to_host_f32(out).astype(np.float64) - exp).max()) <= tol


def test_matmul_in_place_operands_with_leading_dimensions():
    """Operands that are views of larger buffers (leading dimension beyond the row): the matrix-core kernel that reads
    contraction-major operands in place takes their strides; against torch's fp32 product of the same values."""
    L = _capi.lib()
    st = torch.cuda.current_stream().cuda_stream
    g = torch.Generator(device="cuda").manual_seed(7)
    M, N, K = 392, 328, 256
    for ta, tb in ((True, False), (False, False), (True, True)):
        abuf = torch.randn((K, M + 40) if ta else (M, K + 24), device="cuda", generator=g).bfloat16()
        bbuf = torch.randn((N, K + 8) if tb else (K, N + 16), device="cuda", generator=g).bfloat16()
        a = abuf[:, 8:8 + M] if ta else abuf[:, 16:16 + K]
        b = bbuf[:, :K] if tb else bbuf[:, 8:8 + N]
        obuf = torch.zeros(M, N + 12, device="cuda", dtype=torch.bfloat16)
        out = obuf[:, 4:4 + N]
        rc = L.ttlinear_matmul(_capi.BF16, a.data_ptr(), b.data_ptr(), None, out.data_ptr(), M, N, K, int(ta), int(tb),
                               a.stride(0), b.stride(0), out.stride(0), None, 0, st)
        torch.cuda.synchronize()
        assert rc == 0
        ref = (a.float().t() if ta else a.float()) @ (b.float().t() if tb else b.float())
        err = float((out.float() - ref).abs().max())
        say("in-place operands transA=%d transB=%d: max-abs-err %.3e" % (ta, tb, err))
        assert err <= 2e-2 * np.sqrt(K)
        assert float(obuf[:, :4].abs().max()) == 0 and float(obuf[:, 4 + N:].abs().max()) == 0   # nothing beyond the view


def test_linear_backward_against_torch_autograd():
    """FuncLinear::backward (reference src/Function/FuncNNLayer.h:20-33) at a projection's shape: grad . w, grad^T . x and
    the column sums of grad, against torch's fp32 autograd on the same bf16 values."""
    from tinytorch_amd import linearBackward
    M, N, K = 2048, 1536, 1024
    gen = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn(M, K, device="cuda", generator=gen).bfloat16()
    w = (torch.randn(N, K, device="cuda", generator=gen) * K ** -0.5).bfloat16()
    g = torch.randn(M, N, device="cuda", generator=gen).bfloat16()
    xf, wf = x.float().requires_grad_(), w.float().requires_grad_()
    bf = torch.zeros(N, device="cuda", requires_grad=True)
    torch.nn.functional.linear(xf, wf, bf).backward(g.float())
    gi, gw, gb = linearBackward(g, x, w)
    for got, exp, k in ((gi, xf.grad, N), (gw, wf.grad, M), (gb, bf.grad, M)):
        err = (got.float() - exp).abs().max().item()
        assert err <= 2e-2 * max(1.0, k ** 0.5), err


def test_matmul_batch_rules_reference_vectors():
    """op::matmul with batch dimensions, broadcasting and 1-D operands: the reference's own vectors
    (reference test/test_operation.cpp:1223-1396) through the Python mirror, exact in fp32."""
    import tinytorch_amd

    ar = lambda *shape: torch.arange(int(np.prod(shape)), dtype=torch.float32, device="cuda").reshape(shape)
    t = lambda v: torch.tensor(v, dtype=torch.float32, device="cuda")

    def check(y, shape, vals):
        assert tuple(y.shape) == tuple(shape), (tuple(y.shape), shape)
        assert np.array_equal(y.cpu().numpy().ravel(), np.array(vals, np.float32))

    mm = tinytorch_amd.matmul
    check(mm(t([[1, 0], [0, 1]]), t([1, 2])), (2,), [1, 2])
    check(mm(t([1, 2]), t([[1, 0], [0, 1]])), (2,), [1, 2])
    check(mm(t([2]), t([2])), (), [4])
    check(mm(ar(2, 2, 4), ar(1, 2, 4, 2)), (1, 2, 2, 2), [28, 34, 76, 98, 428, 466, 604, 658])
    check(mm(ar(2, 2, 4), ar(1, 4, 2)), (2, 2, 2), [28, 34, 76, 98, 124, 162, 172, 226])
    check(mm(ar(2, 3, 4), ar(2, 4, 2)), (2, 3, 2), [28, 34, 76, 98, 124, 162, 604, 658, 780, 850, 956, 1042])
    check(mm(ar(2, 3, 4), ar(4, 2)), (2, 3, 2), [28, 34, 76, 98, 124, 162, 172, 226, 220, 290, 268, 354])
    check(mm(ar(3, 4), ar(2, 4, 2)), (2, 3, 2), [28, 34, 76, 98, 124, 162, 76, 82, 252, 274, 428, 466])
    check(mm(ar(1, 3, 4), ar(2, 4, 2)), (2, 3, 2), [28, 34, 76, 98, 124, 162, 76, 82, 252, 274, 428, 466])
    check(mm(ar(2, 3, 4), ar(2, 2, 4), False, True), (2, 3, 2), [14, 38, 38, 126, 62, 214, 518, 734, 670, 950, 822, 1166])
    check(mm(ar(2, 4, 3), ar(2, 4, 2), True, False), (2, 3, 2), [84, 102, 96, 118, 108, 134, 756, 822, 800, 870, 844, 918])
    check(mm(ar(2, 1, 3, 4), ar(2, 1, 4, 2)), (2, 1, 3, 2), [28, 34, 76, 98, 124, 162, 604, 658, 780, 850, 956, 1042])
    check(mm(ar(1, 2, 3), ar(6, 3, 2)), (6, 2, 2), [10, 13, 28, 40, 28, 31, 100, 112, 46, 49, 172, 184, 64, 67, 244, 256, 82, 85,
                                                  316, 328, 100, 103, 388, 400])
    check(mm(ar(8, 2, 3), ar(1, 3, 2)), (8, 2, 2), [10, 13, 28, 40, 46, 67, 64, 94, 82, 121, 100, 148, 118, 175, 136, 202, 154, 229,
                                                  172, 256, 190, 283, 208, 310, 226, 337, 244, 364, 262, 391, 280, 418])


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("case", [
    # a shape, b shape, transA, transB, bias
    ((3, 40, 72), (3, 72, 24), False, False, False),
    ((2, 3, 130, 128), (2, 3, 200, 128), False, True, False),      # q . k^T of an attention call: the MFMA kernel per entry
    ((2, 1, 64, 130), (1, 4, 64, 40), True, False, True),         # both operands broadcast, transposed first operand
    ((5, 33, 128), (128, 48), False, False, True),                 # a batch against one matrix
    ((2, 2, 1, 256, 256), (2, 1, 3, 256, 256), False, True, False),  # two broadcast axes, tile-sized entries
    ((16, 8, 64, 32), (16, 8, 48, 32), False, True, True),         # 128 small entries: one grid on the vector-ALU kernel
    ((4, 8, 96, 160), (4, 8, 160, 64), False, False, False),       # probabilities x values: one grid, operands read in place
    ((6, 1, 70, 64), (6, 5, 36, 64), False, True, False),           # a shared by five entries each: no uniform stride, entry by entry
])
def test_matmul_batched_against_oracle(dtype, case):
    import tinytorch_amd

    sa, sb, ta, tb, with_bias = case
    N = sb[-2] if tb else sb[-1]
    K = sa[-2] if ta else sa[-1]
    a_h, a_bits = oracle.round_to(oracle.randn(61, 0, sa, K ** -0.5), dtype)
    b_h, b_bits = oracle.round_to(oracle.randn(61, 1, sb), dtype)
    bias_h, bias_bits = oracle.round_to(oracle.randn(61, 2, (N,)), dtype)
    a, b, bias = to_device(a_h, a_bits, dtype), to_device(b_h, b_bits, dtype), to_device(bias_h, bias_bits, dtype)
    y = tinytorch_amd.matmul(a, b, ta, tb, bias if with_bias else None)
    exp = oracle.matmul_nd(a_h, b_h, ta, tb, bias_h if with_bias else None)
    assert tuple(y.shape) == exp.shape
    tol = (1e-4 if dtype == "f32" else 2e-2) * max(1.0, float(np.sqrt(K)) / 4)
    err = float(np.abs(y.float().cpu().numpy() - exp).max())
    print("matmul batched %s %s x %s: max-abs-err %.3e" % (dtype, sa, sb, err), flush=True)
    assert err <= tol
