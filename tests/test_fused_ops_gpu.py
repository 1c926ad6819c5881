"""GPU parity of the row-wise ops next to attention (include/ttfused.h) against the CPU oracle (oracle/fused_oracle.c)
on identical seeded inputs.  Bars: fp32 max-abs-error <= 1e-4 on unit-scale values; fp16/bf16: the oracle's 16-bit form
(float arithmetic, each stored tensor rounded once) within one unit in the last place of the element type, since a
different summation order may move a result across a rounding boundary."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from gpu_util import TORCH_DTYPE, to_device, to_host_f32
from tinytorch_amd import _capi, fusedAddRmsNorm, logSoftmax, rmsNorm, siluMul, softmax

pytestmark = pytest.mark.gpu

ULP = {"f32": 0.0, "bf16": 2.0 ** -7, "f16": 2.0 ** -10}  # largest spacing of neighbours relative to the value


def say(*a):
    print(*a, flush=True)


def inputs(seed, stream, shape, dtype, mul=1.0):
    vals, bits = oracle.round_to(oracle.randn(seed, stream, shape, mul), dtype)
    return vals, to_device(vals, bits, dtype)


def close(y_dev, exp, dtype):
    y = to_host_f32(y_dev)
    assert y.shape == exp.shape and np.isfinite(y).all()
    err = np.abs(y.astype(np.float64) - exp)
    tol = 1e-4 if dtype == "f32" else 1.01 * ULP[dtype] * np.maximum(np.abs(exp), 2.0 ** -14) + 1e-7
    bad = err > tol
    assert not bad.any(), (float(err.max()), int(bad.sum()))


ROWS_DIMS = [(1, 1), (3, 7), (5, 24), (64, 128), (33, 1000), (16, 4096), (7, 5120), (4, 8192), (2, 16384), (2, 40000),
             (300, 64), (1000, 256)]


@pytest.mark.parametrize("dtype", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("rows,dim", ROWS_DIMS)
def test_rms_norm(rows, dim, dtype):
    say("rmsNorm", rows, dim, dtype)
    xh, xd = inputs(100 + dim, 0, (rows, dim), dtype, 1.5)
    wh, wd = inputs(100 + dim, 1, (dim,), dtype)
    close(rmsNorm(xd, [dim], wd, 1e-6), oracle.rms_norm(xh, wh, 1e-6, dtype), dtype)
    close(rmsNorm(xd, [dim], None, 1e-5), oracle.rms_norm(xh, None, 1e-5, dtype), dtype)


@pytest.mark.parametrize("dtype", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("rows,dim", ROWS_DIMS)
def test_fused_add_rms_norm(rows, dim, dtype):
    say("fusedAddRmsNorm", rows, dim, dtype)
    xh, xd = inputs(200 + dim, 0, (rows, dim), dtype)
    rh, rd = inputs(200 + dim, 1, (rows, dim), dtype)
    wh, wd = inputs(200 + dim, 2, (dim,), dtype)
    ea, eb = oracle.fused_add_rms_norm(xh, rh, wh, 1e-6, dtype)
    fusedAddRmsNorm(xd, rd, wd, 1e-6)
    # the residual is an exact sum rounded once: bit for bit
    assert np.array_equal(to_host_f32(rd), eb)
    close(xd, ea, dtype)


@pytest.mark.parametrize("dtype", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("rows,d", [(1, 1), (3, 5), (7, 64), (128, 1024), (33, 11008), (5, 13824), (2, 100001)])
def test_silu_mul(rows, d, dtype):
    say("siluMul", rows, d, dtype)
    xh, xd = inputs(300 + d, 0, (rows, 2 * d), dtype, 2.0)
    close(siluMul(xd), oracle.silu_mul(xh, dtype), dtype)


@pytest.mark.parametrize("dtype", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("shape,dim", [((4,), 0), ((3, 7), -1), ((3, 7), 0), ((64, 1000), 1), ((5, 32000), -1),
                                       ((2, 151936), -1), ((4, 9, 6), 1), ((2, 3, 300, 64), 2), ((8, 4096), 1),
                                       ((2, 70000), 1), ((6, 128, 33), 1),
                                       # few very long rows (1024 lanes per row): kept whole, kept in part, unaligned
                                       ((64, 128256), -1), ((3, 40000), 1), ((1, 262144), 0 + 1), ((2, 100003), -1)])
def test_softmax_and_log_softmax(shape, dim, dtype):
    say("softmax", shape, dim, dtype)
    xh, xd = inputs(400 + sum(shape), 0, shape, dtype, 3.0)
    close(softmax(xd, dim), oracle.softmax(xh, dim, False, dtype), dtype)
    yl = to_host_f32(logSoftmax(xd, dim))
    el = oracle.softmax(xh, dim, True, dtype)
    if shape[dim] > 8192:
        # The oracle adds the exponentials left to right in fp32 like the reference's CPU loop; over this many terms
        # that sum itself is off by more than the bar (2e-4 at 151936 terms), while the kernel adds pairwise.  Long
        # rows are therefore held to the fp64 closed form instead.
        x64 = xh.astype(np.float64)
        m = x64.max(dim, keepdims=True)
        el = oracle.round_to((x64 - m - np.log(np.exp(x64 - m).sum(dim, keepdims=True))).astype(np.float32), dtype)[0]
    tol = 1e-4 if dtype == "f32" else 1.01 * ULP[dtype] * np.abs(el) + 1e-4
    assert (np.abs(yl - el) <= tol).all()


@pytest.mark.parametrize("dtype", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("shape,dim", [((4,), 0), ((3, 7), -1), ((3, 7), 0), ((64, 1000), 1), ((5, 32000), -1),
                                       ((4, 9, 6), 1), ((2, 3, 300, 64), 2), ((8, 4096), 1), ((6, 128, 33), 1)])
def test_softmax_backward(shape, dim, dtype):
    """op::softmaxBackward / op::logSoftmaxBackward (reference src/Operation/OpNNLayerCpu.h:79-150) from the same rounded
    gradient and forward output the oracle sees.  The sums run over up to 32000 terms in another order than the oracle's
    left-to-right loop: the bar is the forward's, widened by the size of the terms that cancel in (g - sum)."""
    from tinytorch_amd import logSoftmaxBackward, softmaxBackward
    say("softmax backward", shape, dim, dtype)
    xh, _ = inputs(450 + sum(shape), 0, shape, dtype, 2.0)
    gh, gd = inputs(450 + sum(shape), 1, shape, dtype)
    for log, fn in ((False, softmaxBackward), (True, logSoftmaxBackward)):
        yh, yb = oracle.round_to(oracle.softmax(xh, dim, log), dtype)
        yd = to_device(yh, yb, dtype)
        exp = oracle.softmax_backward(gh, yh, dim, log, dtype)
        got = to_host_f32(fn(gd, yd, dim))
        assert got.shape == exp.shape and np.isfinite(got).all()
        n = shape[dim]
        scale = np.abs(gh).max() * (np.sqrt(n) if log else 1.0)   # |sum| the result is a difference against
        tol = (1e-4 if dtype == "f32" else 1.01 * ULP[dtype] * np.abs(exp)) + 1e-5 * max(1.0, scale)
        assert (np.abs(got.astype(np.float64) - exp) <= tol).all(), (log, float(np.abs(got - exp).max()))


def test_reference_known_answers_on_the_gpu():
    """reference test/test_function.cpp:147-152, 385-391 through the HIP kernels."""
    x = torch.tensor([[1.4176, 0.1874, 0.8367], [-0.1203, 2.5638, -1.2554]], device="cuda")
    w = torch.tensor([1.4072, -0.4768, -0.6006], device="cuda")
    y = rmsNorm(x, [3], w).cpu().numpy().ravel()
    assert np.abs(y - [2.0855, -0.0934, -0.5254, -0.1026, -0.7410, 0.4571]).max() < 1e-3
    v = torch.tensor([1.1, 1.2, 1.3, 1.6], device="cuda")
    assert np.abs(softmax(v, 0).cpu().numpy() - [0.2010, 0.2221, 0.2455, 0.3314]).max() < 1e-3
    assert np.abs(logSoftmax(v, 0).cpu().numpy() - [-1.6045, -1.5045, -1.4045, -1.1045]).max() < 1e-3


def test_in_place_and_unaligned_and_degenerate():
    L = _capi.lib()
    st = torch.cuda.current_stream().cuda_stream
    # out aliasing x (the header allows it), fp32
    xh, xd = inputs(9, 0, (17, 640), "f32")
    wh, wd = inputs(9, 1, (640,), "f32")
    exp = oracle.rms_norm(xh, wh, 1e-6)
    assert L.ttfused_rms_norm(_capi.F32, xd.data_ptr(), wd.data_ptr(), xd.data_ptr(), 17, 640, 1e-6, st) == 0
    torch.cuda.synchronize()
    close(xd, exp, "f32")
    # a view that starts 2 bytes into a buffer: rows cannot be read as 16-byte vectors
    buf = torch.zeros(8 * 256 + 1, dtype=torch.bfloat16, device="cuda")
    xh, xd = inputs(10, 0, (8, 256), "bf16")
    view = buf[1:].view(8, 256)
    view.copy_(xd)
    out = torch.empty_like(buf)
    assert L.ttfused_softmax(_capi.BF16, view.data_ptr(), out[1:].data_ptr(), 8, 256, 1, 0, st) == 0
    torch.cuda.synchronize()
    close(out[1:].view(8, 256), oracle.softmax(xh, -1, False, "bf16"), "bf16")
    # nothing to do / bad arguments: no launch
    assert L.ttfused_rms_norm(_capi.F32, None, None, None, 0, 128, 1e-6, st) == 0
    assert L.ttfused_silu_mul(_capi.F32, None, None, 5, 0, st) == 0
    assert L.ttfused_softmax(_capi.F32, None, None, 4, 4, 1, 0, st) == _capi.ERR_NULL
    assert L.ttfused_add_rms_norm(_capi.BF16, xd.data_ptr(), xd.data_ptr(), None, 8, 256, 1e-6, st) == _capi.ERR_NULL
    assert L.ttfused_rms_norm(7, xd.data_ptr(), None, xd.data_ptr(), 8, 256, 1e-6, st) == _capi.ERR_DTYPE
    assert L.ttfused_silu_mul(_capi.BF16, xd.data_ptr(), xd.data_ptr(), -1, 8, st) == _capi.ERR_SHAPE
    # an all-equal row and a row with one huge entry
    x = torch.zeros(2, 100, device="cuda")
    x[1, 37] = 1e4
    p = softmax(x, -1).cpu().numpy()
    assert np.allclose(p[0], 0.01) and p[1, 37] == 1.0 and p[1].sum() == 1.0
