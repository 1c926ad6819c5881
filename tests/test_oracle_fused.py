"""Pins oracle/fused_oracle.c (rmsNorm, fusedAddRmsNorm, siluMul, softmax / logSoftmax) before anything is checked
against it: the reference's own known answers (reference test/test_function.cpp:139-176, 385-391), the compiled
reference when oracle/_ref is present (bit for bit in fp32), fp64 closed forms, and identities a wrong index, a
dropped term or a swapped half would break."""
import numpy as np
import pytest


def rng(seed):
    return np.random.default_rng(seed)


def test_reference_known_answers(oracle_mod):
    o = oracle_mod
    # func_rmsNorm, reference test/test_function.cpp:385-391 (default eps 1e-8, src/Function/FuncNNLayer.h:294)
    x = np.array([[1.4176, 0.1874, 0.8367], [-0.1203, 2.5638, -1.2554]], np.float32)
    w = np.array([1.4072, -0.4768, -0.6006], np.float32)
    assert np.abs(o.rms_norm(x, w, 1e-8).ravel() - [2.0855, -0.0934, -0.5254, -0.1026, -0.7410, 0.4571]).max() < 1e-3
    # func_softmax / func_logSoftmax, reference test/test_function.cpp:147-176
    v = np.array([1.1, 1.2, 1.3, 1.6], np.float32)
    assert np.abs(o.softmax(v, 0) - [0.2010, 0.2221, 0.2455, 0.3314]).max() < 1e-3
    assert np.abs(o.softmax(v, 0, log=True) - [-1.6045, -1.5045, -1.4045, -1.1045]).max() < 1e-3
    m = np.array([[1, 2], [3, 4]], np.float32)
    assert np.abs(o.softmax(m, 0, log=True).ravel() - [-2.1269, -2.1269, -0.1269, -0.1269]).max() < 1e-3
    assert np.abs(o.softmax(m, 1, log=True).ravel() - [-1.3133, -0.3133, -1.3133, -0.3133]).max() < 1e-3
    # func_silu, reference test/test_function.cpp:139-143: siluMul with up == 1 is silu
    g = np.array([-1.0, -0.5, 0.5, 1.0], np.float32)
    assert np.abs(o.silu_mul(np.concatenate([g, np.ones(4, np.float32)])[None, :]).ravel()
                  - [-0.2689, -0.1888, 0.3112, 0.7311]).max() < 1e-3


@pytest.mark.parametrize("rows,dim", [(1, 1), (3, 7), (5, 128), (2, 4096), (4, 1000)])
def test_against_compiled_reference_bitwise(oracle_mod, rows, dim):
    o = oracle_mod
    if not o.have_ref():
        pytest.skip("oracle/_ref not built")
    r = rng(rows * 1000 + dim)
    x = r.standard_normal((rows, dim)).astype(np.float32) * 2
    res = r.standard_normal((rows, dim)).astype(np.float32)
    w = r.standard_normal(dim).astype(np.float32)
    assert np.array_equal(o.rms_norm(x, w, 1e-6), o.ref_rms_norm(x, w, 1e-6))
    assert np.array_equal(o.rms_norm(x, None, 1e-5), o.ref_rms_norm(x, None, 1e-5))
    a, b = o.fused_add_rms_norm(x, res, w, 1e-6)
    ra, rb = o.ref_fused_add_rms_norm(x, res, w, 1e-6)
    assert np.array_equal(a, ra) and np.array_equal(b, rb)
    if dim % 2 == 0:
        assert np.array_equal(o.silu_mul(x), o.ref_silu_mul(x))
    for log in (False, True):
        assert np.array_equal(o.softmax(x, -1, log), o.ref_softmax(x, -1, log))
        assert np.array_equal(o.softmax(x, 0, log), o.ref_softmax(x, 0, log))
    x3 = r.standard_normal((3, max(dim // 4, 1), 5)).astype(np.float32)
    assert np.array_equal(o.softmax(x3, 1), o.ref_softmax(x3, 1))


def test_closed_forms_and_identities(oracle_mod):
    o = oracle_mod
    r = rng(7)
    x = r.standard_normal((6, 320)).astype(np.float32) * 3
    res = r.standard_normal((6, 320)).astype(np.float32)
    w = r.standard_normal(320).astype(np.float32)
    x64, w64 = x.astype(np.float64), w.astype(np.float64)
    ref = x64 / np.sqrt((x64 ** 2).mean(-1, keepdims=True) + 1e-6) * w64
    assert np.abs(o.rms_norm(x, w, 1e-6) - ref).max() < 1e-5
    # scale invariance (eps = 0): rmsNorm(c x) == rmsNorm(x); unit mean square of the unweighted result
    assert np.abs(o.rms_norm(4 * x, w, 0.0) - o.rms_norm(x, w, 0.0)).max() < 1e-5
    assert np.abs((o.rms_norm(x, None, 0.0).astype(np.float64) ** 2).mean(-1) - 1).max() < 1e-5
    # fusedAddRmsNorm(x, r, w) == rmsNorm(x + r, w), and its residual output is x + r
    a, b = o.fused_add_rms_norm(x, res, w, 1e-6)
    assert np.array_equal(b, x + res)
    assert np.abs(a - o.rms_norm(x + res, w, 1e-6)).max() < 1e-5
    # siluMul: gate is the FIRST half, up the second; against the fp64 closed form
    g, u = x[:, :160].astype(np.float64), x[:, 160:].astype(np.float64)
    assert np.abs(o.silu_mul(x) - g / (1 + np.exp(-g)) * u).max() < 1e-5
    assert np.abs(o.silu_mul(x) - o.silu_mul(np.concatenate([x[:, 160:], x[:, :160]], -1))).max() > 0.1
    # softmax: rows sum to one, shift invariance, log form is the log, an axis in the middle equals a transposed last axis
    p = o.softmax(x, -1)
    assert np.abs(p.sum(-1) - 1).max() < 1e-5 and (p >= 0).all()
    assert np.abs(o.softmax(x + 5, -1) - p).max() < 1e-6
    assert np.abs(np.exp(o.softmax(x, -1, log=True)) - p).max() < 1e-6
    x3 = r.standard_normal((4, 9, 6)).astype(np.float32)
    assert np.array_equal(o.softmax(x3, 1), np.swapaxes(o.softmax(np.swapaxes(x3, 1, 2).copy(), -1), 1, 2))
    e = np.exp(x3.astype(np.float64) - x3.max(1, keepdims=True))
    assert np.abs(o.softmax(x3, 1) - e / e.sum(1, keepdims=True)).max() < 1e-6


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
def test_16bit_results_are_representable_and_close(oracle_mod, dtype):
    """16-bit form: float arithmetic on the rounded inputs, every stored tensor rounded once (the reference's device
    kernels, src/Operation/OpFusedCuda.cuh:104-127, OpNNLayerCuda.cuh:253-299)."""
    o = oracle_mod
    r = rng(3)
    x, _ = o.round_to(r.standard_normal((4, 256)).astype(np.float32), dtype)
    res, _ = o.round_to(r.standard_normal((4, 256)).astype(np.float32), dtype)
    w, _ = o.round_to(r.standard_normal(256).astype(np.float32), dtype)
    outs = [o.rms_norm(x, w, 1e-6, dtype), *o.fused_add_rms_norm(x, res, w, 1e-6, dtype), o.silu_mul(x, dtype),
            o.softmax(x, -1, False, dtype)]
    fp32 = [o.rms_norm(x, w, 1e-6), *o.fused_add_rms_norm(x, res, w, 1e-6), o.silu_mul(x), o.softmax(x, -1)]
    ulp = 2.0 ** -8 if dtype == "bf16" else 2.0 ** -11
    for y, y32 in zip(outs, fp32):
        assert np.array_equal(o.round_to(y, dtype)[0], y)              # representable
        assert (np.abs(y - y32) <= 2 * ulp * np.abs(y32) + 1e-7).all()  # one or two roundings away from fp32
    # the normalised row is computed from the ROUNDED residual (what the reference stores and re-reads)
    a, b = o.fused_add_rms_norm(x, res, w, 1e-6, dtype)
    assert np.array_equal(b, o.round_to(x + res, dtype)[0])


def test_linear_known_answer_reference_and_closed_form(oracle_mod):
    o = oracle_mod
    # func_linear, reference test/test_function.cpp:234-241: the sum of linear(x, w, b)
    x = np.array([[-0.3089, 0.5301, -0.0245], [1.5852, 0.8954, 0.7485]], np.float32)
    w = np.array([[0.8397, 1.7990, -0.2738], [-0.8910, -0.6746, 0.3419]], np.float32)
    b = np.array([-0.9601, -1.4163], np.float32)
    assert abs(float(o.linear(x, w, b).sum()) - (-3.1661377)) < 1e-5
    r = rng(21)
    for M, N, K in ((1, 1, 1), (5, 7, 3), (8, 16, 16), (33, 65, 129), (64, 128, 256)):
        x = r.standard_normal((M, K)).astype(np.float32)
        w = r.standard_normal((N, K)).astype(np.float32)
        b = r.standard_normal(N).astype(np.float32)
        y = o.linear(x, w, b)
        ref64 = x.astype(np.float64) @ w.astype(np.float64).T + b
        assert np.abs(y - ref64).max() < 1e-4 * max(1.0, np.sqrt(K))
        assert np.abs(o.linear(x, w) - (ref64 - b)).max() < 1e-4 * max(1.0, np.sqrt(K))
        # w is [N, K] (not [K, N]): transposing the operand must change the answer for a non-symmetric case
        if N == K and N > 1:
            assert np.abs(o.linear(x, w) - o.linear(x, w.T.copy())).max() > 0.1
        if o.have_ref():
            assert np.array_equal(y, o.ref_linear(x, w, b))
            assert np.array_equal(o.linear(x, w), o.ref_linear(x, w))
    # 16-bit: one rounding of the fp32 result
    xb, _ = o.round_to(x, "bf16")
    wb, _ = o.round_to(w, "bf16")
    y16 = o.linear(xb, wb, None, "bf16")
    assert np.array_equal(y16, o.round_to(o.linear(xb, wb), "bf16")[0])


def test_matmul_transpose_flags_reference_and_closed_form(oracle_mod):
    """oracle_matmul with every transpose flag pair: bit-exact against the compiled reference's op::matmul (with and without
    bias), the fp64 closed form, (False, True) == oracle_linear, and a wrong flag must change the answer."""
    o = oracle_mod
    r = rng(31)
    for M, N, K in ((1, 1, 1), (5, 7, 3), (16, 16, 16), (33, 65, 129)):
        for ta in (False, True):
            for tb in (False, True):
                a = r.standard_normal((K, M) if ta else (M, K)).astype(np.float32)
                b = r.standard_normal((N, K) if tb else (K, N)).astype(np.float32)
                bias = r.standard_normal(N).astype(np.float32)
                y = o.matmul(a, b, ta, tb, bias)
                A = a.T if ta else a
                Bm = b.T if tb else b
                ref64 = A.astype(np.float64) @ Bm.astype(np.float64) + bias
                assert np.abs(y - ref64).max() < 1e-4 * max(1.0, np.sqrt(K)), (M, N, K, ta, tb)
                assert np.abs(o.matmul(a, b, ta, tb) - (ref64 - bias)).max() < 1e-4 * max(1.0, np.sqrt(K))
                if o.have_ref():
                    assert np.array_equal(y, o.ref_matmul(a, b, ta, tb, bias)), (M, N, K, ta, tb)
                    assert np.array_equal(o.matmul(a, b, ta, tb), o.ref_matmul(a, b, ta, tb))
                if not ta and tb:
                    assert np.array_equal(y, o.linear(a, b, bias))
                if M == N == K and K > 1:   # square: the flags are not interchangeable
                    assert np.abs(y - o.matmul(a, b, not ta, tb, bias)).max() > 0.1
                    assert np.abs(y - o.matmul(a, b, ta, not tb, bias)).max() > 0.1
    a16, _ = o.round_to(r.standard_normal((8, 12)).astype(np.float32), "bf16")
    b16, _ = o.round_to(r.standard_normal((8, 20)).astype(np.float32), "bf16")
    y16 = o.matmul(a16, b16, True, False, None, "bf16")
    assert np.array_equal(y16, o.round_to(o.matmul(a16, b16, True, False), "bf16")[0])


def test_softmax_backward_reference_and_differences(oracle_mod):
    """oracle_softmax_backward: bit-exact against the compiled reference's op::softmaxBackward / op::logSoftmaxBackward on
    every axis; central differences of a float64 forward; the softmax gradient sums to 0 along the axis."""
    o = oracle_mod
    r = rng(41)
    for shape, dim in (((5, 7), 1), ((4, 6, 3), 1), ((3, 4, 5), 0), ((2, 3, 4, 5), 2), ((6, 33), -1)):
        x = r.standard_normal(shape).astype(np.float32)
        g = r.standard_normal(shape).astype(np.float32)
        for log in (False, True):
            y = o.softmax(x, dim, log)
            d = o.softmax_backward(g, y, dim, log)
            if o.have_ref():
                assert np.array_equal(d, o.ref_softmax_backward(g, y, dim, log)), (shape, dim, log)
            # d/dx of sum(f(x) * g) by central differences in float64
            def f(z):
                z = z - z.max(axis=dim, keepdims=True)
                e = np.exp(z)
                s = e.sum(axis=dim, keepdims=True)
                return z - np.log(s) if log else e / s
            x64 = x.astype(np.float64)
            num = np.zeros_like(x64)
            flat = x64.reshape(-1)
            for i in range(flat.size):
                old = flat[i]
                flat[i] = old + 1e-5
                up = (f(x64) * g).sum()
                flat[i] = old - 1e-5
                dn = (f(x64) * g).sum()
                flat[i] = old
                num.reshape(-1)[i] = (up - dn) / 2e-5
            assert np.abs(num - d).max() < 2e-5 * max(1.0, np.abs(num).max()), (shape, dim, log)
            if not log:
                assert np.abs(d.sum(axis=dim)).max() < 1e-5
    g16, _ = o.round_to(g, "bf16")
    y16, _ = o.round_to(o.softmax(x, -1), "bf16")
    d16 = o.softmax_backward(g16, y16, -1, False, "bf16")
    assert np.array_equal(d16, o.round_to(o.softmax_backward(g16, y16, -1), "bf16")[0])


def test_matmul_nd_against_the_references_vectors(oracle_mod):
    """The batch / broadcast / 1-D rules of op::matmul, pinned by the reference's own known answers
    (test/test_operation.cpp:1223-1396): the entries of a batch are the 2-D products the tests above hold bit-exact
    against the compiled reference; these vectors fix which slices meet and what shape comes out."""
    ar = lambda *shape: np.arange(int(np.prod(shape)), dtype=np.float32).reshape(shape)
    oracle = oracle_mod
    mm = oracle.matmul_nd
    eq = lambda got, shape, vals: got.shape == tuple(shape) and np.array_equal(got.ravel(), np.array(vals, np.float32))
    # :1223-1262
    assert eq(mm(np.array([[1, 2], [3, 4]], np.float32), np.array([[2, 3], [4, 5]], np.float32)), (2, 2), [10, 13, 22, 29])
    assert eq(mm(np.eye(2, dtype=np.float32), np.array([1, 2], np.float32)), (2,), [1, 2])
    assert eq(mm(np.array([1, 2], np.float32), np.eye(2, dtype=np.float32)), (2,), [1, 2])
    assert eq(mm(np.array([2], np.float32), np.array([2], np.float32)), (), [4])
    assert eq(mm(ar(2, 2, 4), ar(1, 2, 4, 2)), (1, 2, 2, 2), [28, 34, 76, 98, 428, 466, 604, 658])
    assert eq(mm(ar(2, 2, 4), ar(1, 4, 2)), (2, 2, 2), [28, 34, 76, 98, 124, 162, 172, 226])
    # :1264-1277 (transposed second operand)
    assert eq(mm(np.array([[1, 2], [3, 4]], np.float32), np.array([[2, 3], [4, 5]], np.float32), False, True), (2, 2), [8, 14, 18, 32])
    # :1279-1372
    assert eq(mm(ar(2, 3, 4), ar(2, 4, 2)), (2, 3, 2), [28, 34, 76, 98, 124, 162, 604, 658, 780, 850, 956, 1042])
    assert eq(mm(ar(2, 3, 4), ar(4, 2)), (2, 3, 2), [28, 34, 76, 98, 124, 162, 172, 226, 220, 290, 268, 354])
    assert eq(mm(ar(3, 4), ar(2, 4, 2)), (2, 3, 2), [28, 34, 76, 98, 124, 162, 76, 82, 252, 274, 428, 466])
    assert eq(mm(ar(1, 3, 4), ar(2, 4, 2)), (2, 3, 2), [28, 34, 76, 98, 124, 162, 76, 82, 252, 274, 428, 466])
    assert eq(mm(ar(2, 3, 4), ar(1, 4, 2)), (2, 3, 2), [28, 34, 76, 98, 124, 162, 172, 226, 220, 290, 268, 354])
    assert eq(mm(ar(2, 3, 4), ar(2, 2, 4), False, True), (2, 3, 2), [14, 38, 38, 126, 62, 214, 518, 734, 670, 950, 822, 1166])
    assert eq(mm(ar(2, 4, 3), ar(2, 4, 2), True, False), (2, 3, 2), [84, 102, 96, 118, 108, 134, 756, 822, 800, 870, 844, 918])
    assert eq(mm(ar(2, 1, 3, 4), ar(2, 1, 4, 2)), (2, 1, 3, 2), [28, 34, 76, 98, 124, 162, 604, 658, 780, 850, 956, 1042])
    # :1374-1396 (more than four batch entries)
    assert eq(mm(ar(1, 2, 3), ar(6, 3, 2)), (6, 2, 2), [10, 13, 28, 40, 28, 31, 100, 112, 46, 49, 172, 184, 64, 67, 244, 256, 82,
                                                      85, 316, 328, 100, 103, 388, 400])
    assert eq(mm(ar(8, 2, 3), ar(1, 3, 2)), (8, 2, 2), [10, 13, 28, 40, 46, 67, 64, 94, 82, 121, 100, 148, 118, 175, 136, 202, 154,
                                                      229, 172, 256, 190, 283, 208, 310, 226, 337, 244, 364, 262, 391, 280, 418])
    # against numpy's own broadcasting product on a shape none of the vectors has
    a, b = oracle.randn(5, 0, (2, 1, 3, 7, 5)), oracle.randn(5, 1, (4, 1, 5, 6))
    assert np.allclose(mm(a, b), np.matmul(a.astype(np.float64), b.astype(np.float64)), atol=1e-5)
