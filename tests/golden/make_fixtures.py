"""Writes tests/golden/*.npz: inputs and the outputs of the *compiled reference* (oracle/_ref/libtt_ref.so, i.e.
tinytorch::function::sdpAttention on CPU, reference src/Function/FuncNNLayer.h:298-302) for small cases.

Run where /root/reference is mounted:   python tests/golden/make_fixtures.py
The fixtures are data only (inputs, expected outputs, the call's flags); they let the GPU box — which has no
reference tree — pin oracle/sdpa_oracle.c, and through it the HIP kernels, to the reference's own arithmetic.
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))

# the reference's own known-answer inputs (reference test/test_function.cpp:394-402)
KAT_Q = [0.6201, 0.5199, 0.2614, 0.9816, 0.9369, 0.8059, 0.8578, 0.7864, 0.8947, 0.4272, 0.7566, 0.2975, 0.4676,
         0.1170, 0.1046, 0.7130]
KAT_K = [0.8691, 0.8571, 0.9015, 0.3962, 0.7809, 0.0260, 0.7946, 0.6102, 0.0999, 0.9367, 0.3174, 0.1418, 0.6388,
         0.4654, 0.5967, 0.3617]
KAT_V = [0.9904, 0.8726, 0.8662, 0.3096, 0.4391, 0.9327, 0.5259, 0.6763, 0.6314, 0.8901, 0.6936, 0.2933, 0.0599,
         0.3249, 0.3593, 0.8228]


def gen(seed, B, Hq, Hkv, L, S, D, mul=1.0, dtype="f32"):
    q = oracle.randn(seed, 0, (B, Hq, L, D), mul)
    k = oracle.randn(seed, 1, (B, Hkv, S, D), mul)
    v = oracle.randn(seed, 2, (B, Hkv, S, D), mul)
    return [oracle.round_to(t, dtype)[0] for t in (q, k, v)]


def case(name, q, k, v, causal=False, scale=None, mask=None):
    if os.path.exists(os.path.join(HERE, name + ".npz")) and "--force" not in sys.argv:
        print("%-28s kept (pass --force to rewrite)" % name)
        return
    out = oracle.ref_sdpa_f32(q, k, v, causal=causal, scale=scale, mask=mask)
    extra = {}
    if mask is not None:
        extra["mask"] = mask
    if scale is not None:
        extra["scale"] = np.float32(scale)
    np.savez(os.path.join(HERE, name + ".npz"), q=q, k=k, v=v, out=out, causal=np.int32(causal), **extra)
    print("%-28s q%s k%s causal=%d -> out%s" % (name, q.shape, k.shape, causal, out.shape))


def main():
    if not oracle.have_ref():
        oracle.build(ref=True)
    kq, kk, kv = [np.array(x, np.float32).reshape(2, 2, 2, 2) for x in (KAT_Q, KAT_K, KAT_V)]
    case("kat_plain", kq, kk, kv)
    case("kat_causal", kq, kk, kv, causal=True)
    case("kat_boolmask", kq, kk, kv, mask=np.array([[0, 0], [1, 0]], np.uint8))
    case("c1_f32_causal", *gen(0x5EED0001, 1, 4, 4, 128, 128, 64), causal=True)
    case("nonsquare_l3_s5", *gen(11, 2, 3, 3, 3, 5, 16))
    case("nonsquare_l3_s5_causal", *gen(11, 2, 3, 3, 3, 5, 16), causal=True)
    case("nonsquare_l7_s4_causal", *gen(12, 1, 2, 2, 7, 4, 8), causal=True)
    case("gqa_hq8_hkv2", *gen(13, 2, 8, 2, 33, 33, 32), causal=True)
    case("decode_l1_s64", *gen(14, 3, 8, 2, 1, 64, 128))
    case("decode_l1_s300_scale", *gen(15, 2, 4, 1, 1, 300, 128), scale=0.05)
    case("bf16_inputs_causal", *gen(16, 1, 4, 2, 96, 96, 128, dtype="bf16"), causal=True)
    case("f16_inputs_causal", *gen(17, 1, 4, 4, 80, 80, 128, mul=0.5, dtype="f16"), causal=True)
    rng = np.random.RandomState(5)
    bm = (rng.rand(9, 12) > 0.4).astype(np.uint8)
    bm[:, 0] = 1  # keep every row non-empty: an empty row is NaN in the reference
    case("boolmask_l9_s12", *gen(18, 2, 2, 2, 9, 12, 64), mask=bm)
    fm = oracle.randn(19, 7, (9, 12))
    case("floatmask_l9_s12", *gen(19, 2, 2, 1, 9, 12, 64), mask=fm)
    # attnMask shapes other than [L,S]: the reference's bias add broadcasts them (reference FuncNNLayer.h:249-260)
    pad = np.ones((3, 1, 1, 20), np.uint8)  # per-batch key padding [B,1,1,S]
    pad[0, ..., 13:] = 0
    pad[1, ..., 5:] = 0
    case("boolmask_keypad_b3_s20", *gen(20, 3, 4, 2, 6, 20, 32), mask=pad)
    case("floatmask_b2_h4_l5_s9", *gen(21, 2, 4, 4, 5, 9, 16), mask=oracle.randn(21, 7, (2, 4, 5, 9)))
    hm = (np.random.RandomState(6).rand(4, 1, 11) > 0.5).astype(np.uint8)  # per-head key mask [H,1,S]
    hm[..., 0] = 1
    case("boolmask_h4_1_s11", *gen(22, 2, 4, 2, 3, 11, 16), mask=hm)
    case("floatmask_row_s10", *gen(23, 1, 2, 2, 4, 10, 8), mask=oracle.randn(23, 7, (10,)))


if __name__ == "__main__":
    main()
