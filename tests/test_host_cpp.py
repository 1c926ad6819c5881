"""The C++ host layer (tinytorch_amd/host): tinytorch::function::sdpAttention over the dispatch table and the C ABI.
The GPU part runs the compiled C++ test program, which restates the reference's own attention unit test
(reference test/test_function.cpp:393-419) with the tensors on the accelerator."""
import ctypes
import os
import subprocess

import pytest

from conftest import ROOT

LIBDIR = os.path.join(ROOT, "tinytorch_amd", "lib")
HOST_SO = os.path.join(LIBDIR, "libtinytorch_host.so")
TEST_EXE = os.path.join(LIBDIR, "test_sdpa_host")


def _need_built():
    if not (os.path.exists(HOST_SO) and os.path.exists(TEST_EXE)):
        pytest.fail("host layer not built: run `make -C tinytorch_amd/host` (or __graft_entry__.build())")


def test_host_library_loads_and_links_the_c_abi():
    _need_built()
    import torch  # noqa: F401  (one HIP runtime per process: torch's, see tinytorch_amd/_capi.py)
    lib = ctypes.CDLL(HOST_SO)
    # the registration function of the GPU slot is exported; the C ABI it calls resolves from libttsdpa.so
    assert lib._ZN9tinytorch2op20registerAttentionGpuEv is not None
    needed = subprocess.run(["readelf", "-d", HOST_SO], capture_output=True, text=True).stdout
    assert "libttsdpa.so" in needed and "libamdhip64" in needed


def test_cpp_sources_keep_the_reference_interface():
    """Names a TinyTorch caller relies on (reference src/Function/FuncNNLayer.h:229-302, src/Tensor/Dispatch.h:110-142)."""
    func = open(os.path.join(ROOT, "tinytorch_amd", "host", "FuncNNLayer.h")).read()
    assert "class FuncSDPAttention : public Function<FuncSDPAttention>" in func
    assert "inline Tensor sdpAttention(const Tensor& query, const Tensor& key, const Tensor& value, bool isCausal = false," in func
    assert "const Tensor& attnMask = {}, float dropoutP = 0.f," in func and "std::optional<float> scale = std::nullopt" in func
    assert "static void backward(AutogradContext* ctx, const Tensor& grad)" in func and "op::sdpAttentionBackward(" in func
    disp = open(os.path.join(ROOT, "tinytorch_amd", "host", "Dispatch.h")).read()
    assert "#define DEFINE_OP(NAME, FN_TYPE)" in disp and "#define REGISTER_OP_IMPL(NAME, DEVICE, DTYPE, FUNC)" in disp
    op = open(os.path.join(ROOT, "tinytorch_amd", "host", "OpAttention.cpp")).read()
    for dt in ("Float32", "Float16", "BFloat16"):
        assert "REGISTER_OP_IMPL(sdpAttention, GPU, %s" % dt in op
    assert "REGISTER_OP_IMPL(sdpAttention, CPU" not in op  # no CPU route behind this op


@pytest.mark.gpu
def test_cpp_host_program_on_gpu():
    _need_built()
    print("running", TEST_EXE, flush=True)
    r = subprocess.run([TEST_EXE], capture_output=True, text=True, timeout=100)
    print(r.stdout[-3000:], r.stderr[-2000:], flush=True)
    assert r.returncode == 0 and "ALL PASSED" in r.stdout


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
def test_host_16bit_conversions_bit_exact(dtype):
    """The host layer's own fp32 <-> 16-bit conversions (tinytorch_amd/host/Tensor.cpp; the reference's are
    src/Utils/BFloat16.h:72-85 and src/Utils/Half.h:226-257) against the oracle's rounding, which is itself held
    bit-exact to the reference's casts (test_oracle.py): specials, ties, subnormals, overflow, eight decades of
    magnitudes — every bit pattern must agree, both directions."""
    _need_built()
    import numpy as np
    import torch  # noqa: F401
    import oracle

    lib = ctypes.CDLL(HOST_SO)
    to_bits = getattr(lib, "_ZN9tinytorch19floatToBFloat16BitsEf" if dtype == "bf16" else "_ZN9tinytorch15floatToHalfBitsEf")
    to_float = getattr(lib, "_ZN9tinytorch19bfloat16BitsToFloatEt" if dtype == "bf16" else "_ZN9tinytorch15halfBitsToFloatEt")
    to_bits.argtypes, to_bits.restype = [ctypes.c_float], ctypes.c_uint16
    to_float.argtypes, to_float.restype = [ctypes.c_uint16], ctypes.c_float
    x = np.concatenate(
        [oracle.randn(3, i, (4000,)) * s for i, s in enumerate((1e-8, 1e-6, 1e-4, 1e-2, 1, 100, 7e4, 1e30))] +
        [np.array([np.inf, -np.inf, np.nan, 0, -0.0, 65504, 65519.99, 65520, 65536, 2.0**-24, 2.0**-25,
                   2.0**-25 * 1.0001, 2.0**-14, 1.0 + 2.0**-8, 1.0 + 2.0**-7 + 2.0**-8, 1.0 + 2.0**-11,
                   1.0 + 2.0**-10 + 2.0**-11, 3.3895314e38, -1.0 - 2.0**-8, 2.0**-133, 2.0**-126 * 0.75], np.float32)]
    ).astype(np.float32)
    vals, bits = oracle.round_to(x, dtype)
    got_bits = np.array([to_bits(float(v)) for v in x], dtype=np.uint16)
    nan = np.isnan(x)
    assert np.array_equal(got_bits[~nan], bits[~nan])
    # NaN: the reference's bf16 cast gives 0x7FC0 (BFloat16.h:75-77); a half NaN keeps the sign and is quiet
    assert all(np.isnan(oracle.bits_to_f32(got_bits[nan], dtype)))
    if dtype == "bf16":
        assert all(b == 0x7FC0 for b in got_bits[nan])
    # back to fp32: every one of the 65536 patterns
    every = np.arange(65536, dtype=np.uint16)
    back = np.array([to_float(int(b)) for b in every], dtype=np.float32)
    want = oracle.bits_to_f32(every, dtype)
    keep = ~np.isnan(want)
    assert np.array_equal(back[keep].view(np.uint32), want[keep].view(np.uint32)) and np.isnan(back[~keep]).all()
