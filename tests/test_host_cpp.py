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
