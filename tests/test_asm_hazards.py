"""The kernels' asm statements against the hazard the compiler does not guard them from (a scalar register restored by
a vector instruction and read as a memory address within five wait states): the compiler's own listing of every source
that issues memory instructions from asm statements is scanned by tinytorch_amd/csrc/check_asm_hazards.py.
Runs on the CPU (hipcc cross-compiles); about a minute."""
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "tinytorch_amd", "csrc")
SOURCES = ["sdpa_prefill_d128.hip", "sdpa_prefill_d64.hip", "sdpa_backward_mfma.hip", "linear.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


def listing(src, out):
    cmd = [HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           "-Wno-unused-command-line-argument", "-Wno-inline-asm", "-I" + CSRC, "-I" + os.path.join(ROOT, "include"),
           "--cuda-device-only", "-S", os.path.join(CSRC, src), "-o", out]
    return subprocess.run(cmd, capture_output=True, text=True)


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not installed")
def test_no_scalar_restore_hazard_before_asm_memory_instructions(tmp_path):
    outs = [str(tmp_path / (s + ".s")) for s in SOURCES]
    with ThreadPoolExecutor(max_workers=4) as pool:
        results = list(pool.map(lambda p: listing(*p), zip(SOURCES, outs)))
    for src, r in zip(SOURCES, results):
        assert r.returncode == 0, "%s did not compile:\n%s" % (src, r.stderr[-2000:])
    r = subprocess.run([sys.executable, os.path.join(CSRC, "check_asm_hazards.py")] + outs, capture_output=True, text=True)
    assert r.returncode == 0, r.stdout[-4000:]


def test_the_checker_sees_the_hazard(tmp_path):
    bad = tmp_path / "bad.s"
    bad.write_text("\tv_readlane_b32 s0, v246, 13\n\tv_readlane_b32 s1, v246, 14\n\tglobal_load_dwordx4 v[120:123], v84, s[0:1]\n")
    good = tmp_path / "good.s"
    good.write_text("\tv_readlane_b32 s1, v246, 14\n\ts_mov_b32 m0, s86\n\ts_nop 3\n\tglobal_load_lds_dwordx4 v90, s[0:1]\n")
    tool = os.path.join(CSRC, "check_asm_hazards.py")
    assert subprocess.run([sys.executable, tool, str(bad)], capture_output=True).returncode == 1
    assert subprocess.run([sys.executable, tool, str(good)], capture_output=True).returncode == 0


def test_the_checker_passes_nothing_asm_issued_that_it_cannot_classify(tmp_path):
    tool = os.path.join(CSRC, "check_asm_hazards.py")
    run = lambda name, text: (tmp_path / name).write_text(text) and subprocess.run(
        [sys.executable, tool, str(tmp_path / name)], capture_output=True, text=True)
    asm = lambda body: "\ts_add_u32 s4, s4, 1\n\t;;#ASMSTART\n%s\t;;#ASMEND\n" % body
    # a statement with its own five wait states in front of the load: proven whatever ran before it
    assert run("ok.s", ".LBB0_1:\n" + asm("\ts_mov_b32 m0, s9\n\ts_nop 3\n\tglobal_load_lds_dwordx4 v1, s[2:3]\n")).returncode == 0
    # the same load at the head of a statement behind a label: nothing is known about the path that led here
    r = run("label.s", ".LBB0_1:\n" + asm("\tglobal_load_dwordx4 v[0:3], v4, s[2:3]\n"))
    assert r.returncode == 1 and "provably" in r.stdout
    # a scalar compare result written by a vector instruction three instructions before the statement's load
    r = run("cmp.s", "\tv_cmp_lt_i32_e64 s[2:3], v0, v1\n\ts_nop 0\n" + asm("\ts_nop 0\n\tbuffer_load_dword v1, v2, s[0:3], 0 offen\n"))
    assert r.returncode == 1
    # no scalar base: nothing to prove
    assert run("off.s", ".LBB0_1:\n" + asm("\tglobal_load_dwordx4 v[0:3], v[4:5], off\n")).returncode == 0
    # scalar-memory instructions and unknown mnemonics in a statement are findings, not passes
    r = run("smem.s", asm("\ts_load_dwordx2 s[2:3], s[0:1], 0x0\n"))
    assert r.returncode == 1 and "unclassified" in r.stdout
    r = run("unknown.s", asm("\timage_load v[0:3], v4, s[0:7] dmask:0xf\n"))
    assert r.returncode == 1 and "cannot classify" in r.stdout
