"""The generated instruction streams kept in the tree (prefill128_steps.inc, prefill64_steps.inc, linear256_loop.inc) are
what their generators write today: an edit to a generator without a regeneration would otherwise ship a stale kernel
silently.  CPU only."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "tinytorch_amd", "csrc")


@pytest.mark.parametrize("generator, args, inc", [
    ("gen_prefill128_steps.py", [], "prefill128_steps.inc"),
    ("gen_prefill128_steps.py", ["64"], "prefill64_steps.inc"),
    ("gen_linear256_loop.py", [], "linear256_loop.inc"),
])
def test_committed_stream_is_what_its_generator_writes(generator, args, inc):
    r = subprocess.run([sys.executable, os.path.join(CSRC, generator)] + args, capture_output=True, text=True, check=True)
    with open(os.path.join(CSRC, inc)) as f:
        assert f.read() == r.stdout, "%s is stale: run `python3 %s %s > %s` in %s" % (inc, generator, " ".join(args), inc, CSRC)
