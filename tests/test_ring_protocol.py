"""The tile pipeline of the ring kernels (forward, dQ, dK/dV) replayed on the host, no GPU.

`sample_efficient_gpt_amd/csrc/ring_protocol.hpp` holds the numbers the kernels compile in (which tiles are requested
when and into which LDS stage, which stages the stationary rows borrow, the `s_waitcnt vmcnt` immediates);
`tests/ring_protocol_check.cpp` generates, from those numbers, the order of requests / waits / barriers / fragment
reads one wave executes, and checks with in-order retirement that every read hits a landed, published tile and no
stage is refilled while readable.  The same program feeds itself protocols that are wrong on purpose (among them the
dQ start-up that once shipped: tile 1 requested late and not awaited before the loop, which the GPU tests only caught
in 0.8-8 % of the launches) and fails unless each is reported.
"""

import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "sample_efficient_gpt_amd", "csrc")


@pytest.fixture(scope="module")
def checker(tmp_path_factory):
    cxx = shutil.which("g++") or shutil.which("c++")
    if cxx is None:
        pytest.skip("no host C++ compiler")
    exe = str(tmp_path_factory.mktemp("ring") / "ring_protocol_check")
    subprocess.run([cxx, "-std=c++17", "-O1", "-Wall", "-Werror", f"-I{CSRC}",
                    os.path.join(ROOT, "tests", "ring_protocol_check.cpp"), "-o", exe], check=True)
    return exe


def test_shipped_protocols_hold_and_broken_ones_are_caught(checker):
    proc = subprocess.run([checker], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    out = proc.stdout
    assert proc.returncode == 0, out
    lines = out.strip().splitlines()
    ok = [l for l in lines if l.rstrip().endswith(" ok")]
    assert len(ok) == 10, out  # five pipelines (forward 2 shapes, dQ, dQ with rotary tables, dK/dV) at both head dims
    assert "VIOLATION" not in out and "NOT CAUGHT" not in out, out
    caught = [l for l in lines if "caught:" in l]
    assert len(caught) == 9, out
    # the start-up bug that once shipped must be reported as exactly what it was
    bug = next(l for l in caught if l.startswith("dQ without the wait before the loop"))
    assert "read of content 1" in bug and "before it has landed" in bug, bug


def test_kernels_compile_the_shared_numbers_in():
    """The kernels must take every pipeline number from the shared header, not from literals of their own."""
    for name, ctor in (("fwd_mfma.hip", "ring::forward("), ("bwd_mfma.hip", "ring::dq("), ("bwd_mfma.hip", "ring::dkdv(")):
        src = open(os.path.join(CSRC, name)).read()
        assert '#include "ring_protocol.hpp"' in src and ctor in src, name
        assert "ring::loads_kept_after_iteration(R, true)" in src, name
    bwd = open(os.path.join(CSRC, "bwd_mfma.hip")).read()
    assert "ring::loads_kept_before_loop(R, R.startup_tiles)" in bwd
    for src_name in ("fwd_mfma.hip", "bwd_mfma.hip"):
        src = open(os.path.join(CSRC, src_name)).read()
        # no hand-typed vmcnt immediates besides "everything"
        import re
        for m in re.finditer(r"wait_vmcnt<([^>]*)>", src):
            assert m.group(1) == "0" or m.group(1).startswith("ring::"), (src_name, m.group(0))
