"""The C++ operator header (warpdecode_amd/host/wd_ops.hpp) exercised by tests/host/test_wd_ops.cpp:
a caller in the reference's style (routed, shared, finish; resident and LRU cache) against the oracle."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "host", "test_wd_ops")


def _run(args):
    env = dict(os.environ, WD_GOLDEN_DIR=os.path.join(ROOT, "tests", "golden"))
    p = subprocess.run([EXE] + args, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300, env=env)
    assert p.returncode == 0, p.stdout
    assert " 0 failures" in p.stdout, p.stdout
    return p.stdout


def test_header_compiles_and_host_checks_pass():
    from warpdecode_amd import build
    if not os.path.exists(build.LIB):
        pytest.skip("HIP library not built")
    build.build_host_test()
    _run(["--host-only"])


@pytest.mark.gpu
def test_reference_style_caller_matches_oracle():
    assert os.path.exists(EXE), "tests/host/test_wd_ops is built by __graft_entry__.build()"
    out = _run([])
    assert int(out.split(" checks")[0].split()[-1]) > 60, out


def test_expert_prefetcher_host_checks():
    """tests/host/test_prefetch.cpp: the expert prefetcher and its planner, no GPU
    (the contract of the reference's tests/expert_prefetch_host_test.cpp)."""
    from warpdecode_amd import build
    if not os.path.exists(build.LIB):
        pytest.skip("HIP library not built")
    build.build_host_test()
    exe = os.path.join(ROOT, "tests", "host", "test_prefetch")
    p = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert p.returncode == 0 and " 0 failures" in p.stdout, p.stdout


def test_hand_off_word_never_reads_as_not_yet_written():
    """tests/host/test_handword.cpp: the helper every producer of the resident launch passes its values through - the
    bit pattern that means "not yet written" (one NaN) leaves as the default quiet NaN, every other NaN and a sweep of
    all other patterns unchanged."""
    from warpdecode_amd import build
    if not os.path.exists(build.LIB):
        pytest.skip("HIP library not built")
    build.build_host_test()
    exe = os.path.join(ROOT, "tests", "host", "test_handword")
    p = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert p.returncode == 0 and "16777214 NaN patterns" in p.stdout and " 0 failures" in p.stdout, p.stdout
