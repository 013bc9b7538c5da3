"""Runs the C++ tests of the host shim (tests/cpp/test_engine.cpp): the reference's own
operator-level tests (tests/test_qwen.cpp:277-283, 634-659, 744-754, 827-842, 1087-1099,
1188-1208, 1500-1533) restated against the shim, plus moe() against the CPU oracle."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BINARY = os.path.join(HERE, "cpp", "test_engine")


@pytest.mark.gpu
def test_engine_cpp_suite():
    assert os.path.exists(BINARY), "tests/cpp/test_engine is not built (run __graft_entry__.build())"
    done = subprocess.run([BINARY], capture_output=True, text=True, timeout=600)
    print(done.stdout[-4000:], done.stderr[-2000:])
    assert done.returncode == 0, done.stdout[-2000:] + done.stderr[-2000:]
    assert " 0 failures" in done.stdout
