"""Runs the C++ tests of the on-disk expert record readers (tests/cpp/test_records.cpp): the prepared
"zc-affine-records-v1" directory and the safetensors checkpoint layout, with the refusals of the reference's
PreparedArtifact / ExpertStore (src/engine/storage.cpp:316-394, 493-516).  No GPU needed."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
BINARY = os.path.join(HERE, "cpp", "test_records")


def test_records_cpp_suite():
    if not os.path.exists(BINARY):
        subprocess.run(["make", "-C", os.path.join(HERE, "cpp"), "test_records"], check=True, capture_output=True)
    done = subprocess.run([BINARY], capture_output=True, text=True, timeout=300)
    print(done.stdout[-4000:], done.stderr[-2000:])
    assert done.returncode == 0, done.stdout[-2000:] + done.stderr[-2000:]
    assert " 0 failures" in done.stdout
