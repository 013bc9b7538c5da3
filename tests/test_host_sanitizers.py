"""Host code under AddressSanitizer + UndefinedBehaviorSanitizer (the reference's QWEN_SANITIZE builds,
cmake/qwen.cmake:21-28): `make -C tests/cpp asan` compiles the record readers, the route traces and the host shim
(records.cpp, engine.cpp), the slot cache policy (zc_store.hpp) and the CPU oracle from source with
-fsanitize=address,undefined, and the three binaries run here.  Nothing in them touches a GPU."""
import os
import subprocess
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
CPP = os.path.join(HERE, "cpp")


@pytest.fixture(scope="module")
def built():
    subprocess.run(["make", "-C", CPP, "-j4", "asan"], check=True, capture_output=True)


@pytest.mark.parametrize("name", ["test_records", "test_store_policy_host", "test_oracle_sanitized"])
def test_runs_clean_under_the_sanitizers(built, name):
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1:halt_on_error=1",
               OMP_NUM_THREADS="4")
    r = subprocess.run([os.path.join(CPP, "asan", name)], capture_output=True, text=True, timeout=600, env=env)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-6000:]
    assert "runtime error" not in r.stderr and "AddressSanitizer" not in r.stderr, r.stderr[-6000:]
