"""The host-side allocator (marian-dev_amd/host/allocator.h) on a malloc-backed slab, under
AddressSanitizer and UndefinedBehaviorSanitizer: a seeded random sequence of alloc / free / grow /
clear / exhaustion / failing-device steps against a plain interval model and the behaviours of the
reference's allocator (src/tensors/allocator.h:93-115 grow re-points, :121-124 throw, :139-155
merge, :205 double free).  No GPU, no HIP."""
import os
import subprocess

import pytest

from conftest import ROOT

HOST = os.path.join(ROOT, "marian-dev_amd", "host")


@pytest.fixture(scope="module")
def exe():
    subprocess.run(["make", "-C", HOST, "-s", "allocator_check"], check=True)
    path = os.path.join(HOST, "allocator_check")
    assert os.path.exists(path)
    return path


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_allocator_against_model_under_sanitizers(exe, seed):
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    out = subprocess.run([exe, str(seed), "20000"], capture_output=True, text=True, env=env, timeout=300)
    assert out.returncode == 0, out.stdout[-2000:] + out.stderr[-4000:]
    assert "0 failure(s) -> OK" in out.stdout
    assert "ERROR: AddressSanitizer" not in out.stderr and "runtime error" not in out.stderr
