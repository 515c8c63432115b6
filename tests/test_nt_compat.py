"""The C++ facade (neurotensor_amd/nt_compat): the reference's own test cases replayed through
`tests/cpp/nt_compat_tests` (built by neurotensor_amd/nt_compat/Makefile)."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "nt_compat_tests")
GOLDEN = os.path.join(ROOT, "tests", "golden")


def _run(*extra):
    assert os.path.exists(BIN), f"{BIN} is not built (run __graft_entry__.build())"
    r = subprocess.run([BIN, GOLDEN, *extra], capture_output=True, text=True, timeout=300)
    print(r.stdout[-4000:])
    print(r.stderr[-2000:])
    return r


def test_facade_rejects_bad_arguments_before_any_device_work():
    """Shape / dtype / mutability / contiguity violations throw like the reference's
    utils::throw_exception does; none of these cases may need a GPU."""
    r = _run("--host-only")
    assert r.returncode == 0
    assert "0 failed" in r.stdout and "[FAIL]" not in r.stdout


@pytest.mark.gpu
def test_facade_replays_reference_tests_on_gpu():
    r = _run()
    assert r.returncode == 0, r.stdout[-3000:]
    assert "0 failed" in r.stdout and "[FAIL]" not in r.stdout
    assert r.stdout.count("[ok]") >= 100
