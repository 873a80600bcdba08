"""Runs the C++ host contract tests (tests/native/*.cpp): plain programs that
return a distinct non-zero code per failed check, as the reference's
tests/native do.  They need no GPU: typed errors precede any device call."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
NATIVE = os.path.join(HERE, "native")
BUILD = os.path.join(NATIVE, "build")


def _binary(name):
    path = os.path.join(BUILD, name)
    if not os.path.exists(path):
        subprocess.check_call(["make", "-C", NATIVE, os.path.join("build", name)])
    return path


@pytest.mark.parametrize("name", ["geometry_contract_test", "state_slot_contract_test",
                                  "backend_contract_test", "prefix_state_contract_test"])
def test_host_contract(name):
    result = subprocess.run([_binary(name)], capture_output=True, text=True, timeout=120)
    assert result.returncode == 0, f"{name} failed check {result.returncode}\n{result.stdout}"


@pytest.mark.gpu
def test_runtime_on_gpu():
    """Layer walk, state pool, the norm and 4-bit projection stages either side of the
    family, block prefill, state record, prefix snapshot, tape rollback and lane reset of
    the C++ host layer against the CPU checker."""
    result = subprocess.run([_binary("runtime_gpu_test")], capture_output=True, text=True,
                            timeout=300)
    print(result.stdout, flush=True)
    assert result.returncode == 0, f"runtime_gpu_test failed check {result.returncode}\n" \
                                   f"{result.stdout[-3000:]}\n{result.stderr[-2000:]}"
