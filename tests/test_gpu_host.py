"""The C++ host layer (Deep8's Tensor / Device / Function / Executor API) on the GPU: runs the
driver once and reports each of its tests."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST_TESTS = os.path.join(ROOT, "deep8_amd", "host", "deep8_host_tests")


@pytest.fixture(scope="module")
def run():
    out = subprocess.run([HOST_TESTS], capture_output=True, text=True, timeout=300)
    print(out.stdout[-4000:], out.stderr[-2000:])
    return out


def _names():
    try:
        listed = subprocess.run([HOST_TESTS, "--list"], capture_output=True, text=True, timeout=60).stdout
        return [ln.split()[1] for ln in listed.splitlines() if ln.strip()]
    except OSError:
        return ["binary_missing"]


@pytest.mark.parametrize("name", _names())
def test_host_case(run, name):
    assert "PASS %s\n" % name in run.stdout, run.stdout[-3000:] + run.stderr[-1000:]


def test_host_exit_code(run):
    assert run.returncode == 0
