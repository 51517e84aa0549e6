"""The C ABI from plain C: tests/abi_c/abi_check.c allocates with hipMalloc, calls the library on the null stream and
holds its outputs to the CPU oracle it links, with no Python or torch between the caller and the library."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "abi_c")


def test_abi_from_plain_c(oracle):
    exe = os.path.join(HERE, "abi_check")
    if not os.path.exists(exe):  # a tree where nothing is built yet
        subprocess.run(["make", "-C", HERE], check=True)
    res = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    print(res.stdout)
    assert res.returncode == 0, res.stdout + res.stderr
    assert "all checks hold" in res.stdout
    assert res.stdout.count(" ok") >= 10
