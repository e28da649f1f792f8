"""The C ABI without PyTorch: tests/cabi_native_check.cpp is a plain C++/HIP host program that owns its
device memory, calls libmetis_hip.so as a C caller would and compares with the C restatement of the
reference arithmetic.  It is compiled next to the library by the package Makefile; this test runs it."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cabi_native_check")

pytestmark = pytest.mark.gpu


def test_native_caller_of_the_c_abi():
    assert os.path.exists(BIN), "build first: python -c 'import __graft_entry__ as g; g.build()'"
    env = dict(os.environ)
    env["LD_LIBRARY_PATH"] = os.pathsep.join([os.path.join(ROOT, "fp4-post_amd", "metis_hip"), os.path.join(ROOT, "oracle"),
                                              env.get("LD_LIBRARY_PATH", "")])
    out = subprocess.run([BIN], capture_output=True, text=True, env=env, timeout=300)
    print(out.stdout)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "all checks passed" in out.stdout
    assert "FAIL" not in out.stdout
