"""Host-side exhaustive check of the persistent chain's work decomposition: compiles
tests/cpp/chain_math_check.cpp against the header the kernel itself uses and runs it."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.abspath(os.path.join(os.path.dirname(__file__), ".."))


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_chain_decomposition_exhaustive(tmp_path):
    exe = tmp_path / "chain_math_check"
    subprocess.run(["g++", "-O2", "-std=c++17", "-I", os.path.join(ROOT, "llama.cl_amd", "csrc"), "-o", str(exe),
                    os.path.join(ROOT, "tests", "cpp", "chain_math_check.cpp")], check=True)
    out = subprocess.run([str(exe)], check=True, stdout=subprocess.PIPE, text=True).stdout
    assert out.startswith("ok ")
