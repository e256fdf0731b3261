"""Build the gfx950 shared library in-tree:  python llama.cl_amd/build.py

hipcc cross-compiles for the MI355X without a GPU present.  The output,
``llama.cl_amd/llmops/libllmops_hip.so``, is what the ``llmops`` Python module loads.
"""
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "llmops", "libllmops_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-fhip-fp32-correctly-rounded-divide-sqrt",  # quantization divides must be IEEE-exact
    "-ffp-contract=on",  # contract only within a statement; never across statements
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-attributes",
]


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")) + glob.glob(os.path.join(CSRC, "*.cpp")))


def build(verbose=False):
    cmd = [HIPCC] + FLAGS + ["-o", OUT] + sources()
    if verbose:
        print(" ".join(cmd))
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass does not know the AMDGPU feature name and says so; that line is noise
    log = "\n".join(l for l in proc.stdout.splitlines() if "is not a recognized feature for this target" not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + log)
    if verbose and log.strip():
        print(log)
    return OUT


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
