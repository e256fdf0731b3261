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
    "-Wall", "-Wno-unused-function", "-Wno-unknown-attributes", "-Wno-inline-asm",
]


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")) + glob.glob(os.path.join(CSRC, "*.cpp")))


# Kernels that must compile without VGPR spills: the 256-row GEMM reads LDS with hand-placed ds_read /
# s_waitcnt pairs (a register spilled between the two would be saved before its data has arrived); the
# one-row group-128 decode kernels are written to fit the 64 registers that two 16-wave workgroups per
# CU leave each wave, and scratch traffic in their loop costs what the rewrite gained.
NO_SPILL = ["fc_gemm_pp_kernelILb0E", "fc_gemv_fused_kernelILi128ELi1E"]


def check_spills(remarks):
    """remarks: the -Rpass-analysis=kernel-resource-usage lines of the compile"""
    name = None
    for line in remarks:
        if "Function Name:" in line:
            name = line.split("Function Name:")[1].split()[0]
        elif "VGPRs Spill:" in line and name is not None:
            spilled = int(line.split("VGPRs Spill:")[1].split()[0])
            if spilled and any(k in name for k in NO_SPILL):
                raise RuntimeError(f"{name} spills {spilled} VGPRs; this kernel must not spill (see NO_SPILL)")


def build(verbose=False):
    cmd = [HIPCC] + FLAGS + ["-Rpass-analysis=kernel-resource-usage", "-o", OUT] + sources()
    if verbose:
        print(" ".join(cmd))
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    lines = proc.stdout.splitlines()
    remarks = [l for l in lines if "[-Rpass-analysis=kernel-resource-usage]" in l]
    # the host pass does not know the AMDGPU feature name and says so; that line is noise, and so are
    # the resource remarks and the source lines the compiler quotes under each of them
    keep, skip = [], 0
    for l in lines:
        if "[-Rpass-analysis=kernel-resource-usage]" in l:
            skip = 2 if "Function Name:" in l else 0
            continue
        if skip:
            skip -= 1
            continue
        if "is not a recognized feature for this target" not in l:
            keep.append(l)
    log = "\n".join(keep)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + log)
    check_spills(remarks)
    if verbose and log.strip():
        print(log)
    return OUT


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
