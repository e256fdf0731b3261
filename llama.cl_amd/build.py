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
    # the first 14 dwords of a kernel's arguments arrive in scalar registers with the wave instead of being
    # fetched by its first instructions: the short decode kernels take what their first loads need there
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-attributes", "-Wno-inline-asm",
]


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")) + glob.glob(os.path.join(CSRC, "*.cpp")))


# Kernels that must compile without VGPR spills: the 256-row GEMM reads LDS with hand-placed ds_read /
# s_waitcnt pairs (a register spilled between the two would be saved before its data has arrived); the
# one-row group-128 decode kernels are written to fit the 64 registers that two 16-wave workgroups per
# CU leave each wave, and scratch traffic in their loop costs what the rewrite gained.
NO_SPILL = ["fc_gemm_pp_kernelILb0E", "fc_gemv_fused_kernelILi128ELi1E", "attn_prefill_kernel"]


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


def _compile(src, obj):
    cmd = [HIPCC] + [f for f in FLAGS if f != "-shared"] + ["-Rpass-analysis=kernel-resource-usage", "-c", "-o", obj, src]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    return src, proc.returncode, proc.stdout.splitlines()


def _readable(lines):
    """the host pass does not know the AMDGPU feature name and says so; that line is noise, and so are
    the resource remarks and the source lines the compiler quotes under each of them"""
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
    return "\n".join(keep)


def build(verbose=False, jobs=None):
    """Compiles every source to an object of its own (in parallel) and links the shared library.  Always
    recompiles everything: the objects live in a scratch directory that is emptied first."""
    import concurrent.futures
    import shutil
    import tempfile

    objdir = tempfile.mkdtemp(prefix="llmops_build_")
    try:
        srcs = sources()
        jobs = jobs or min(len(srcs), max(1, (os.cpu_count() or 2) - 1), 16)
        objs = [os.path.join(objdir, os.path.basename(s) + ".o") for s in srcs]
        with concurrent.futures.ThreadPoolExecutor(jobs) as ex:
            results = list(ex.map(lambda so: _compile(*so), zip(srcs, objs)))
        remarks, logs = [], []
        for src, rc, lines in results:
            remarks += [l for l in lines if "[-Rpass-analysis=kernel-resource-usage]" in l]
            log = _readable(lines)
            if rc != 0:
                raise RuntimeError(f"hipcc failed on {src}:\n" + log)
            if log.strip():
                logs.append(log)
        check_spills(remarks)
        link = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", OUT] + objs
        proc = subprocess.run(link, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if proc.returncode != 0:
            raise RuntimeError("link failed:\n" + proc.stdout)
        if verbose and logs:
            print("\n".join(logs))
    finally:
        shutil.rmtree(objdir, ignore_errors=True)
    return OUT


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
