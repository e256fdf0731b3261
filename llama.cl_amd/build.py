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


# Kernels that must compile without VGPR spills: the one-row group-128 decode kernels are written to fit
# the 64 registers that two 16-wave workgroups per CU leave each wave, and scratch traffic in their loop
# costs what the rewrite gained; the prompt attention kernel likewise (a reload in its loop waits for the
# next tile's loads).
NO_SPILL = ["fc_gemv_fused_kernelILi128ELi1E", "attn_prefill_kernel"]
# Kernels that may park a few registers around rarely-run code but whose main loop must be free of spill
# code: the 256-row GEMM reads LDS there with hand-placed ds_read / s_waitcnt pairs (a register spilled
# between the two would be saved before its data has arrived).  Checked in the device assembly: no scratch
# instruction between the kernel's first and last instruction of the kind that marks the loop.
NO_SPILL_IN_LOOP = {"fc_gemm_pp_kernelILb0E": "v_mfma_i32_16x16x64_i8"}


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


def check_loop_spills(asm_path):
    """asm_path: the device assembly of one source (kept by -save-temps); returns the kernels it has checked"""
    with open(asm_path) as fh:
        lines = fh.read().splitlines()
    seen = []
    for key, marker in NO_SPILL_IN_LOOP.items():
        # a function starts at a line "<mangled name>:" in column 0
        starts = [i for i, l in enumerate(lines) if l[:1] not in (" ", "\t", ".", ";", "") and key in l.split(":")[0] and ":" in l]
        for a in starts:
            seen.append(key)
            b = next((j for j in range(a, len(lines)) if lines[j].startswith(".Lfunc_end")), len(lines))
            marks = [j for j in range(a, b) if marker in lines[j]]
            if not marks:
                raise RuntimeError(f"{key}: no {marker} found in {asm_path}; the loop check cannot tell where the loop is")
            bad = [j for j in range(marks[0], marks[-1] + 1) if "scratch_" in lines[j]]
            if bad:
                raise RuntimeError(f"{key} has spill code inside its main loop ({lines[bad[0]].strip()}); see NO_SPILL_IN_LOOP")
    return seen


def _compile(src, obj):
    cmd = [HIPCC] + [f for f in FLAGS if f != "-shared"] + ["-Rpass-analysis=kernel-resource-usage", "-save-temps=obj", "-c", "-o", obj, src]
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
        checked = []
        for asm in glob.glob(os.path.join(objdir, "*-hip-amdgcn-amd-amdhsa-gfx950.s")):
            checked += check_loop_spills(asm)
        missing = sorted(set(NO_SPILL_IN_LOOP) - set(checked))
        if missing:
            raise RuntimeError(f"kernels named in NO_SPILL_IN_LOOP were not found in the device assembly: {missing}")
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
