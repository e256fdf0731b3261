#!/usr/bin/env python3
"""Benchmark of the Q4_1 decode FC path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Workload (BASELINE.json configs[1]): the Llama-7B-shape decode FC set, Q4_1 group 128, M=1 --
per layer q/k/v/o 4096->4096, gate/up 4096->11008, down 11008->4096 -- over 32 layers of DISTINCT
packed weights (3.45 GB, far beyond the 256 MB Infinity Cache), one activation row.  One "step" is
one pass over all 224 FCs through the C ABI (`llmops_fc_Q4A`), replayed as a HIP graph.  Inputs and
weights are resident in HBM before the timed region.

Prints one JSON line: whole-job GB/s over the algorithmic bytes (packed weights + fp32 x + fp32 y),
the roofline record of the dominant kernel (`fc_gemv_fused_kernel`), and the CPU baseline (the
reference's own AVX kernels from oracle/_ref when present, else this repo's C restatement) timed
on this machine's host cores over a bounded sample of the same workload.
"""
import argparse
import json
import os
import sys
import time

# the plain read / copy kernels behind `read_ceiling`, `read_only_chain` and `--calib` are test hooks of the library
os.environ.setdefault("LLMOPS_TEST_HOOKS", "1")

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "llama.cl_amd"))

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth
# HBM bytes per launch of the dominant kernel over the fused plan, from hardware counters: FETCH_SIZE and WRITE_SIZE
# of two `rocprofv3 --pmc` runs of this file, each scaled by what the same counter reads for the plain 1 GiB copy
# of `--calib` (one FETCH_SIZE count = 2.000 KiB, one WRITE_SIZE count = 1.000 KiB on this part); the summary with
# the per-shape figures is profiles/fc_gemv_fused_kernel__hbm_traffic_pmc.md.  Counters cannot be read from inside
# this process, so the figure is the recorded one and only holds for the fused plan at group 128, M=1.
MEASURED_TRAFFIC_BYTES_PER_LAUNCH = 27191835
MEASURED_TRAFFIC_PROFILE = "profiles/fc_gemv_fused_kernel__hbm_traffic_pmc.md"
# Counter summaries under profiles/ and the kernel sources each was taken from: sha256 (first 16 hex digits) of the
# sources when the counters were read.  The bench line says for each whether the sources have changed since, i.e.
# whether the recorded figures are stale.
PROFILE_SOURCES = {
    "profiles/fc_gemv_fused_kernel__hbm_traffic_pmc.md": (("fc_gemv.hip", "gemv_device.h"), "13290cb794320013"),
    "profiles/fc_gemv_fused_kernel__vector_alu_pmc.md": (("fc_gemv.hip", "gemv_device.h"), "13290cb794320013"),
    "profiles/fc_gemm_kernels__prefill_g128_pmc.md": (("fc_gemm.hip", "fc_rows.hip", "q8_act.hip"), "e8ede7feb8d88665"),
    "profiles/attn_prefill_kernel__prompt_2048_pmc.md": (("attn.hip",), "08562b1e2698a706"),
}
MEASURED_TRAFFIC_KERNEL_SHA16 = PROFILE_SOURCES[MEASURED_TRAFFIC_PROFILE][1]
G = 128
LAYERS = 32
# (name, N, K) of one layer's FCs, in the order the model calls them (chatllama/main.py:344-375)
LAYER_FCS = [("q", 4096, 4096), ("k", 4096, 4096), ("v", 4096, 4096), ("o", 4096, 4096),
             ("gate", 11008, 4096), ("up", 11008, 4096), ("down", 4096, 11008)]


def kernel_source_sha16(files=("fc_gemv.hip", "gemv_device.h")):
    import hashlib
    h = hashlib.sha256()
    for f in files:
        with open(os.path.join(ROOT, "llama.cl_amd", "csrc", f), "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:16]


def profiles_staleness():
    """for every counter summary under profiles/: have the kernel sources it was taken from changed since?"""
    return {prof: {"sources": list(files), "sha16_when_measured": sha, "sha16_now": kernel_source_sha16(files),
                   "stale": kernel_source_sha16(files) != sha} for prof, (files, sha) in PROFILE_SOURCES.items()}


def host_cpu_model():
    try:
        with open("/proc/cpuinfo") as fh:
            for line in fh:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def blk_bytes(g):
    return (g // 8) * 128 + 128


def fc_bytes(N, K, M=1, g=G):
    """Algorithmic bytes of one FC: packed weights (reference format, fp16 d/m) + fp32 x + fp32 y."""
    return -(-N // 32) * -(-K // g) * blk_bytes(g) + 4 * M * K + 4 * M * N


# launch plan of the decode step: packed tensors of FCs that share their input are concatenated
# along N (the packed format is [strip][k-block][bytes], so this is a plain torch.cat), which
# turns q|k|v and gate|up into one launch each: same bytes, same outputs, fewer launches
FUSED_PLAN = [("qkv", ("q", "k", "v")), ("o", ("o",)), ("gate_up", ("gate", "up")), ("down", ("down",))]
UNFUSED_PLAN = [(n, (n,)) for n, _, _ in LAYER_FCS]
SHAPE = {n: (N, K) for n, N, K in LAYER_FCS}


def main():
    import faulthandler
    faulthandler.enable()  # a crash inside a native library still names the Python line it happened under
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-decode", action="store_true", help="skip the full decode-step timing (BASELINE config 5)")
    ap.add_argument("--no-extra", action="store_true", help="skip the prefill GEMM (config 3) and attention (config 4) legs")
    ap.add_argument("--concurrent", action="store_true",
                    help="refused: the leg that dealt the FC set to 2-4 streams inside one graph is switched off (replaying "
                         "such a multi-branch graph ended twice in a host-side segmentation fault under hipGraphLaunch and "
                         "no cause has been shown)")
    ap.add_argument("--no-concurrent", action="store_true", help="accepted and ignored (that leg no longer exists)")
    ap.add_argument("--calib", action="store_true",
                    help="only run the plain copy/read kernels over 1 GiB (reference points for traffic counters and "
                         "for the attainable HBM rate) and print their rates")
    args = ap.parse_args()
    if args.calib:
        return calib()
    if args.concurrent:
        print("bench.py: --concurrent is switched off. The leg replayed one HIP graph with 2-4 branches (the FC set dealt "
              "to side streams); twice in about twenty runs that replay ended in a host-side segmentation fault under "
              "hipGraphLaunch (the fault handler named graph.replay() of that leg). During a replay no code of this "
              "repository runs on the host, no cause has been shown, and the case must not be run again before one is. "
              "The product captures single-branch graphs only.", file=sys.stderr)
        sys.exit(2)
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (the path is data-parallel per GPU; nothing here uses a second "
              "one). Re-run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch
    import llmops

    assert torch.cuda.is_available(), "bench.py needs the MI355X"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    gen = torch.Generator(device="cpu").manual_seed(2)

    # ---- synthetic weights: quantize+pack once per FC on the device, then make every layer distinct ----
    t0 = time.time()
    packed = {}
    for name, N, K in LAYER_FCS:
        w = (torch.randn(N, K, generator=gen) * 0.02).to(dev)
        packed[name] = llmops.offline_FC_quant_Q4A(w, G)
        del w

    def layer_weights(plan, layer):
        out = []
        for _, parts in plan:
            t = torch.cat([packed[p] for p in parts], dim=0) if len(parts) > 1 else packed[parts[0]]
            # rolling the strips makes each layer's bytes distinct without re-quantizing 32 times
            out.append(torch.roll(t, shifts=layer + 1, dims=0).contiguous())
        return out

    xs = {K: torch.randn(1, 1, K, generator=gen).to(dev) for K in (4096, 11008)}
    step_bytes = LAYERS * sum(fc_bytes(N, K) for _, N, K in LAYER_FCS)
    stream = torch.cuda.Stream()
    results = {}
    with torch.cuda.stream(stream):
        for label, plan in (("fused", FUSED_PLAN), ("unfused", UNFUSED_PLAN)):
            weights = [layer_weights(plan, layer) for layer in range(LAYERS)]
            dims = [(sum(SHAPE[p][0] for p in parts), SHAPE[parts[0]][1]) for _, parts in plan]
            torch.cuda.synchronize()

            def run_step():
                for layer in range(LAYERS):
                    for (N, K), wq in zip(dims, weights[layer]):
                        llmops.fc_Q4A(xs[K], wq, N)

            run_step()  # loads code objects, sizes the workspace
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                run_step()
            for _ in range(args.warmup):
                graph.replay()
            torch.cuda.synchronize()
            # wall clock for `value`, HIP events on the launch stream for the kernel's average duration
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            t1 = time.perf_counter()
            e0.record(stream)
            for _ in range(args.steps):
                graph.replay()
            e1.record(stream)
            torch.cuda.synchronize()
            dt = time.perf_counter() - t1
            results[label] = {"ms_per_step": dt / args.steps * 1e3, "event_ms_per_step": e0.elapsed_time(e1) / args.steps,
                              "launches": LAYERS * len(plan)}
            if label == "fused":
                per_shape = measure_shapes(torch, llmops, plan, dims, weights, xs, stream)
            del weights, graph
        floor_us = dispatch_floor(torch, stream)
        read_chain = read_only_chain(torch, llmops, stream,
                                     [(sum(SHAPE[p][0] for p in parts), SHAPE[parts[0]][1]) for _, parts in FUSED_PLAN])
    ceiling_gbs = read_ceiling(torch, llmops)
    setup_s = time.time() - t0

    main_r = results["fused"]
    value = step_bytes / (main_r["ms_per_step"] * 1e-3) / 1e9
    avg_us = main_r["event_ms_per_step"] * 1e3 / main_r["launches"]
    achieved = step_bytes / (main_r["event_ms_per_step"] * 1e-3) / 1e9
    roof = {"bound": "hbm", "kernel": "fc_gemv_fused_kernel<128,1,16,0>", "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": MEASURED_TRAFFIC_BYTES_PER_LAUNCH,
            "traffic_source": {"how": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by a 1 GiB copy kernel (recorded run)",
                               "profile": MEASURED_TRAFFIC_PROFILE, "kernel_sources_sha16_when_measured": MEASURED_TRAFFIC_KERNEL_SHA16,
                               "kernel_sources_sha16_now": kernel_source_sha16(),
                               "stale": kernel_source_sha16() != MEASURED_TRAFFIC_KERNEL_SHA16},
            "avg_launch_us": round(avg_us, 3), "launches_per_step": main_r["launches"],
            "bytes_per_launch_avg": int(step_bytes / main_r["launches"]), "per_shape": per_shape,
            "dispatch_floor_us": round(floor_us, 3), "read_only_chain": read_chain,
            "read_ceiling": {"GB/s": round(ceiling_gbs, 1), "frac_of_it": round(achieved / ceiling_gbs, 4),
                             "what": "plain read kernel (16-byte non-temporal loads, contiguous slab per workgroup) over "
                                     "2 GiB, one launch: what this part's HBM delivers to a kernel that does nothing else"},
            "timing": "HIP events on the launch stream around the timed graph replays; every node of the graph is this "
                      "kernel, so the average includes the dispatch gap between dependent launches (dispatch_floor_us)"}
    out = {
        "metric": "Q4_1 FC decode GB/s (% HBM peak); ms/token Llama-7B shape @ kv-len 2048",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(main_r["ms_per_step"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8 x int4 -> int32 dot, fp32 scales and accumulation",
        "data": "synthetic",
        "config": {"workload": "Llama-7B-shape decode FC set, Q4_1 group 128, M=1: 32 layers x (q,k,v,o 4096x4096; gate,up "
                               "11008x4096; down 4096x11008), distinct weights per layer, x~N(0,1), W~N(0,0.02)",
                   "bytes_per_step": step_bytes, "launch": "hip-graph replay of llmops.fc_Q4A calls",
                   "launches_per_layer": len(FUSED_PLAN),
                   "plan": "q|k|v and gate|up packed tensors concatenated along N (one launch each), o and down separate"},
        "pct_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
        "unfused_7_launches_per_layer": {"GB/s": round(step_bytes / (results["unfused"]["ms_per_step"] * 1e-3) / 1e9, 2),
                                         "ms_per_step": round(results["unfused"]["ms_per_step"], 4)},
        "roofline": roof,
        "profiles": profiles_staleness(),
    }
    if not args.no_decode:
        out["decode_step"] = decode_step(torch, stream)
    if not args.no_extra:
        out["decode_fc_g32"] = decode_fc_g32(torch, llmops, stream)
        out["prefill_gemm"] = prefill_gemm(torch, llmops, stream)
        out["decode_attention"] = decode_attention(torch, llmops, stream)
        out["prefill_attention"] = prefill_attention(torch, llmops, stream)
    if not args.no_cpu:
        # the reference's allocator announces itself on stdout (ops/tensor.hpp:88-91); keep stdout for the JSON line
        sys.stdout.flush()
        saved = os.dup(1)
        os.dup2(2, 1)
        try:
            out["cpu_baseline"] = cpu_baseline()
        finally:
            sys.stdout.flush()
            os.dup2(saved, 1)
            os.close(saved)
    out["setup_s"] = round(setup_s, 1)
    print(json.dumps(out))


def measure_shapes(torch, llmops, plan, dims, weights, xs, stream, reps=10):
    """Per-shape average launch duration: one graph per shape over the 32 distinct weight sets."""
    per_shape = {}
    for i, ((name, _), (N, K)) in enumerate(zip(plan, dims)):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=stream):
            for layer in range(LAYERS):
                llmops.fc_Q4A(xs[K], weights[layer][i], N)
        g.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(reps):
            g.replay()
        e1.record(stream)
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / (reps * LAYERS)
        b = fc_bytes(N, K)
        per_shape[f"{name} {N}x{K}"] = {"us": round(us, 3), "GB/s": round(b / us / 1e3, 1), "bytes": b}
        del g
    return per_shape


def dispatch_floor(torch, stream, n=64, reps=10):
    """Average time per launch of a do-nothing kernel in a replayed graph: the gap between dependent launches."""
    t = torch.zeros(64, device="cuda")
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=stream):
        for _ in range(n):
            t.add_(1.0)
    g.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    for _ in range(reps):
        g.replay()
    e1.record(stream)
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / (n * reps)


def read_only_chain(torch, llmops, stream, dims, layers=32, reps=10):
    """The plain read kernel (non-temporal 16-byte loads, a slab per workgroup) in the launch structure of `value`:
    a graph of dependent launches over `layers` distinct buffers of each FC tensor's size.  What a kernel that only
    reads reaches in this chain; the FC kernel's quantization, products, reduction and stores come on top."""
    import ctypes
    lib = llmops._lib.load()
    out4 = torch.zeros(4, dtype=torch.int32, device="cuda")
    sizes = [fc_bytes(N, K) // 16 * 16 for (N, K) in dims]
    stride = (max(sizes) + 4095) // 4096 * 4096
    pool = torch.zeros(layers * stride, dtype=torch.uint8, device="cuda")
    st = ctypes.c_void_p(stream.cuda_stream)
    per_shape, total = {}, 0.0
    for (N, K), nbytes in zip(dims, sizes):
        best = None
        for wgs in (512, 1024, 2048):
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=stream):
                for l in range(layers):
                    llmops._lib.check(lib.llmops_test_calib_read(pool.data_ptr() + l * stride, nbytes, wgs, out4.data_ptr(), st))
            for _ in range(3):
                g.replay()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for _ in range(reps):
                g.replay()
            e1.record(stream)
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / (reps * layers)
            best = us if best is None else min(best, us)
            del g
        per_shape[f"{N}x{K}"] = round(best, 3)
        total += best
    layer_bytes = sum(fc_bytes(N, K) for (N, K) in dims)
    return {"us_per_layer": round(total, 2), "GB/s": round(layer_bytes / total / 1e3, 1), "us_per_shape": per_shape,
            "what": "plain read kernel over buffers of the FC tensors' sizes, same graph of dependent launches (best of "
                    "512/1024/2048 workgroups per size)"}


def decode_step(torch, stream, kv_len=2048, reps=50, warm=10):
    """BASELINE config 5: one token through a random-init Llama-2-7B-shape model (32 layers, hidden 4096, FFN 11008,
    32 heads, vocab 55296 lm_head, all FC Q4_1 group 128), fp32 KV cache filled to kv_len-1, batch 1; the step is
    captured once as a HIP graph and replayed."""
    from llmops.decode import LlamaDecoder, LLAMA_7B
    from llmops.opset import KVCache

    out = {}
    model = LlamaDecoder(group_k=G, seed=5, embed_rows=1024)
    for name, dtype in (("fp32_kv", torch.float32), ("fp16_kv", torch.float16)):
        kv = KVCache(LLAMA_7B, 1, kv_len, dtype=dtype)
        kv.cache.normal_()
        dg = model.capture_decode(kv.cache, kv_len - 1, kv_len - 1, stream=stream)
        with torch.cuda.stream(stream):
            for _ in range(warm):  # the first replays of a fresh graph run 3-4 % slower than the steady state
                dg.replay()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(reps):
                dg.replay()
            torch.cuda.synchronize()
            ms = (time.perf_counter() - t0) / reps * 1e3
        # the same step launched op by op (no graph): what a caller that cannot capture graphs gets
        with torch.cuda.stream(stream):
            ids = torch.zeros(1, 1, dtype=torch.int64, device="cuda")
            slots = torch.tensor([kv_len - 1], dtype=torch.int32, device="cuda")
            model.forward(ids, kv.cache, slots, kv_len - 1)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(5):
                model.forward(ids, kv.cache, slots, kv_len - 1)
            torch.cuda.synchronize()
            eager_ms = (time.perf_counter() - t0) / 5 * 1e3
        if name == "fp32_kv":
            # the prompt pass of the same model: kv_len tokens at position 0 through all layers and the lm_head
            # (rows > 8: rmsnorm / silu*up inside the quantization launches, MFMA GEMMs, tiled attention), op by op
            with torch.cuda.stream(stream):
                pids = torch.zeros(1, kv_len, dtype=torch.int64, device="cuda")
                pslots = torch.arange(kv_len, dtype=torch.int32, device="cuda")
                model.forward(pids, kv.cache, pslots, 0)
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(3):
                    model.forward(pids, kv.cache, pslots, 0)
                torch.cuda.synchronize()
                pms = (time.perf_counter() - t0) / 3 * 1e3
            out["prefill_step"] = {"tokens": kv_len, "ms": round(pms, 3), "tokens_per_s": round(kv_len / pms * 1e3, 0),
                                   "what": "prompt of kv_len tokens, batch 1, fp32 KV cache, logits for every token"}
            del pids, pslots
            kv.cache.normal_()
        kv_bytes = 2 * LLAMA_7B["layer_num"] * LLAMA_7B["head_num"] * kv_len * LLAMA_7B["head_size"] * kv.cache.element_size()
        fc = model.fc_weight_size()
        out[name] = {"ms_per_token": round(ms, 4), "ms_per_token_eager": round(eager_ms, 3),
                     "GB_per_token": round((fc + kv_bytes) / 1e9, 3), "GB/s": round((fc + kv_bytes) / ms / 1e6, 1)}
        del dg, kv
    out["config"] = "Llama-2-7B shape, 32 layers, Q4_1(128) FCs incl. 55296x4096 lm_head, kv-len 2048, batch 1, HIP graph"
    return out


def read_ceiling(torch, llmops, nbytes=2 << 30, reps=4):
    """GB/s of a plain read kernel over a buffer far larger than the caches (the measured ceiling beside the nominal peak)."""
    import ctypes
    lib = llmops._lib.load()
    src = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
    out4 = torch.zeros(4, dtype=torch.int32, device="cuda")
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    llmops._lib.check(lib.llmops_test_calib_read(src.data_ptr(), nbytes, 8192, out4.data_ptr(), st))
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        llmops._lib.check(lib.llmops_test_calib_read(src.data_ptr(), nbytes, 8192, out4.data_ptr(), st))
    e1.record()
    torch.cuda.synchronize()
    return nbytes * reps / (e0.elapsed_time(e1) * 1e-3) / 1e9


def calib(nbytes=1 << 30, reps=5):
    """Plain copy (reads nbytes, writes nbytes per launch) and plain read (reads nbytes) with 16-byte accesses."""
    import ctypes
    import torch
    import llmops
    lib = llmops._lib.load()
    src = torch.randint(0, 255, (nbytes,), dtype=torch.uint8, device="cuda")
    dst = torch.empty_like(src)
    out4 = torch.zeros(4, dtype=torch.int32, device="cuda")
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    res = {"bytes": nbytes}
    for name, fn in (("copy", lambda: lib.llmops_test_calib_copy(src.data_ptr(), dst.data_ptr(), nbytes, 4096, st)),
                     ("read", lambda: lib.llmops_test_calib_read(src.data_ptr(), nbytes, 8192, out4.data_ptr(), st))):
        fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            llmops._lib.check(fn())
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / reps
        res[name] = {"us": round(us, 1), "GB/s_read": round(nbytes / us / 1e3, 1)}
    print(json.dumps({"calib": res}))


INT8_MFMA_PEAK_TOPS = 5033.0  # MI355X published dense int8 rate


def _time_graph(torch, stream, fn, reps=5):
    """Average milliseconds of one fn() call inside a replayed HIP graph (HIP events on the launch stream)."""
    fn()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=stream):
        fn()
    g.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    for _ in range(reps):
        g.replay()
    e1.record(stream)
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / reps


def prefill_gemm(torch, llmops, stream):
    """BASELINE config 3: Q4_1(128) prefill FC, x fp32 [1,M,K], M in {16,128,512,2048}, 4096->11008 and
    11008->4096.  Time covers activation quantization + int8 MFMA GEMM (+ split-K reduce), cycling 8 distinct
    weight copies.  Q8 activation groups are 128 wide, like the weights (the reference has one group size)."""
    out = {}
    gen = torch.Generator(device="cpu").manual_seed(3)
    with torch.cuda.stream(stream):
        for N, K in ((11008, 4096), (4096, 11008)):
            w0 = llmops.offline_FC_quant_Q4A((torch.randn(N, K, generator=gen) * 0.02).cuda(), G)
            ws = [torch.roll(w0, i + 1, 0).contiguous() for i in range(8)]
            for M in (16, 128, 512, 2048):
                x = torch.randn(1, M, K, generator=gen).cuda()

                def run():
                    for w in ws:
                        llmops.fc_Q4A(x, w, N)

                us = _time_graph(torch, stream, run) * 1e3 / len(ws)
                ops = 2.0 * M * N * K
                out[f"{K}->{N} M={M}"] = {"us": round(us, 2), "TOPS": round(ops / us / 1e6, 1),
                                          "pct_int8_mfma_peak": round(ops / us / 1e6 / INT8_MFMA_PEAK_TOPS * 100, 2),
                                          "GB/s": round(fc_bytes(N, K, M) / us / 1e3, 1)}
            del ws, w0
    return out


def decode_fc_g32(torch, llmops, stream):
    """BASELINE config 1: the reference's own CPU-runnable case, one 4096x4096 FC at Q4_1 group 32, M=1
    (seed 1), cycling 32 distinct weight copies in a replayed graph."""
    gen = torch.Generator(device="cpu").manual_seed(1)
    N = K = 4096
    with torch.cuda.stream(stream):
        w0 = llmops.offline_FC_quant_Q4A((torch.randn(N, K, generator=gen) * 0.02).cuda(), 32)
        ws = [torch.roll(w0, i + 1, 0).contiguous() for i in range(32)]
        x = torch.randn(1, 1, K, generator=gen).cuda()

        def run():
            for w in ws:
                llmops.fc_Q4A(x, w, N)

        us = _time_graph(torch, stream, run) * 1e3 / len(ws)
    b = fc_bytes(N, K, 1, 32)
    return {"4096x4096 g32 M=1": {"us": round(us, 2), "GB/s": round(b / us / 1e3, 1), "bytes": b,
                                   "pct_hbm_peak": round(b / us / 1e3 / HBM_PEAK_GBS * 100, 2)}}


def decode_attention(torch, llmops, stream):
    """BASELINE config 4: decode attention with rotary over the KV cache: 32 heads x 128, one query token,
    kv-len 256 / 2048, fp32 and fp16 cache, cycling the 32 layers' planes of one cache."""
    out = {}
    H, S, layers = 32, 128, 32
    gen = torch.Generator(device="cpu").manual_seed(4)
    inv_freq = (1.0 / (10000.0 ** (torch.arange(0, S, 2).float() / S))).cuda()
    with torch.cuda.stream(stream):
        for kv in (256, 2048):
            for name, dt, e in (("fp32", torch.float32, 4), ("fp16", torch.float16, 2)):
                cache = torch.randn(2 * layers, 1, H, kv, S, generator=gen).to(dt).cuda()
                q, k, v = (torch.randn(1, 1, H * S, generator=gen).cuda() for _ in range(3))
                slots = torch.tensor([kv - 1], dtype=torch.int32).cuda()

                def run():
                    for layer in range(layers):
                        llmops.attention_rope2(q, k, v, inv_freq, cache, slots, kv - 1, layer)

                us = _time_graph(torch, stream, run) * 1e3 / layers
                byts = 2 * H * kv * S * e + 16 * H * S
                out[f"kv={kv} {name}"] = {"us": round(us, 2), "GB/s": round(byts / us / 1e3, 1),
                                          "pct_hbm_peak": round(byts / us / 1e3 / HBM_PEAK_GBS * 100, 2), "bytes": byts}
                del cache
    return out


def prefill_attention(torch, llmops, stream):
    """Prompt attention (rope + cache update + causal attention over the chunk itself): 32 heads x 128, fp32
    cache, qL tokens starting at position 0.  FLOPs counted for the causal half: 4 * H * S * qL^2 / 2.  The
    kernel carries every fp32 operand as two fp16 halves and spends 3 fp16 MFMAs (fp32 accumulation) per product:
    `pct_fp32_mfma_peak` compares the useful rate with what the fp32 MFMA could deliver at its peak (the path the
    kernel avoids), `pct_fp16_mfma_peak_3x` with the fp16 peak for the three products it actually issues."""
    out = {}
    H, S = 32, 128
    gen = torch.Generator(device="cpu").manual_seed(6)
    inv_freq = (1.0 / (10000.0 ** (torch.arange(0, S, 2).float() / S))).cuda()
    with torch.cuda.stream(stream):
        for qL in (128, 512, 2048):
            cache = torch.zeros(2, 1, H, 2048, S).cuda()
            q0, k0, v = (torch.randn(1, qL, H * S, generator=gen).cuda() for _ in range(3))
            slots = torch.arange(qL, dtype=torch.int32).cuda()
            qs = [q0.clone() for _ in range(4)]
            ks = [k0.clone() for _ in range(4)]

            def run():
                for q, k in zip(qs, ks):
                    llmops.attention_rope2(q, k, v, inv_freq, cache, slots, 0, 0)

            ms = _time_graph(torch, stream, run, reps=3) / len(qs)
            flops = 4.0 * H * S * qL * qL / 2
            out[f"qL={qL}"] = {"ms": round(ms, 4), "TFLOP/s_causal": round(flops / ms / 1e9, 2),
                               "pct_fp32_mfma_peak": round(flops / ms / 1e9 / 157.3 * 100, 2),
                               "pct_fp16_mfma_peak_3x": round(3 * flops / ms / 1e9 / 2500.0 * 100, 2)}
            del cache
    return out


def cpu_baseline(budget_s=12.0):
    """The CPU path timed on this machine's host cores: a bounded sample (whole layers of the same FC
    set, cycling distinct weight copies as ops/perf_ops.py:234-241 does) for about `budget_s` seconds."""
    import numpy as np
    import oracle

    kind = "reference" if oracle.Reference.available(G) else "port"
    eng = oracle.Reference(G) if kind == "reference" else oracle.Oracle()
    rng = np.random.default_rng(2)
    copies = 4  # 4 distinct layers = 431 MB of packed weights, well beyond the host's last-level cache
    O = oracle.Oracle()
    base = {}
    for name, N, K in LAYER_FCS:
        if (N, K) not in base:
            base[(N, K)] = O.quant_w((rng.standard_normal((N, K)) * 0.02).astype(np.float32), G)
    layers = [[np.roll(base[(N, K)], c * 7 + i + 1, axis=0).copy() for i, (name, N, K) in enumerate(LAYER_FCS)]
              for c in range(copies)]
    xs = {K: rng.standard_normal((1, 1, K)).astype(np.float32) for K in (4096, 11008)}
    for (name, N, K), wq in zip(LAYER_FCS, layers[0]):  # warm-up: thread pool, page faults
        eng.fc(xs[K], wq, N)
    done = 0
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < budget_s:
        for (name, N, K), wq in zip(LAYER_FCS, layers[done % copies]):
            eng.fc(xs[K], wq, N)
        done += 1
    dt = time.perf_counter() - t0
    layer_bytes = sum(fc_bytes(N, K) for _, N, K in LAYER_FCS)
    all_cores = eng.max_threads()
    # the same sample on 8 threads, the thread count of the reference's published CPU figures (README.md:54-57,
    # doc/fc-perf.md:22-26), for about a third of the budget
    eight = None
    if all_cores > 8:
        eng.set_threads(8)
        for (name, N, K), wq in zip(LAYER_FCS, layers[0]):
            eng.fc(xs[K], wq, N)
        n8, t8 = 0, time.perf_counter()
        while time.perf_counter() - t8 < budget_s / 3:
            for (name, N, K), wq in zip(LAYER_FCS, layers[n8 % copies]):
                eng.fc(xs[K], wq, N)
            n8 += 1
        d8 = time.perf_counter() - t8
        eight = {"value": round(n8 * sum(fc_bytes(N, K) for _, N, K in LAYER_FCS) / d8 / 1e9, 2), "unit": "GB/s", "cores": 8,
                 "sample": f"{n8} passes, {d8:.1f} s"}
        eng.set_threads(0)
    res = {"value": round(done * layer_bytes / dt / 1e9, 2), "unit": "GB/s", "cores": all_cores, "kind": kind,
           "isa": eng.isa, "cpu_model": host_cpu_model(), "eight_threads": eight,
           "sample": f"{done} passes over one layer's 7 decode FCs (Q4_1 g128, M=1), cycling {copies} distinct "
                     f"layer weight sets, {dt:.1f} s", "ms_per_layer": round(dt / done * 1e3, 3),
           "ms_per_32_layers": round(dt / done * 32e3, 2)}
    # the other two pieces of a decode step on the same host cores: attention over a 2048-row fp32 cache
    # (4 layers' planes cycled) and the 55296x4096 lm_head, a few seconds each
    H, S, kv, nl = 32, 128, 2048, 4
    cache = rng.standard_normal((2 * nl, 1, H, kv, S)).astype(np.float32)
    q, k, v = (rng.standard_normal((1, 1, H * S)).astype(np.float32) for _ in range(3))
    inv_freq = (1.0 / (10000.0 ** (np.arange(0, S, 2, dtype=np.float32) / np.float32(S)))).astype(np.float32)
    slots = np.array([kv - 1], np.int32)
    att = _CpuAttention(eng, q, k, v, inv_freq, cache, slots, kv - 1)
    att.run(0)
    n, t0 = 0, time.perf_counter()
    while time.perf_counter() - t0 < 4.0:
        att.run(n % nl)
        n += 1
    attn_ms = (time.perf_counter() - t0) / n * 1e3
    wl = O.quant_w((rng.standard_normal((55296, 4096)) * 0.02).astype(np.float32), G)
    eng.fc(xs[4096], wl, 55296)
    n, t0 = 0, time.perf_counter()
    while time.perf_counter() - t0 < 3.0:
        eng.fc(xs[4096], wl, 55296)
        n += 1
    head_ms = (time.perf_counter() - t0) / n * 1e3
    res["decode_step_cpu"] = {"attention_ms_per_layer_kv2048_fp32": round(attn_ms, 3), "lm_head_ms": round(head_ms, 3),
                              "ms_per_token_fc_attention_lm_head": round(32 * (dt / done * 1e3 + attn_ms) + head_ms, 2),
                              "note": "32 x (7 FCs + attention_rope2 at kv-len 2048) + lm_head; norms and element-wise ops "
                                      "not included"}
    return res


class _CpuAttention:
    """attention_rope2 on the host through the raw C entry point (no array copies inside the timed call)."""

    def __init__(self, eng, q, k, v, inv_freq, cache, slots, pos):
        import ctypes
        self.eng, self.arrs, self.pos = eng, (q, k, v, inv_freq, cache, slots), pos
        self.c = ctypes

    def run(self, layer):
        c = self.c
        q, k, v, f, cache, slots = self.arrs
        P = lambda a: c.c_void_p(a.ctypes.data)
        i64 = c.c_int64
        planes, B, H, maxlen, S = cache.shape
        if self.eng.kind == "reference":
            self.eng._warm_rope_table(f)
            rc = self.eng.lib.ref_attention_rope(c.c_int(2), P(q), P(k), P(v), i64(B), i64(1), i64(H), i64(S), P(f),
                                                 i64(f.shape[0]), P(cache), i64(planes), i64(maxlen), P(slots),
                                                 c.c_int(self.pos), c.c_int(layer))
            assert rc == 0
        else:
            self.eng.lib.orc_attention(P(q), P(k), P(v), i64(B), i64(1), i64(H), i64(S), P(f), i64(f.shape[0]), P(cache),
                                       i64(planes), i64(maxlen), P(slots), c.c_int(self.pos), c.c_int(layer))


if __name__ == "__main__":
    main()
