// Integer bookkeeping of the persistent decode chain, shared by the host planner and the kernel
// (and by the CPU-side exhaustive check of the decomposition in the tests).
//
// An FC with Ng strips of T steps each is one linear stream of Ng*T steps (a step is what a
// wavefront loads at once: one group-128 block or two group-32 blocks; strips are contiguous in the
// packed tensor, so the stream is contiguous memory).  Strips are dealt out in whole "units" (one
// strip, or a gate/up strip pair when the op ends in silu(gate)*up): every active workgroup gets m
// consecutive units, so every output column is finished inside one workgroup.  Consecutive ops
// start at different workgroups (rot), so the workgroups that idle in one op are the ones that
// stream the next op's weights ahead.  Inside a workgroup the steps are cut into nearly equal
// contiguous runs, one per streaming wavefront; a run never covers more than two strips.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define LLMOPS_HD __host__ __device__ inline
#else
#define LLMOPS_HD inline
#endif

namespace llmops {

constexpr int kChainWaves = 16;       // wavefronts per workgroup
constexpr int kChainStreamWaves = 8;  // of which stream weights; the others handle activations
constexpr int kChainServiceWaves = kChainWaves - kChainStreamWaves;

struct ChainGeom {
    int T;       // steps per strip
    int us;      // strips per unit (1, or 2 for gate/up pairs)
    int units;   // units of the op
    int m;       // units per active workgroup
    int active;  // workgroups that get work
    int rot;     // first active workgroup
};

// the units [u0, u1) of workgroup `wg` in a grid of P (empty when the workgroup idles in this op)
LLMOPS_HD void chain_wg_units(const ChainGeom& g, int wg, int P, int& u0, int& u1) {
    int local = wg - g.rot;
    if (local < 0) local += P;
    if (local >= g.active) {
        u0 = u1 = 0;
        return;
    }
    u0 = local * g.m;
    u1 = u0 + g.m;
    if (u1 > g.units) u1 = g.units;
}

// steps [a, b) (in the op's linear stream) of streaming wave `w` of a workgroup that owns units [u0, u1)
LLMOPS_HD void chain_wave_range(const ChainGeom& g, int u0, int u1, int w, int& a, int& b) {
    const int tu = g.T * g.us;
    const int ga = u0 * tu, len = (u1 - u0) * tu;
    a = ga + (w * len) / kChainStreamWaves;
    b = ga + ((w + 1) * len) / kChainStreamWaves;
}

// Host-side plan of one op for a grid of P workgroups; `rot` is where the previous op's active
// workgroups ended.  Returns false when the op does not fit the kernel's fixed bounds.
inline bool chain_plan_geom(int Ng, int T, int us, int P, int rot, ChainGeom& g) {
    if (Ng <= 0 || T <= 0 || P <= 0 || (us != 1 && us != 2) || (Ng % us) != 0) return false;
    if ((int64_t)Ng * T >= ((int64_t)1 << 30)) return false;
    g.T = T;
    g.us = us;
    g.units = Ng / us;
    g.m = (g.units + P - 1) / P;
    // a wave's run must not span more than two strips: (m*us*T)/waves <= T
    if (g.m * us > kChainStreamWaves) return false;
    g.active = (g.units + g.m - 1) / g.m;
    g.rot = rot % P;
    return true;
}

}  // namespace llmops
