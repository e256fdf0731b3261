// Integer bookkeeping of the persistent decode chain, shared by the host planner and the kernel
// (and by the CPU-side exhaustive check of the decomposition in the tests).
//
// An FC with Ng strips of T steps each is one linear stream of Ttot = Ng*T steps (a step is what a
// wavefront loads at once: one group-128 block or two group-32 blocks; strips are contiguous in the
// packed tensor, so the stream is contiguous memory).  The stream is cut into equal runs of W steps,
// one per workgroup, and every run into 16 nearly equal wave runs.  A strip whose steps fall into
// several workgroups gets one partial sum per workgroup ("contributor"), stored side by side; whoever
// needs the FC's output adds the contributors in workgroup order.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define LLMOPS_HD __host__ __device__ inline
#else
#define LLMOPS_HD inline
#endif

namespace llmops {

constexpr int kChainWaves = 16;          // wavefronts per workgroup
constexpr int kChainMaxStripsPerWg = 17;  // W <= 16*T  =>  a workgroup touches at most 17 strips
constexpr int kChainMaxContrib = 5;       // W >= ceil(T/4) => a strip has at most 5 contributors

struct ChainGeom {
    int T;     // steps per strip
    int Ttot;  // steps of the whole FC
    int W;     // steps per workgroup
};

LLMOPS_HD int chain_wg_begin(const ChainGeom& g, int wg) {
    const int64_t v = (int64_t)wg * g.W;
    return v < g.Ttot ? (int)v : g.Ttot;
}
LLMOPS_HD int chain_wg_end(const ChainGeom& g, int wg) { return chain_wg_begin(g, wg + 1); }

// steps [a, b) of wave `w` inside the workgroup run [ga, gb)
LLMOPS_HD void chain_wave_range(int ga, int gb, int w, int& a, int& b) {
    const int len = gb - ga;
    a = ga + (w * len) / kChainWaves;
    b = ga + ((w + 1) * len) / kChainWaves;
}

// (strip+1)*T <= Ttot < 2^30, so 32-bit arithmetic is exact
LLMOPS_HD int chain_first_wg(const ChainGeom& g, int strip) { return (int)(((uint32_t)strip * (uint32_t)g.T) / (uint32_t)g.W); }
LLMOPS_HD int chain_last_wg(const ChainGeom& g, int strip) {
    return (int)((((uint32_t)strip + 1u) * (uint32_t)g.T - 1u) / (uint32_t)g.W);
}

// Host-side choice of W for a grid of P workgroups; returns false when the FC does not fit the
// kernel's fixed bounds (then the caller must split it along N).
inline bool chain_plan_geom(int Ng, int T, int P, ChainGeom& g, int& active_wgs, int& contributors) {
    const int64_t Ttot = (int64_t)Ng * T;
    if (Ng <= 0 || T <= 0 || P <= 0 || Ttot >= ((int64_t)1 << 30)) return false;
    int64_t W = (Ttot + P - 1) / P;
    const int64_t Wmin = (T + 3) / 4;
    if (W < Wmin) W = Wmin;
    if (W > (int64_t)kChainWaves * T) return false;
    g.T = T;
    g.Ttot = (int)Ttot;
    g.W = (int)W;
    active_wgs = (int)((Ttot + W - 1) / W);
    contributors = 1;
    for (int s = 0; s < Ng; s++) {
        const int c = chain_last_wg(g, s) - chain_first_wg(g, s) + 1;
        if (c > contributors) contributors = c;
    }
    return contributors <= kChainMaxContrib;
}

}  // namespace llmops
