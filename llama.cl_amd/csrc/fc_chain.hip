// A chain of dependent decode FCs (one activation row) in ONE persistent launch.
//
// Why.  A decode step is a string of small dependent FCs (9-48 MB of weights each).  Launched one
// by one, each pays the dispatch gap plus a load -> quantize -> dot -> reduce latency chain during
// which HBM idles.  Weights do not depend on activations, so here one resident grid (one workgroup
// of 16 wavefronts per CU) walks the whole chain and never stops streaming weights:
//
//   * Wavefronts are specialised.  Streaming waves own a ring of R step slots in LDS (160 KB per CU)
//     that they fill with direct global->LDS loads (global_load_lds_dwordx4: no registers are held
//     while data is in flight) and they issue nothing else to memory, so the ring runs ahead across
//     op boundaries: while an op's result travels across the chip, the next op's weights arrive.
//     Service waves do everything that has memory latency on the critical path: they fetch and
//     quantize the input row, sum the streaming waves' results and publish the outputs.  (Loads of
//     one wave return in issue order, so a wave that keeps a deep weight ring in flight would see
//     every activation load queue behind it; hence the split.)
//   * Work is dealt out in whole output strips (chain_math.h): every output column is finished
//     inside one workgroup, in a fixed order, so results do not depend on timing.
//   * There is no grid barrier.  Outputs are published as 8-byte (value, launch epoch) pairs with
//     write-through stores and consumers poll the pairs they need until the epoch matches: an op
//     boundary costs one store->load trip through the memory side instead of store -> acknowledge ->
//     counter -> poll -> load.  The epoch is a counter in the workspace that the last workgroup to
//     leave advances, so stale pairs of earlier launches (also graph replays) never match.
//
// Per op and workgroup: service waves resolve the input row (plain or published pairs; optional
// rmsnorm) and quantize it once into LDS (same operations as FC_dynamic_quantize_x,
// /root/reference/ops/op_fc.hpp:221-272); streaming waves run the dot4 inner product and fp32 fold
// of the single-FC kernel over their steps (arithmetic of fc_Q4A, ops/op_fc.hpp:286-426); service
// waves add the waves per strip, apply residual or silu(gate)*up, and publish.
//
// Memory visibility across the 8 XCDs (each has its own L2): published pairs are written with
// device-scope write-through stores and read with device-scope (L2-bypassing) loads; everything
// else the kernel reads was written before the launch.  No cache-wide fences.
//
// Every wait is bounded: a poll that does not complete within `spin_limit` ticks of the 100 MHz
// wall clock raises the status word and lets every workgroup leave.
#include "chain_math.h"
#include "common.h"
#include "gemv_device.h"
#include "lds_ring.h"

#include <vector>

namespace llmops {

constexpr int kChainThreads = kChainWaves * 64;
constexpr int kChainMaxK = 16384;  // input row length the LDS staging is sized for
constexpr int kChainSyncBytes = 256;

// sync words at the start of the workspace
enum { kSyncEpoch = 0, kSyncDone = 1, kSyncStatus = 2 };

struct ChainOpDev {
    const uint8_t* w;          // packed weights [Ng][Kg][block]
    const float* x_plain;      // input row written before the launch, or
    const uint64_t* x_pairs;   //   (value, epoch) pairs published by an earlier op of this launch
    const float* norm_w;       // optional rmsnorm weight
    const float* res_plain;    // optional residual, plain or
    const uint64_t* res_pairs;  //   published by an earlier op
    float* y;                  // plain output for the caller
    uint64_t* y_pairs;         // published output for later ops of this launch
    ChainGeom geom;
    int32_t N_out;  // valid outputs
    int32_t K;
    int32_t Tin;  // input steps: K / Step::kK
    int32_t grid;  // workgroups the plan was made for
    float eps;
    int32_t pad_;
};

template <int G>
struct ChainCfg {
    static constexpr int kStepBytes = RingCfg<G>::kStepBytes;
    static constexpr int kLoads = RingCfg<G>::kLoads;
    static constexpr int kXSteps = kChainMaxK / Step<G>::kK;
    static constexpr int kUnitsPerWave = kXSteps / kChainServiceWaves;
    static constexpr int kElemsPerLane = Step<G>::kK / 64;
};

// The op table holds plain pointers, which the compiler would have to treat as generic ("flat")
// addresses; every one of them is device global memory, and saying so gives global_load/_store.
typedef __attribute__((address_space(1))) float gfloat;
typedef __attribute__((address_space(1))) uint64_t gu64;
__device__ __forceinline__ float ld_global(const float* p) { return *(const gfloat*)p; }
__device__ __forceinline__ uint64_t ld_pair(const uint64_t* p) {
    return __hip_atomic_load((const gu64*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_pair(uint64_t* p, float v, uint32_t epoch) {
    __hip_atomic_store((gu64*)p, ((uint64_t)epoch << 32) | (uint64_t)__float_as_uint(v), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
}

// Bounded wait bookkeeping of a polling loop: returns true when the caller should give up.
struct ChainClock {
    long long t_begin, limit;
    unsigned* sync;
    int* pending;
    __device__ __forceinline__ bool expired() const {
        if (*reinterpret_cast<volatile int*>(pending) != 0) return true;
        if (wall_clock64() - t_begin > limit) {
            __hip_atomic_store(&sync[kSyncStatus], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            *reinterpret_cast<volatile int*>(pending) = 1;
            return true;
        }
        return false;
    }
};

// position of a streaming wave in the chain-long sequence of its steps
struct ChainCursor {
    int op, t, end;
    const uint8_t* base;
};

template <int G>
__device__ __forceinline__ bool cursor_next(ChainCursor& c, const ChainOpDev* __restrict__ ops, int n_ops, int wg,
                                            int grid, int wave, const uint8_t*& src) {
    while (c.t >= c.end) {
        c.op++;
        if (c.op >= n_ops) return false;
        const ChainGeom g = ops[c.op].geom;
        int u0, u1;
        chain_wg_units(g, wg, grid, u0, u1);
        chain_wave_range(g, u0, u1, wave, c.t, c.end);
        c.base = ops[c.op].w;
    }
    src = c.base + (int64_t)c.t * ChainCfg<G>::kStepBytes;
    c.t++;
    return true;
}

template <int G, int R>
__global__ __launch_bounds__(kChainThreads) void fc_chain_kernel(const ChainOpDev* __restrict__ ops, int n_ops,
                                                                 unsigned* sync, long long spin_limit,
                                                                 long long* trace) {
    using Cfg = ChainCfg<G>;
    constexpr int SB = Cfg::kStepBytes, KK = Step<G>::kK, UPW = Cfg::kUnitsPerWave, EPL = Cfg::kElemsPerLane;
    constexpr int NS = kChainStreamWaves, NV = kChainServiceWaves;
    __shared__ __align__(16) uint8_t ring[NS][R][SB];
    __shared__ __align__(16) XSlot<G> xrow[Cfg::kXSteps];
    __shared__ float red[NS][2][kGroupN];
    __shared__ int winfo[NS][2];  // first strip of the wave's run, number of strips it flushed
    __shared__ float nred[NV];
    __shared__ int svc_count;  // service-wave rendezvous (the workgroup barrier also involves the streaming waves)
    __shared__ int abort_sh;       // read by every wave right after S1; only written before S1
    __shared__ int abort_pending;  // raised by whoever runs out of time, folded into abort_sh before the next S1

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int quad = lane & 7, rs = lane >> 3;
    const int wg = blockIdx.x, grid = gridDim.x;
    const bool streamer = wave < NS;
    const uint32_t epoch = __hip_atomic_load(&sync[kSyncEpoch], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1u;

    if (threadIdx.x == 0) {
        abort_sh = (ops[0].grid != grid) ? 1 : 0;  // a plan cut for another grid: nothing would line up
        abort_pending = abort_sh;
        svc_count = 0;
        if (ops[0].grid != grid)
            __hip_atomic_store(&sync[kSyncStatus], 2u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();

    if (streamer) {
        // ================= streaming waves: weights only =================
        const bool first_row = (G == 128) ? (rs == 0) : ((rs & 3) == 0);
        uint8_t* myring = &ring[wave][0][0];
        ChainCursor cur{-1, 0, 0, nullptr};
        int issued = 0, consumed = 0, fill = 0, slot = 0;
        if (abort_sh == 0) {
            const uint8_t* src;
            while (issued < R && cursor_next<G>(cur, ops, n_ops, wg, grid, wave, src)) {
                ring_issue<G>(src, myring + fill * SB, lane);
                issued++;
                fill = (fill + 1 == R) ? 0 : fill + 1;
            }
        }
        for (int i = 0; i < n_ops; i++) {
            __syncthreads();  // S1: the input row of op i is quantized in LDS
            if (abort_sh != 0) break;
            const ChainGeom g = ops[i].geom;
            int u0, u1, a, b;
            chain_wg_units(g, wg, grid, u0, u1);
            chain_wave_range(g, u0, u1, wave, a, b);
            const int T = g.T;
            float f[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            int ts = a % T, nseg = 0;
            for (int c = 0; c < b - a; c++) {
                wait_vm((issued - consumed - 1) * Cfg::kLoads);
                Step<G> st;
                ring_read<G>(st, myring + slot * SB, lane);
                const XSlot<G>* xs = &xrow[ts];
                int acc[4];
                dot_step<G>(st, xs->codes, lane, acc);
                const float2 sc = xs->scale[(G == 128) ? 0 : (rs >> 2)];
                fold(f, acc, st.dh, st.mh, sc.x, first_row ? sc.y : 0.0f);
                // the slot is free once its reads have returned; refill it with the next step of the chain
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                consumed++;
                slot = (slot + 1 == R) ? 0 : slot + 1;
                const uint8_t* src;
                if (cursor_next<G>(cur, ops, n_ops, wg, grid, wave, src)) {
                    ring_issue<G>(src, myring + fill * SB, lane);
                    issued++;
                    fill = (fill + 1 == R) ? 0 : fill + 1;
                }
                if (++ts == T || c + 1 == b - a) {  // end of a strip, or of the run: hand the sums over
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        float v = f[j];
                        v += dpp<kRowRor8>(v);
                        v += __shfl_xor(v, 16, 64);
                        v += __shfl_xor(v, 32, 64);
                        if (rs == 0) red[wave][nseg][quad * 4 + j] = v;
                        f[j] = 0.0f;
                    }
                    nseg++;
                    ts = 0;
                }
            }
            if (lane == 0) {
                winfo[wave][0] = a / T;
                winfo[wave][1] = nseg;
            }
            __syncthreads();  // S2: this op's sums are in LDS
        }
        // ring loads still in flight target this workgroup's LDS: drain before leaving
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    } else {
        // ================= service waves: activations in, results out =================
        const int sw = wave - NS;                     // 0..NV-1
        const int stid = threadIdx.x - NS * 64;       // 0..NV*64-1
        const ChainClock clk{wall_clock64(), spin_limit, sync, &abort_pending};
        int rendezvous = 0;
        for (int i = 0; i < n_ops; i++) {
            const ChainOpDev op = ops[i];  // by value: the table entry lives in scalar registers
            int u0, u1;
            chain_wg_units(op.geom, wg, grid, u0, u1);
            const bool active = u0 < u1;
            if (trace != nullptr && stid == 0) trace[((int64_t)wg * n_ops + i) * 4 + 0] = wall_clock64();
            if (*reinterpret_cast<volatile int*>(&abort_pending) != 0) abort_sh = 1;  // before S1, see above

            if (active && *reinterpret_cast<volatile int*>(&abort_pending) == 0) {
                // ---- input row: fetch, optional rmsnorm, quantize once into LDS ----------------------
                XRaw<G> xv[UPW];
                if (op.x_pairs != nullptr) {
                    bool done = false;
                    unsigned spins = 0;
                    while (!done) {
                        bool ok = true;
#pragma unroll
                        for (int j = 0; j < UPW; j++) {
                            const int unit = sw + NV * j;
#pragma unroll
                            for (int e = 0; e < EPL; e++) {
                                float v = 0.0f;
                                if (unit < op.Tin) {
                                    const uint64_t pr = ld_pair(op.x_pairs + unit * KK + lane * EPL + e);
                                    ok = ok && ((uint32_t)(pr >> 32) == epoch);
                                    v = __uint_as_float((uint32_t)pr);
                                }
                                xv[j].v[e] = v;
                            }
                        }
                        done = __all(ok);
                        if (!done) {
                            __builtin_amdgcn_s_sleep(4);
                            if ((++spins & 15u) == 0u && clk.expired()) break;
                        }
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < UPW; j++) {
                        const int unit = sw + NV * j;
#pragma unroll
                        for (int e = 0; e < EPL; e++)
                            xv[j].v[e] = (unit < op.Tin) ? ld_global(op.x_plain + unit * KK + lane * EPL + e) : 0.0f;
                    }
                }
                if (op.norm_w != nullptr) {  // rmsnorm (ops/op_misc.hpp:142-181): x * rsqrt(mean(x^2)+eps) * w
                    XRaw<G> nw[UPW];
#pragma unroll
                    for (int j = 0; j < UPW; j++) {
                        const int unit = sw + NV * j;
#pragma unroll
                        for (int e = 0; e < EPL; e++)
                            nw[j].v[e] = (unit < op.Tin) ? ld_global(op.norm_w + unit * KK + lane * EPL + e) : 0.0f;
                    }
                    float ss = 0.0f;
#pragma unroll
                    for (int j = 0; j < UPW; j++)
#pragma unroll
                        for (int e = 0; e < EPL; e++) ss = fmaf(xv[j].v[e], xv[j].v[e], ss);
                    ss = wave_sum_dpp(ss);
                    // rendezvous of the service waves only (the streaming waves sit in the workgroup barrier)
                    rendezvous += NV;
                    if (lane == 0) {
                        nred[sw] = ss;
                        __hip_atomic_fetch_add(&svc_count, 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
                    }
                    unsigned spins = 0;
                    while (__hip_atomic_load(&svc_count, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) < rendezvous) {
                        __builtin_amdgcn_s_sleep(1);
                        if ((++spins & 255u) == 0u && clk.expired()) break;
                    }
                    float tot = 0.0f;
#pragma unroll
                    for (int w = 0; w < NV; w++) tot += nred[w];
                    const float rsn = 1.0f / sqrtf(tot / (float)op.K + op.eps);
#pragma unroll
                    for (int j = 0; j < UPW; j++)
#pragma unroll
                        for (int e = 0; e < EPL; e++) xv[j].v[e] = xv[j].v[e] * rsn * nw[j].v[e];
                }
#pragma unroll
                for (int j = 0; j < UPW; j++) {
                    const int unit = sw + NV * j;
                    if (unit < op.Tin) quantize_step<G>(xv[j], &xrow[unit], lane);
                }
            }
            if (trace != nullptr && stid == 0) trace[((int64_t)wg * n_ops + i) * 4 + 1] = wall_clock64();
            __syncthreads();  // S1
            if (abort_sh != 0) break;

            // ---- while the streaming waves work: fetch the residual of the columns this thread finishes ----
            const int j = stid >> 5, col = stid & 31;
            const int unit = u0 + j;
            const bool mine = active && unit < u1;
            const int n = unit * kGroupN + col;  // output column (glu: of silu(gate)*up)
            float resv = 0.0f;
            if (mine && n < op.N_out) {
                if (op.res_pairs != nullptr) {
                    unsigned spins = 0;
                    for (;;) {
                        const uint64_t pr = ld_pair(op.res_pairs + n);
                        if ((uint32_t)(pr >> 32) == epoch) {
                            resv = __uint_as_float((uint32_t)pr);
                            break;
                        }
                        __builtin_amdgcn_s_sleep(4);
                        if ((++spins & 15u) == 0u && clk.expired()) break;
                    }
                } else if (op.res_plain != nullptr) {
                    resv = ld_global(op.res_plain + n);
                }
            }
            __syncthreads();  // S2
            if (trace != nullptr && stid == 0) trace[((int64_t)wg * n_ops + i) * 4 + 2] = wall_clock64();

            // ---- add the waves per strip in a fixed order, finish and publish ---------------------
            if (mine) {
                const int us = op.geom.us;
                float sum[2] = {0.0f, 0.0f};
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    const int s = unit * us + h;
                    if (h < us) {
#pragma unroll
                        for (int w = 0; w < NS; w++) {
                            const int fs = winfo[w][0], ns = winfo[w][1];
                            if (ns > 0 && fs == s) sum[h] += red[w][0][col];
                            if (ns > 1 && fs + 1 == s) sum[h] += red[w][1][col];
                        }
                    }
                }
                float v = sum[0];
                if (us == 2) v = silu_times(v, sum[1]);  // silu(gate)*up (ops/op_misc.hpp:83-138)
                v += resv;
                st_pair(op.y_pairs + n, v, epoch);
                if (n < op.N_out) *(gfloat*)(op.y + n) = v;
            }
            if (trace != nullptr && stid == 0) trace[((int64_t)wg * n_ops + i) * 4 + 3] = wall_clock64();
        }
    }

    __syncthreads();
    if (threadIdx.x == 0) {
        const unsigned old = __hip_atomic_fetch_add(&sync[kSyncDone], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (old == (unsigned)grid - 1u) {  // last one out: the next launch gets a fresh epoch
            __hip_atomic_store(&sync[kSyncEpoch], epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&sync[kSyncDone], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

// ---- host side ---------------------------------------------------------------------------------

static int g_chain_ring = 0;  // 0 = default depth
static int g_chain_grid = 0;  // 0 = one workgroup per CU
static long long g_chain_spin_limit = 100000000LL;  // 1 s of the 100 MHz wall clock
static long long* g_chain_trace = nullptr;          // optional per-workgroup phase timestamps

static int chain_grid(int* out) {
    int dev = 0, cus = 0;
    LLMOPS_HIP_CHECK(hipGetDevice(&dev));
    LLMOPS_HIP_CHECK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    if (cus <= 0) return fail(LLMOPS_EHIP, "device reports %d compute units", cus);
    *out = (g_chain_grid > 0 && g_chain_grid < cus) ? g_chain_grid : cus;
    return LLMOPS_OK;
}

static inline size_t chain_align(size_t v) { return (v + 255) / 256 * 256; }

// bytes of the published (value, epoch) pairs of one op
static inline size_t chain_pairs_bytes(const llmops_chain_op& o) {
    return chain_align((size_t)(o.Ng / (o.glu ? 2 : 1)) * kGroupN * sizeof(uint64_t));
}

// the latest op before `i` whose output buffer is `p` (-1: none), and whether `i` or a later op writes `p`
static int chain_producer(const llmops_chain_op* ops, int i, const void* p) {
    for (int j = i - 1; j >= 0; j--)
        if (ops[j].y == p) return j;
    return -1;
}
static bool chain_written_from(const llmops_chain_op* ops, int n_ops, int i, const void* p) {
    for (int j = i; j < n_ops; j++)
        if (ops[j].y == p) return true;
    return false;
}

// checks one op of the chain and cuts it; on failure the thread's error text says why
static int chain_check_op(const llmops_chain_op* ops, int n_ops, int i, int G, int P, int rot, ChainGeom& geom) {
    const llmops_chain_op& o = ops[i];
    const int bps = (G == 128) ? 1 : 2;
    LLMOPS_REQUIRE(o.weiq != nullptr && o.y != nullptr);
    LLMOPS_REQUIRE(o.Ng > 0 && o.Kg > 0 && o.Ng <= 65536 && o.Kg <= 65536);
    LLMOPS_REQUIRE((o.Kg % bps) == 0);  // a step never straddles two strips
    const int64_t K = o.Kg * G;
    LLMOPS_REQUIRE(K <= kChainMaxK);
    LLMOPS_REQUIRE(aligned(o.weiq, 16) && aligned(o.y, 4));
    if (o.glu) {
        LLMOPS_REQUIRE((o.Ng % 2) == 0 && o.residual == nullptr);
        LLMOPS_REQUIRE(o.N_out > (o.Ng / 2 - 1) * kGroupN && o.N_out <= o.Ng / 2 * kGroupN);
    } else {
        LLMOPS_REQUIRE(o.N_out > (o.Ng - 1) * kGroupN && o.N_out <= o.Ng * kGroupN);
    }
    if (o.x == nullptr) {
        LLMOPS_REQUIRE(i > 0);  // "previous op's output" needs a previous op
        LLMOPS_REQUIRE(ops[i - 1].N_out == K);
    } else {
        LLMOPS_REQUIRE(aligned(o.x, 4));
        const int src = chain_producer(ops, i, o.x);
        if (src >= 0) LLMOPS_REQUIRE(ops[src].N_out == K);
        // a row that is read as it was before the launch must not be overwritten during the launch:
        // without grid-wide barriers a fast workgroup may be ops ahead of a slow one
        if (src < 0) LLMOPS_REQUIRE(!chain_written_from(ops, n_ops, i, o.x));
    }
    if (o.residual != nullptr) {
        LLMOPS_REQUIRE(aligned(o.residual, 4));
        const int src = chain_producer(ops, i, o.residual);
        if (src >= 0) LLMOPS_REQUIRE(ops[src].N_out == o.N_out);
        // plain residual: only this op itself may write the buffer (in place, column by column)
        if (src < 0) LLMOPS_REQUIRE(!chain_written_from(ops, n_ops, i + 1, o.residual));
    }
    // an output buffer is written by one op only: plain stores of two ops to one address could reach
    // memory in either order (different L2s)
    LLMOPS_REQUIRE(chain_producer(ops, i, o.y) < 0);
    if (!chain_plan_geom((int)o.Ng, (int)(o.Kg / bps), o.glu ? 2 : 1, P, rot, geom))
        return fail(LLMOPS_EINVAL, "chain op %d (Ng=%lld, Kg=%lld) does not fit the persistent kernel; split it along N", i,
                    (long long)o.Ng, (long long)o.Kg);
    return LLMOPS_OK;
}

template <int G, int R>
static void chain_launch(const ChainOpDev* plan, int n_ops, unsigned* sync, int grid, hipStream_t st) {
    fc_chain_kernel<G, R><<<(unsigned)grid, kChainThreads, 0, st>>>(plan, n_ops, sync, g_chain_spin_limit, g_chain_trace);
}

}  // namespace llmops

using namespace llmops;

extern "C" size_t llmops_fc_chain_plan_bytes(int n_ops) {
    return n_ops > 0 ? chain_align((size_t)n_ops * sizeof(ChainOpDev)) : 0;
}

extern "C" int llmops_fc_chain_workspace_bytes(const llmops_chain_op* ops, int n_ops, int group_k, size_t* bytes) {
    LLMOPS_REQUIRE(ops != nullptr && bytes != nullptr && n_ops > 0 && n_ops <= 4096);
    LLMOPS_REQUIRE(valid_group(group_k));
    int P = 0;
    int rc = chain_grid(&P);
    if (rc) return rc;
    size_t total = kChainSyncBytes;
    int rot = 0;
    for (int i = 0; i < n_ops; i++) {
        ChainGeom g;
        rc = chain_check_op(ops, n_ops, i, group_k, P, rot, g);
        if (rc) return rc;
        rot = (g.rot + g.active) % P;
        total += chain_pairs_bytes(ops[i]);
    }
    *bytes = total;
    return LLMOPS_OK;
}

extern "C" int llmops_fc_chain_build(const llmops_chain_op* ops, int n_ops, int group_k, void* plan, size_t plan_bytes,
                                     void* workspace, size_t workspace_bytes) {
    LLMOPS_REQUIRE(ops != nullptr && plan != nullptr && workspace != nullptr && n_ops > 0 && n_ops <= 4096);
    LLMOPS_REQUIRE(valid_group(group_k));
    LLMOPS_REQUIRE(aligned(plan, 16) && aligned(workspace, 256));
    LLMOPS_REQUIRE(plan_bytes >= llmops_fc_chain_plan_bytes(n_ops));
    int P = 0;
    int rc = chain_grid(&P);
    if (rc) return rc;
    const int bps = (group_k == 128) ? 1 : 2;
    std::vector<ChainOpDev> dev((size_t)n_ops);
    size_t off = kChainSyncBytes;
    int rot = 0;
    for (int i = 0; i < n_ops; i++) {
        const llmops_chain_op& o = ops[i];
        ChainOpDev& d = dev[(size_t)i];
        rc = chain_check_op(ops, n_ops, i, group_k, P, rot, d.geom);
        if (rc) return rc;
        rot = (d.geom.rot + d.geom.active) % P;
        d.w = reinterpret_cast<const uint8_t*>(o.weiq);
        const int xsrc = (o.x == nullptr) ? i - 1 : chain_producer(ops, i, o.x);
        d.x_plain = (xsrc < 0) ? o.x : nullptr;
        d.x_pairs = (xsrc >= 0) ? dev[(size_t)xsrc].y_pairs : nullptr;
        d.norm_w = o.norm_w;
        const int rsrc = (o.residual == nullptr) ? -1 : chain_producer(ops, i, o.residual);
        d.res_plain = (o.residual != nullptr && rsrc < 0) ? o.residual : nullptr;
        d.res_pairs = (rsrc >= 0) ? dev[(size_t)rsrc].y_pairs : nullptr;
        d.y = o.y;
        d.y_pairs = reinterpret_cast<uint64_t*>(reinterpret_cast<uint8_t*>(workspace) + off);
        d.N_out = (int32_t)o.N_out;
        d.K = (int32_t)(o.Kg * group_k);
        d.Tin = (int32_t)(o.Kg / bps);
        d.grid = P;
        d.eps = o.eps;
        d.pad_ = 0;
        off += chain_pairs_bytes(o);
    }
    if (workspace_bytes < off)
        return fail(LLMOPS_EWORKSPACE, "fc chain needs %zu workspace bytes, got %zu", off, workspace_bytes);
    LLMOPS_HIP_CHECK(hipMemcpy(plan, dev.data(), (size_t)n_ops * sizeof(ChainOpDev), hipMemcpyHostToDevice));
    return LLMOPS_OK;
}

extern "C" int llmops_fc_chain_run(const void* plan, int n_ops, int group_k, void* workspace, llmops_stream_t stream) {
    LLMOPS_REQUIRE(plan != nullptr && workspace != nullptr && n_ops > 0);
    LLMOPS_REQUIRE(valid_group(group_k));
    int P = 0;
    const int rc = chain_grid(&P);
    if (rc) return rc;
    const ChainOpDev* p = reinterpret_cast<const ChainOpDev*>(plan);
    unsigned* sync = reinterpret_cast<unsigned*>(workspace);
    hipStream_t st = as_stream(stream);
    const int ring = g_chain_ring > 0 ? g_chain_ring : 6;
    if (group_k == 128) {
        if (ring <= 4) chain_launch<128, 4>(p, n_ops, sync, P, st);
        else if (ring <= 6) chain_launch<128, 6>(p, n_ops, sync, P, st);
        else chain_launch<128, 8>(p, n_ops, sync, P, st);
    } else {
        if (ring <= 4) chain_launch<32, 4>(p, n_ops, sync, P, st);
        else if (ring <= 6) chain_launch<32, 6>(p, n_ops, sync, P, st);
        else chain_launch<32, 8>(p, n_ops, sync, P, st);
    }
    LLMOPS_LAUNCH_CHECK();
    return LLMOPS_OK;
}

extern "C" int llmops_fc_chain_status(const void* workspace, int32_t* status) {
    LLMOPS_REQUIRE(workspace != nullptr && status != nullptr);
    uint32_t words[4] = {0, 0, 0, 0};
    LLMOPS_HIP_CHECK(hipMemcpy(words, workspace, sizeof(words), hipMemcpyDeviceToHost));
    *status = (int32_t)words[kSyncStatus];
    return LLMOPS_OK;
}

extern "C" void llmops_fc_chain_set_trace(void* buffer) { llmops::g_chain_trace = reinterpret_cast<long long*>(buffer); }

extern "C" void llmops_fc_chain_set_tuning(int ring_depth, int grid, long long spin_limit_ticks) {
    if (ring_depth >= 0) llmops::g_chain_ring = ring_depth;
    if (grid >= 0) llmops::g_chain_grid = grid;
    if (spin_limit_ticks > 0) llmops::g_chain_spin_limit = spin_limit_ticks;
}
