// A chain of dependent decode FCs (one activation row) in ONE persistent launch.
//
// Why.  A decode step is a string of small dependent FCs (9-48 MB of weights each).  Launched one
// by one, each pays the dispatch gap plus a load -> quantize -> dot -> reduce latency chain during
// which HBM idles.  Weights do not depend on activations, so here one resident grid (one workgroup
// of 16 wavefronts per CU) walks the whole chain and keeps the weight stream of the NEXT FC in
// flight while the current one finishes and its result crosses the chip:
//
//   * every wavefront owns a ring of R step slots in LDS (160 KB per CU) filled by direct
//     global->LDS loads (global_load_lds_dwordx4: no registers held while the data is in flight);
//   * an FC's steps are cut evenly over all workgroups (chain_math.h), so every CU streams the
//     same number of bytes whatever the shape;
//   * a strip that spans several workgroups is not finished by a ticket hand-off: each workgroup
//     stores its partial sums (write-through) and the CONSUMER of the FC's output adds them while
//     it loads its input row, so an FC boundary costs exactly one grid-wide barrier;
//   * right after arriving at that barrier a wavefront refills its ring with the first steps of the
//     next FC, and only then waits.
//
// Per FC and workgroup: resolve the input row (sum the previous FC's partials, optional
// silu(gate)*up, optional rmsnorm), quantize it once into LDS (same operations as
// FC_dynamic_quantize_x, /root/reference/ops/op_fc.hpp:221-272), stream the workgroup's steps
// (same dot4 inner product and fp32 fold as the single-FC kernel; arithmetic of fc_Q4A,
// ops/op_fc.hpp:286-426), reduce over waves in a fixed order, store the partials, barrier.
// Summation orders are fixed by the decomposition, so results do not depend on timing.
//
// Memory visibility across the 8 XCDs (each has its own L2): partial sums, materialized outputs
// and the barrier counter are written with device-scope write-through stores / atomics; partial
// sums are read back with ordinary cached loads, which is sound because every FC of a chain has
// its own partial region and no line of it is touched before the barrier that completes it;
// residual inputs, which may alias outputs written earlier in the same launch, are read with
// device-scope loads.  No cache-wide fences.
//
// Every wait is bounded: the barrier spin gives up after `spin_limit` ticks of the 100 MHz
// wall clock, raises the status word and lets every workgroup leave.
#include "chain_math.h"
#include "common.h"
#include "gemv_device.h"

#include <vector>

namespace llmops {

constexpr int kChainThreads = kChainWaves * 64;
constexpr int kChainMaxK = 16384;  // input row length the LDS staging is sized for
constexpr int kChainSyncBytes = 256;

// sync words at the start of the workspace
enum { kSyncBar = 0, kSyncDone = 1, kSyncStatus = 2 };

struct ChainOpDev {
    const uint8_t* w;       // packed weights [Ng][Kg][block]
    const float* x;         // input row, or nullptr: the previous op's output
    const float* norm_w;    // optional rmsnorm weight
    const float* residual;  // optional, added to the output
    float* y;               // materialized output (may be nullptr for an inner op)
    float* part;            // partial sums [contributors][Np]
    ChainGeom geom;         // T, Ttot, W
    int32_t contrib;  // partial-sum slots per strip
    int32_t Np;       // Ng*32
    int32_t N_out;  // valid outputs (GLU: Np/2 at most)
    int32_t K;
    int32_t Tin;  // input steps: K / Step::kK
    int32_t glu;
    int32_t grid;  // workgroups the plan was made for
    float eps;
};

template <int G>
struct ChainCfg {
    static constexpr int kStepBytes = Step<G>::kBlocksPerStep * (int)block_bytes(G);  // 2176 / 1280
    static constexpr int kLoads = (kStepBytes + 1023) / 1024;                         // wave-wide 16 B loads per step
    static constexpr int kXSteps = kChainMaxK / Step<G>::kK;
    static constexpr int kUnitsPerWave = kXSteps / kChainWaves;
    static constexpr int kElemsPerLane = Step<G>::kK / 64;
};

// One 16-byte-per-lane asynchronous copy global -> LDS: lane i's 16 bytes land at lds_base + 16*i.
// Written as assembly on purpose.  The compiler, when it knows that such copies are pending, makes
// every later LDS access wait for all of them (it cannot tell which LDS bytes they target), which
// would serialise the ring; this way it sees an opaque memory operation, and the waits on the ring
// are placed by hand (wait_vm).  Hidden loads are harmless for the waits the compiler places for its
// own loads: loads complete in issue order, so an unknown older load only makes such a wait longer.
__device__ __forceinline__ void dma16(const uint8_t* gptr, uint32_t lds_base) {
    asm volatile(
        "s_mov_b32 m0, %1\n\t"
        "s_nop 0\n\t"
        "global_load_lds_dwordx4 %0, off nt"
        :
        : "v"(gptr), "s"(lds_base)
        : "memory", "m0");
}

__device__ __forceinline__ uint32_t lds_addr(const void* p) {
    return (uint32_t)(uintptr_t)((const __attribute__((address_space(3))) void*)p);
}

// one step of the weight stream, global -> LDS (counts in vmcnt)
template <int G>
__device__ __forceinline__ void ring_issue(const uint8_t* src, uint8_t* slot, int lane) {
    constexpr int SB = ChainCfg<G>::kStepBytes;
    const uint32_t base = __builtin_amdgcn_readfirstlane(lds_addr(slot));
#pragma unroll
    for (int o = 0; o < SB; o += 1024) {
        if (SB - o >= 1024) {
            dma16(src + o + lane * 16, base + o);
        } else if (lane * 16 < SB - o) {
            dma16(src + o + lane * 16, base + o);
        }
    }
}

template <int G>
__device__ __forceinline__ void ring_read(Step<G>& st, const uint8_t* slot, int lane) {
    const int quad = lane & 7, rs = lane >> 3;
    st.valid = true;
    if (G == 128) {
        st.w[0] = *reinterpret_cast<const uint4*>(slot + lane * 16);
        st.w[Step<G>::kLoads - 1] = *reinterpret_cast<const uint4*>(slot + 1024 + lane * 16);
        st.dh = *reinterpret_cast<const uint2*>(slot + 2048 + quad * 8);
        st.mh = *reinterpret_cast<const uint2*>(slot + 2048 + 64 + quad * 8);
    } else {
        const uint8_t* blk = slot + (rs >> 2) * (int)block_bytes(32);
        st.w[0] = *reinterpret_cast<const uint4*>(blk + (rs & 3) * kRowBytes + quad * 16);
        st.dh = *reinterpret_cast<const uint2*>(blk + 512 + quad * 8);
        st.mh = *reinterpret_cast<const uint2*>(blk + 512 + 64 + quad * 8);
    }
}

// wait until at most `loads` of this wave's vector-memory operations are outstanding
template <int MAXV>
__device__ __forceinline__ void wait_vm(int loads) {
    static_assert(MAXV <= 15, "ring too deep for the wait table");
    switch (loads) {
#define LLMOPS_W(n) \
    case n:         \
        asm volatile("s_waitcnt vmcnt(" #n ")" ::: "memory"); \
        break;
        LLMOPS_W(1) LLMOPS_W(2) LLMOPS_W(3) LLMOPS_W(4) LLMOPS_W(5) LLMOPS_W(6) LLMOPS_W(7) LLMOPS_W(8)
        LLMOPS_W(9) LLMOPS_W(10) LLMOPS_W(11) LLMOPS_W(12) LLMOPS_W(13) LLMOPS_W(14) LLMOPS_W(15)
#undef LLMOPS_W
        default:
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            break;
    }
}

// The op table holds plain pointers, which the compiler would have to treat as generic ("flat")
// addresses; every one of them is device global memory, and saying so gives global_load/_store.
typedef __attribute__((address_space(1))) float gfloat;
__device__ __forceinline__ float ld_global(const float* p) { return *(const gfloat*)p; }
__device__ __forceinline__ float ld_agent(const float* p) {
    return __hip_atomic_load((const gfloat*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_agent(float* p, float v) {
    __hip_atomic_store((gfloat*)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// sum of the contributor slots at flat column index idx, in workgroup order; every op stores all
// `contrib` slots of every strip (unused ones as zeros), so no per-strip bookkeeping is needed here
__device__ __forceinline__ float chain_sum(const ChainOpDev& p, int idx) {
    // branch-free so that all loads are in flight together: a slot beyond `contrib` re-reads slot 0
    float v[kChainMaxContrib];
#pragma unroll
    for (int c = 0; c < kChainMaxContrib; c++) v[c] = ld_global(p.part + (int64_t)(c < p.contrib ? c : 0) * p.Np + idx);
    float s = v[0];
#pragma unroll
    for (int c = 1; c < kChainMaxContrib; c++) s += (c < p.contrib) ? v[c] : 0.0f;
    return s;
}

// output element k of op p: contributors added up; gate/up pairs combined as silu(gate)*up
// (itrans "silu" + imul, ops/op_misc.hpp:83-138)
__device__ __forceinline__ float chain_resolve(const ChainOpDev& p, int k) {
    if (!p.glu) return chain_sum(p, k);
    const int u = k >> 5, col = k & 31;
    const float g = chain_sum(p, (2 * u) * kGroupN + col);
    const float up = chain_sum(p, (2 * u + 1) * kGroupN + col);
    return up * (g * (1.0f / (1.0f + expf(-g))));
}

// the share of op p's output that this workgroup writes out (128 outputs per wave at a time)
__device__ __forceinline__ void chain_materialize(const ChainOpDev& p, int wg, int grid, int wave, int lane) {
    if (p.y == nullptr) return;
    const int chunks = (p.N_out + 127) >> 7;
    for (int u = wg + grid * wave; u < chunks; u += grid * kChainWaves) {
#pragma unroll
        for (int e = 0; e < 2; e++) {
            const int k = u * 128 + lane * 2 + e;
            if (k < p.N_out) st_agent(p.y + k, chain_resolve(p, k));
        }
    }
}

template <int G, int R>
__global__ __launch_bounds__(kChainThreads) void fc_chain_kernel(const ChainOpDev* __restrict__ ops, int n_ops,
                                                                 unsigned* sync, long long spin_limit,
                                                                 long long* trace) {
    using Cfg = ChainCfg<G>;
    constexpr int SB = Cfg::kStepBytes, KK = Step<G>::kK, UPW = Cfg::kUnitsPerWave, EPL = Cfg::kElemsPerLane;
    __shared__ __align__(16) uint8_t ring[kChainWaves][R][SB];
    __shared__ __align__(16) XSlot<G> xrow[Cfg::kXSteps];
    __shared__ float red[kChainWaves][2][kGroupN];
    __shared__ int winfo[kChainWaves][2];  // first strip of the wave, number of strips it flushed
    __shared__ float nred[kChainWaves];
    __shared__ int abort_sh;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int quad = lane & 7, rs = lane >> 3;
    const int wg = blockIdx.x, grid = gridDim.x;
    const bool first_row = (G == 128) ? (rs == 0) : ((rs & 3) == 0);
    uint8_t* myring = &ring[wave][0][0];
    const long long t_begin = wall_clock64();

    bool aborted = false;
    if (ops[0].grid != grid) {  // the plan was cut for another grid: nothing below would line up
        if (threadIdx.x == 0) __hip_atomic_store(&sync[kSyncStatus], 2u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        aborted = true;
    }

    // ring state of this wave for the op it is about to run: steps [a, b), `issued` of them requested
    int a = 0, b = 0, issued = 0;
    if (!aborted) {
        chain_wave_range(chain_wg_begin(ops[0].geom, wg), chain_wg_end(ops[0].geom, wg), wave, a, b);
        const uint8_t* wsrc = ops[0].w;
        for (; issued < R && a + issued < b; issued++)
            ring_issue<G>(wsrc + (int64_t)(a + issued) * SB, myring + issued * SB, lane);
    }

    for (int i = 0; i < n_ops && !aborted; i++) {
        const ChainOpDev op = ops[i];                  // by value: the table entries live in scalar registers
        const ChainOpDev prev = ops[i > 0 ? i - 1 : 0];
        const int ga = chain_wg_begin(op.geom, wg), gb = chain_wg_end(op.geom, wg);
        const int T = op.geom.T;

        if (trace != nullptr && threadIdx.x == 0) trace[((int64_t)wg * n_ops + i) * 4 + 0] = wall_clock64();
        if (ga < gb) {  // uniform over the workgroup
            // ---- input row: resolve, optional rmsnorm, quantize once into LDS ---------------------
            XRaw<G> xv[UPW];
#pragma unroll
            for (int j = 0; j < UPW; j++) {
                const int unit = wave + kChainWaves * j;
#pragma unroll
                for (int e = 0; e < EPL; e++) {
                    const int k = unit * KK + lane * EPL + e;
                    float v = 0.0f;
                    if (unit < op.Tin) v = (op.x != nullptr) ? ld_global(op.x + k) : chain_resolve(prev, k);
                    xv[j].v[e] = v;
                }
            }
            if (op.norm_w != nullptr) {  // rmsnorm (ops/op_misc.hpp:142-181): x * rsqrt(mean(x^2)+eps) * w
                XRaw<G> nw[UPW];
#pragma unroll
                for (int j = 0; j < UPW; j++) {
                    const int unit = wave + kChainWaves * j;
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
                if (lane == 0) nred[wave] = ss;
                __syncthreads();
                float tot = 0.0f;
#pragma unroll
                for (int w = 0; w < kChainWaves; w++) tot += nred[w];
                const float rsn = 1.0f / sqrtf(tot / (float)op.K + op.eps);
#pragma unroll
                for (int j = 0; j < UPW; j++)
#pragma unroll
                    for (int e = 0; e < EPL; e++)
                        xv[j].v[e] = xv[j].v[e] * rsn * nw[j].v[e];
            }
#pragma unroll
            for (int j = 0; j < UPW; j++) {
                const int unit = wave + kChainWaves * j;
                if (unit < op.Tin) quantize_step<G>(xv[j], &xrow[unit], lane);
            }
            __syncthreads();
            if (trace != nullptr && threadIdx.x == 0) trace[((int64_t)wg * n_ops + i) * 4 + 1] = wall_clock64();

            // ---- stream this wave's steps out of its ring -----------------------------------------
            float f[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            int ts = a % T, nseg = 0, slot = 0, fill = issued % R;
            const uint8_t* wsrc = op.w;
            for (int c = 0; c < b - a; c++) {
                wait_vm<(R - 1) * Cfg::kLoads>((issued - c - 1) * Cfg::kLoads);
                Step<G> st;
                ring_read<G>(st, myring + slot * SB, lane);
                const XSlot<G>* xs = &xrow[ts];
                int acc[4];
                dot_step<G>(st, xs->codes, lane, acc);
                const float2 sc = xs->scale[(G == 128) ? 0 : (rs >> 2)];
                fold(f, acc, st.dh, st.mh, sc.x, first_row ? sc.y : 0.0f);
                // the slot is free once its reads have returned; refill it with this op's next step
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                if (a + issued < b) {
                    ring_issue<G>(wsrc + (int64_t)(a + issued) * SB, myring + fill * SB, lane);
                    issued++;
                    fill = (fill + 1 == R) ? 0 : fill + 1;
                }
                slot = (slot + 1 == R) ? 0 : slot + 1;
                if (++ts == T || c + 1 == b - a) {  // end of a strip, or of the run: hand the sums to the workgroup
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
        }

        // ---- outputs of the previous op that this workgroup writes out ----------------------------
        if (i > 0) chain_materialize(prev, wg, grid, wave, lane);

        if (ga < gb) {
            // ---- sum the waves per strip (fixed order) and store this workgroup's partial sums ------
            __syncthreads();
            if (trace != nullptr && threadIdx.x == 0) trace[((int64_t)wg * n_ops + i) * 4 + 2] = wall_clock64();
            const int s_lo = ga / T, s_hi = (gb - 1) / T;
            const int s = s_lo + (threadIdx.x >> 5), col = threadIdx.x & 31;
            if (s <= s_hi) {
                float v = 0.0f;
#pragma unroll
                for (int w = 0; w < kChainWaves; w++) {
                    const int fs = winfo[w][0], ns = winfo[w][1];
                    if (ns > 0 && fs == s) v += red[w][0][col];
                    if (ns > 1 && fs + 1 == s) v += red[w][1][col];
                }
                const int first = chain_first_wg(op.geom, s);
                const int c = wg - first;
                const int n = s * kGroupN + col;
                if (c == 0) {
                    if (op.residual != nullptr && n < op.N_out) v += ld_agent(op.residual + n);
                    // slots that no workgroup owns for this strip read as zero
                    for (int z = chain_last_wg(op.geom, s) - first + 1; z < op.contrib; z++)
                        st_agent(op.part + (int64_t)z * op.Np + n, 0.0f);
                }
                st_agent(op.part + (int64_t)c * op.Np + n, v);
            }
        }

        // ---- grid barrier: stores acknowledged, arrive, refill the ring for the next op, wait ------
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (threadIdx.x == 0) __hip_atomic_fetch_add(&sync[kSyncBar], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (trace != nullptr && threadIdx.x == 0) trace[((int64_t)wg * n_ops + i) * 4 + 3] = wall_clock64();
        a = b = issued = 0;
        if (i + 1 < n_ops) {
            const ChainGeom ng = ops[i + 1].geom;
            chain_wave_range(chain_wg_begin(ng, wg), chain_wg_end(ng, wg), wave, a, b);
            const uint8_t* wsrc = ops[i + 1].w;
            for (; issued < R && a + issued < b; issued++)
                ring_issue<G>(wsrc + (int64_t)(a + issued) * SB, myring + issued * SB, lane);
        }
        if (threadIdx.x == 0) {
            const unsigned target = (unsigned)(i + 1) * (unsigned)grid;
            int bad = 0;
            unsigned spins = 0;
            while (__hip_atomic_load(&sync[kSyncBar], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
                __builtin_amdgcn_s_sleep(1);
                if ((++spins & 31u) == 0u) {
                    if (__hip_atomic_load(&sync[kSyncStatus], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u) {
                        bad = 1;
                        break;
                    }
                    if (wall_clock64() - t_begin > spin_limit) {
                        __hip_atomic_store(&sync[kSyncStatus], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        bad = 1;
                        break;
                    }
                }
            }
            abort_sh = bad;
        }
        __syncthreads();
        if (abort_sh) aborted = true;
    }

    if (!aborted) {
        const ChainOpDev last = ops[n_ops - 1];
        chain_materialize(last, wg, grid, wave, lane);
    }

    // every ring load that is still in flight targets this workgroup's LDS: drain before leaving
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
        const unsigned old = __hip_atomic_fetch_add(&sync[kSyncDone], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (old == (unsigned)grid - 1u) {  // last one out leaves the counters ready for the next launch
            __hip_atomic_store(&sync[kSyncBar], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
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

struct ChainPlanHost {
    ChainGeom geom;
    int active, contrib;
};

// checks one op of the chain and cuts it; on failure the thread's error text says why
static int chain_check_op(const llmops_chain_op* ops, int i, int G, int P, ChainPlanHost& ph) {
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
        LLMOPS_REQUIRE(i > 0);                // "previous op's output" needs a previous op
        LLMOPS_REQUIRE(ops[i - 1].N_out == K);
    } else {
        LLMOPS_REQUIRE(aligned(o.x, 4));
        // a row that this launch also writes would be read through caches that may hold its old lines
        for (int j = 0; j < i; j++) LLMOPS_REQUIRE(o.x != ops[j].y);
    }
    // the residual is read before the barrier that ends this op; the previous op's output is only
    // written out after that op's barrier by other workgroups, which may still be at it
    if (o.residual != nullptr && i > 0) LLMOPS_REQUIRE(o.residual != ops[i - 1].y);
    if (!chain_plan_geom((int)o.Ng, (int)(o.Kg / bps), P, ph.geom, ph.active, ph.contrib))
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
    for (int i = 0; i < n_ops; i++) {
        ChainPlanHost ph;
        rc = chain_check_op(ops, i, group_k, P, ph);
        if (rc) return rc;
        total += chain_align((size_t)ph.contrib * ops[i].Ng * kGroupN * sizeof(float));
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
    for (int i = 0; i < n_ops; i++) {
        ChainPlanHost ph;
        rc = chain_check_op(ops, i, group_k, P, ph);
        if (rc) return rc;
        const llmops_chain_op& o = ops[i];
        ChainOpDev& d = dev[(size_t)i];
        d.w = reinterpret_cast<const uint8_t*>(o.weiq);
        d.x = o.x;
        d.norm_w = o.norm_w;
        d.residual = o.residual;
        d.y = o.y;
        d.part = reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(workspace) + off);
        d.geom = ph.geom;
        d.contrib = ph.contrib;
        d.Np = (int32_t)(o.Ng * kGroupN);
        d.N_out = (int32_t)o.N_out;
        d.K = (int32_t)(o.Kg * group_k);
        d.Tin = (int32_t)(o.Kg / bps);
        d.glu = o.glu ? 1 : 0;
        d.grid = P;
        d.eps = o.eps;
        off += chain_align((size_t)ph.contrib * o.Ng * kGroupN * sizeof(float));
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
    const int ring = g_chain_ring > 0 ? g_chain_ring : 4;
    if (group_k == 128) {
        if (ring <= 2) chain_launch<128, 2>(p, n_ops, sync, P, st);
        else if (ring == 3) chain_launch<128, 3>(p, n_ops, sync, P, st);
        else chain_launch<128, 4>(p, n_ops, sync, P, st);
    } else {
        if (ring <= 2) chain_launch<32, 2>(p, n_ops, sync, P, st);
        else if (ring == 3) chain_launch<32, 3>(p, n_ops, sync, P, st);
        else chain_launch<32, 4>(p, n_ops, sync, P, st);
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
