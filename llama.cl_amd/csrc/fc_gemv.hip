// Q4_1 x Q8 fully-connected product for a handful of activation rows (decode): an HBM-streaming
// kernel built on v_dot4_i32_i8.
//
// Data movement.  The packed tensor [Ng][Kg][block] is a set of Ng independent strips (32 output
// columns each) whose blocks are contiguous in memory, so a strip is one linear stream.  Work is
// cut into (strip, k-range) tiles: one workgroup per tile, each of its NW wavefronts streaming a
// contiguous run of blocks with 16-byte loads per lane:
//
//   lane = rs*8 + quad,  rs = 0..7 (k8-row slot), quad = 0..7 (4 adjacent columns)
//   one wave-wide 16 B load = 8 k8-rows x 128 B = 64 k-values x 32 columns, perfectly coalesced
//   dword j of the load = column quad*4+j, k-values 8*row..8*row+7 (low nibbles k 0..3,
//   high nibbles k 4..7), so (dw & 0x0F0F0F0F) and ((dw>>4) & 0x0F0F0F0F) feed two v_dot4
//   against the lane's 8 activation codes with no shuffling.
//
// Activations.  The production kernel takes the raw fp32 row and quantizes, inside each
// wavefront, exactly the k-groups that wavefront is about to stream (same operations as
// FC_dynamic_quantize_x, hence the same int8 codes and scales; the raw group sum is a tree sum
// instead of the left-to-right one).  The activation loads are issued ahead of the weight loads
// and the quantization runs while the first weight blocks are still in flight; codes and scales
// go through a wave-private LDS slot to the lanes that need them.  A second kernel variant takes
// activations already quantized by llmops_FC_dynamic_quantize_x.
//
// Each lane keeps fp32 running sums for its 4 columns (x rows); per block it folds its int32
// partial dot product in as (d*dx)*acc, and the lanes on a block's first k8-row add m*gsum.
// The 8 row slots are summed at the end with lane exchanges, the NW waves through LDS, and the
// k-splits of a strip through a scratch buffer: the workgroup that arrives last at the strip's
// counter adds the splits in index order, so results do not depend on scheduling.
//
// Follows fc_Q4A (/root/reference/ops/op_fc.hpp:286-426) for the arithmetic; the int32 partial
// sums are exact, the fp32 accumulation order differs from the reference's kb-sequential chain
// (bounded well inside the 1e-3 contract).
#include "common.h"
#include "gemv_device.h"

#include <type_traits>

namespace llmops {

struct TileRange {
    int nb, s, t0, t1;
};

template <int G, int NW>
__device__ __forceinline__ TileRange tile_range(int Kg, int S, int steps_per_split, int wave) {
    constexpr int BPS = Step<G>::kBlocksPerStep;
    TileRange r;
    r.nb = blockIdx.x / S;
    r.s = blockIdx.x % S;
    const int T = (Kg + BPS - 1) / BPS;  // steps in a strip
    const int t_lo = r.s * steps_per_split;
    const int t_hi = min(T, t_lo + steps_per_split);
    const int per_wave = (t_hi - t_lo + NW - 1) / NW;
    r.t0 = min(t_hi, t_lo + wave * per_wave);
    r.t1 = min(t_hi, r.t0 + per_wave);
    return r;
}

// Sums of squares of a strip's outputs, one per 16 columns (16 adjacent threads hold them, zeros for
// padding); `part` = 2*strip + (which half).  The next FC's rmsnorm adds these partial sums instead of
// re-reading the whole row.
__device__ __forceinline__ void half_strip_sumsq(float out, bool mine, int tr, int part, int strips, float* __restrict__ sumsq_out) {
    float sq = out * out;
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) sq += __shfl_xor(sq, o, 64);
    if (mine && (threadIdx.x & 15) == 0) sumsq_out[(int64_t)tr * 2 * strips + part] = sq;
}

// Sum the lanes' running sums over row slots, waves and k-splits and store the strip's outputs.
template <int MT, int NW>
__device__ __forceinline__ void finish_strip(float f[MT][4], float (*red)[MT][kGroupN], unsigned* ticket_sh, int nb, int s,
                                             int S, int rows, int64_t N, float* __restrict__ y, float* part,
                                             unsigned* counters, const float* __restrict__ residual,
                                             float* __restrict__ sumsq_out = nullptr) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int quad = lane & 7, rs = lane >> 3;
    // sum the 8 row slots (lane bits 3..5)
#pragma unroll
    for (int r = 0; r < MT; r++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            float v = f[r][j];
            v += dpp<kRowRor8>(v);
            v += __shfl_xor(v, 16, 64);
            v += __shfl_xor(v, 32, 64);
            f[r][j] = v;
        }
    if (rs == 0) {
#pragma unroll
        for (int r = 0; r < MT; r++)
#pragma unroll
            for (int j = 0; j < 4; j++) red[wave][r][quad * 4 + j] = f[r][j];
    }
    __syncthreads();

    const int tr = threadIdx.x >> 5, tn = threadIdx.x & 31;  // (row, column) this thread finalises
    const bool mine = tr < MT && tr < rows;
    if (S == 1 && !mine && sumsq_out == nullptr) return;
    const int64_t n = (int64_t)nb * kGroupN + tn;
    const int64_t Np = (int64_t)gridDim.x / S * kGroupN;
    float v = 0.0f;
    if (mine) {
#pragma unroll
        for (int w = 0; w < NW; w++) v += red[w][tr][tn];
    }
    if (S == 1) {
        const float out = (mine && n < N) ? (residual ? v + residual[(int64_t)tr * N + n] : v) : 0.0f;
        if (mine && n < N) y[(int64_t)tr * N + n] = out;
        if (sumsq_out != nullptr) half_strip_sumsq(out, mine, tr, 2 * nb + (tn >> 4), (int)(gridDim.x / S), sumsq_out);
        return;
    }
    // Cross-workgroup hand-off without cache-wide fences: partial sums are written and read with
    // device-scope (write-through / cache-bypassing) accesses, and the arrival counter is a
    // device-scope atomic.  The explicit wait makes sure this workgroup's stores have been
    // acknowledged before thread 0 announces the arrival.  (A __threadfence() here makes every
    // workgroup write back and invalidate its whole L2 slice, which costs far more than the
    // kernel itself.)
    if (mine) __hip_atomic_store(&part[((int64_t)s * rows + tr) * Np + n], v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0)
        *ticket_sh = __hip_atomic_fetch_add(&counters[nb], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (*ticket_sh != (unsigned)(S - 1)) return;
    float out = 0.0f;
    if (mine && n < N) {
        float acc = 0.0f;
        for (int i = 0; i < S; i++)
            acc += __hip_atomic_load(&part[((int64_t)i * rows + tr) * Np + n], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        out = residual ? acc + residual[(int64_t)tr * N + n] : acc;
        y[(int64_t)tr * N + n] = out;
    }
    if (sumsq_out != nullptr) half_strip_sumsq(out, mine, tr, 2 * nb + (tn >> 4), (int)(gridDim.x / S), sumsq_out);
    if (threadIdx.x == 0) __hip_atomic_store(&counters[nb], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // next launch
}

// The same for a workgroup that owns 16 of the strip's 32 columns over all of K (lane = row slot*4 + quad).
template <int MT, int NW>
__device__ __forceinline__ void finish_half_strip(float f[MT][4], float (*red)[MT][kGroupN], int nb, int half, int strips,
                                                  int rows, int64_t N, float* __restrict__ y,
                                                  const float* __restrict__ residual, float* __restrict__ sumsq_out) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // sum the 16 row slots (lane bits 2..5)
#pragma unroll
    for (int r = 0; r < MT; r++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            float v = f[r][j];
            v += dpp<kRowRor8>(v);
            v += dpp<kRowRor4>(v);
            v += __shfl_xor(v, 16, 64);
            v += __shfl_xor(v, 32, 64);
            f[r][j] = v;
        }
    if (lane < 4) {
#pragma unroll
        for (int r = 0; r < MT; r++)
#pragma unroll
            for (int j = 0; j < 4; j++) red[wave][r][lane * 4 + j] = f[r][j];
    }
    __syncthreads();
    const int tr = threadIdx.x >> 4, tn = threadIdx.x & 15;  // (row, column of the half) this thread finalises
    const bool mine = tr < MT && tr < rows;
    if (!mine && sumsq_out == nullptr) return;
    const int64_t n = (int64_t)nb * kGroupN + half * 16 + tn;
    float v = 0.0f;
    if (mine) {
#pragma unroll
        for (int w = 0; w < NW; w++) v += red[w][tr][tn];
    }
    const float out = (mine && n < N) ? (residual ? v + residual[(int64_t)tr * N + n] : v) : 0.0f;
    if (mine && n < N) y[(int64_t)tr * N + n] = out;
    if (sumsq_out != nullptr) half_strip_sumsq(out, mine, tr, 2 * nb + half, strips, sumsq_out);
}

// ---- variant 1: activations already quantized (xq, xd, gs in global memory) -------------------
template <int G, int MT, int NW>
__global__ __launch_bounds__(NW * 64) void fc_gemv_kernel(const uint8_t* __restrict__ weiq, const int8_t* __restrict__ xq,
                                                           const float* __restrict__ xd, const float* __restrict__ gs,
                                                           float* __restrict__ y, float* part, unsigned* counters, int Kg,
                                                           int64_t N, int rows, int S, int steps_per_split,
                                                           const float* __restrict__ residual) {
    __shared__ float red[NW][MT][kGroupN];
    __shared__ unsigned ticket_sh;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int rs = lane >> 3;
    const TileRange tr = tile_range<G, NW>(Kg, S, steps_per_split, wave);
    const uint8_t* strip = weiq + (int64_t)tr.nb * Kg * block_bytes(G);
    const int64_t Kp = (int64_t)Kg * G;  // padded K of the activation codes

    float f[MT][4];
#pragma unroll
    for (int r = 0; r < MT; r++)
#pragma unroll
        for (int j = 0; j < 4; j++) f[r][j] = 0.0f;

    Step<G> cur, nxt;
    if (tr.t0 < tr.t1) load_step<G>(cur, strip, tr.t0, Kg, lane);
    for (int t = tr.t0; t < tr.t1; t++) {
        if (t + 1 < tr.t1) load_step<G>(nxt, strip, t + 1, Kg, lane);
        const int kb = (G == 128) ? t : t * 2 + (rs >> 2);  // block whose scales this lane applies
        const bool first_row = (G == 128) ? (rs == 0) : ((rs & 3) == 0);
        if (cur.valid) {
#pragma unroll
            for (int r = 0; r < MT; r++) {
                if (r < rows) {
                    int acc[4];
                    dot_step<G>(cur, xq + r * Kp + (int64_t)t * Step<G>::kK, lane, acc);
                    const float dx = xd[(int64_t)r * Kg + kb];
                    const float g = first_row ? gs[(int64_t)r * Kg + kb] : 0.0f;
                    fold(f[r], acc, cur.dh, cur.mh, dx, g);
                }
            }
        }
        cur = nxt;
    }
    finish_strip<MT, NW>(f, red, &ticket_sh, tr.nb, tr.s, S, rows, N, y, part, counters, residual);
}

// ---- variant 2: raw fp32 activations, quantized by the wavefront that consumes them -----------
// Optional work folded into the decode kernel (MODE bits):
//   kNorm: the activation row is rmsnorm'ed first (ops/op_misc.hpp:142-181): every workgroup reads
//          the whole row once (L2 resident), reduces the sum of squares and scales the groups it
//          quantizes by rsqrt(mean+eps)*w.  Replaces clone + rmsnorm launches in front of the FC.
//   kGlu : the packed tensor holds gate and up strips interleaved (strip 2i = gate strip i, strip
//          2i+1 = up strip i); a workgroup computes both and stores silu(gate)*up
//          (itrans "silu" + imul, ops/op_misc.hpp:83-138).  Replaces two launches behind the FC.
//   kSums: with kNorm, the sum of squares of the row comes as per-strip partial sums left behind by
//          the FC that produced the row; every wave adds them up by itself (no pass over the row, no
//          workgroup barrier).
//   kGluIn: the activation row is a gate|up row of 2K floats (gate in [0,K), up in [K,2K)) and the
//          FC's input is silu(gate)*up, formed as the two halves are loaded.  The FC that produces
//          the row then keeps one strip per workgroup (no pairing of gate and up strips), which
//          spreads its strips more evenly over the compute units.
//   kHalf: (group 128) a workgroup owns 16 of a strip's 32 columns over all of K: twice the workgroups
//          without a hand-off between them, for tensors with fewer strips than the chip has compute
//          units.  Workgroups b and b+8 share a strip; workgroups are dealt to the 8 XCDs in turn, so
//          the two halves of every 128-byte row are served from the same L2 (a matter of speed only).
constexpr int kNorm = 1, kGlu = 2, kSums = 4, kGluIn = 8, kHalf = 16;

// One activation row needs few registers; asking for eight waves per SIMD (two workgroups of 16 waves
// per CU) keeps every variant at or below 64 registers, so that grids of 257..512 workgroups are
// resident at once.  (The second launch-bound argument counts waves per SIMD.)
//
// The kernel is bound by vector-ALU issue as much as by memory (a wave64 instruction occupies its SIMD
// for 4 cycles; at ~130-200 instructions per 2 KB block a CU streams 20-30 GB/s), so the loop is written
// for instruction count: at group 128 a wave quantizes the activations of two blocks with one pass of all
// 64 lanes (lanes 0-31 the first block's group, lanes 32-63 the second's) and the two weight buffers
// alternate without register copies.
template <int G, int MT, int NW, int MODE>
__global__ __launch_bounds__(NW * 64, (MT == 1 ? NW / 2 : 1)) void fc_gemv_fused_kernel(const uint8_t* __restrict__ weiq, const float* __restrict__ x,
                                                                 float* __restrict__ y, float* part, unsigned* counters,
                                                                 int Kg, int64_t K, int64_t N, int rows, int S,
                                                                 int steps_per_split, const float* __restrict__ residual,
                                                                 const float* __restrict__ norm_w, float eps,
                                                                 const float* __restrict__ sumsq_in, int sumsq_parts,
                                                                 float* __restrict__ sumsq_out) {
    constexpr bool NORM = (MODE & kNorm) != 0, GLU = (MODE & kGlu) != 0, SUMS = (MODE & kSums) != 0;
    constexpr bool GLUIN = (MODE & kGluIn) != 0, HALF = (MODE & kHalf) != 0;
    static_assert(!(GLUIN && NORM), "the gate|up input has no rmsnorm");
    static_assert(!HALF || (G == 128 && !GLU), "half strips: group 128, no gate/up epilogue");
    const int64_t xstride = GLUIN ? 2 * K : K;  // floats between activation rows
    constexpr int NWS = GLU ? NW / 2 : NW;  // waves per strip
    __shared__ float red[NW][MT][kGroupN];
    using Slot = typename std::conditional<G == 128, XPairSlot, XSlot<G>>::type;  // a pair of blocks / a step of two
    __shared__ __align__(16) Slot xs[NW][MT];
    __shared__ float nred[NORM ? NW : 1][MT];
    __shared__ unsigned ticket_sh;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int rs = HALF ? lane >> 2 : lane >> 3;
    TileRange tr;
    int half = 0;
    if (HALF) {  // S == 1: 16 consecutive workgroup ids = both halves of 8 strips
        const int b = blockIdx.x;
        const int per_wave = (Kg + NW - 1) / NW;
        tr.nb = ((b >> 4) << 3) | (b & 7);
        half = (b >> 3) & 1;
        tr.s = 0;
        tr.t0 = min(Kg, wave * per_wave);
        tr.t1 = min(Kg, tr.t0 + per_wave);
    } else if (GLU) {  // S == 1: blockIdx.x is the strip pair, each half of the workgroup owns one strip
        constexpr int BPS = Step<G>::kBlocksPerStep;
        const int T = (Kg + BPS - 1) / BPS;
        const int per_wave = (T + NWS - 1) / NWS;
        tr.nb = blockIdx.x * 2 + wave / NWS;
        tr.s = 0;
        tr.t0 = min(T, (wave % NWS) * per_wave);
        tr.t1 = min(T, tr.t0 + per_wave);
    } else {
        tr = tile_range<G, NW>(Kg, S, steps_per_split, wave);
    }
    const uint8_t* strip = weiq + (int64_t)tr.nb * Kg * block_bytes(G);
    const bool first_row = (G == 128) ? (rs == 0) : ((rs & 3) == 0);

    float f[MT][4];
#pragma unroll
    for (int r = 0; r < MT; r++)
#pragma unroll
        for (int j = 0; j < 4; j++) f[r][j] = 0.0f;

    // The loads return in issue order, so everything the rmsnorm statistic needs is requested
    // before the first weight block: the statistic is then computed while that block is in flight.
    constexpr int NV = (NORM && !SUMS) ? 4 : 1;  // float4 per thread held for the statistic (covers K <= NV*4*threads)
    float4 nv[NORM ? MT : 1][NV];
    // SUMS: this lane's share of the handed-over partial sums: four loads per row in flight together.
    // They are only added up after the first weight loads have been issued (below): using them here
    // would make the wave wait for them before it asks for anything else.
    float p4[(NORM && SUMS) ? MT : 1][4];
    if (NORM && SUMS) {
#pragma unroll
        for (int r = 0; r < MT; r++)
#pragma unroll
            for (int u = 0; u < 4; u++)
                p4[(NORM && SUMS) ? r : 0][u] =
                    (r < rows && lane + 64 * u < sumsq_parts) ? sumsq_in[(int64_t)r * sumsq_parts + lane + 64 * u] : 0.0f;
    } else if (NORM) {
#pragma unroll
        for (int r = 0; r < MT; r++)
#pragma unroll
            for (int i = 0; i < NV; i++) {
                const int64_t e = ((int64_t)i * NW * 64 + threadIdx.x) * 4;
                nv[NORM ? r : 0][i] = (r < rows && e < K) ? *reinterpret_cast<const float4*>(x + (int64_t)r * K + e)
                                                         : make_float4(0.f, 0.f, 0.f, 0.f);
            }
    }
    // two weight blocks in flight per wave, each with its activations (and norm weights):
    //   group 32 : cur/nxt, one step (two blocks) each, the activations of a step fetched one step ahead
    //   group 128: sa/sb alternate; xv/uv/wv hold the activations of a pair of blocks, four per lane
    Step<G> cur, nxt;
    XRaw<G> xcur[MT], xnxt[MT], wcur, wnxt;
    XRaw<G> ucur[GLUIN ? MT : 1], unxt[GLUIN ? MT : 1];  // the up half of a gate|up row
    float4 xv[MT], uv[GLUIN ? MT : 1], wv;
    const int pair_h = lane >> 5;  // group 128: which block of the pair this lane's four activations belong to
    // the pair's 256 activations are contiguous: uniform base + lane*16 bytes
#define LLMOPS_LOAD_PAIR(TP)                                                                                     \
    do {                                                                                                         \
        const bool ok_ = (TP) + pair_h < tr.t1;                                                                  \
        const uint32_t lo_ = (uint32_t)lane * 4u;                                                                \
        _Pragma("unroll") for (int r = 0; r < MT; r++) {                                                         \
            const float* xr_ = x + (int64_t)r * xstride + (int64_t)(TP) * 128;                                   \
            const bool okr_ = ok_ && r < rows;                                                                   \
            xv[r] = okr_ ? *reinterpret_cast<const float4*>(xr_ + lo_) : make_float4(0.f, 0.f, 0.f, 0.f);        \
            if (GLUIN) uv[GLUIN ? r : 0] = okr_ ? *reinterpret_cast<const float4*>(xr_ + K + lo_) : make_float4(0.f, 0.f, 0.f, 0.f); \
        }                                                                                                        \
        if (NORM) wv = ok_ ? *reinterpret_cast<const float4*>(norm_w + (int64_t)(TP) * 128 + lo_) : make_float4(0.f, 0.f, 0.f, 0.f); \
    } while (0)
#define LLMOPS_LOAD_BLOCK(ST, T)                                              \
    do {                                                                      \
        if constexpr (HALF) load_half_step(ST, strip, (T), half, lane);       \
        else load_step<G>(ST, strip, (T), Kg, lane);                          \
    } while (0)
    if (tr.t0 < tr.t1) {
        if constexpr (G == 128) {
            LLMOPS_LOAD_PAIR(tr.t0);
            LLMOPS_LOAD_BLOCK(cur, tr.t0);
            if (tr.t0 + 1 < tr.t1) LLMOPS_LOAD_BLOCK(nxt, tr.t0 + 1);
        } else {
#pragma unroll
            for (int r = 0; r < MT; r++)
                if (r < rows) {
                    load_x<G>(xcur[r], x + (int64_t)r * xstride, tr.t0, K, lane);
                    if (GLUIN) load_x<G>(ucur[GLUIN ? r : 0], x + (int64_t)r * xstride + K, tr.t0, K, lane);
                }
            if (NORM) load_x<G>(wcur, norm_w, tr.t0, K, lane);
            load_step<G>(cur, strip, tr.t0, Kg, lane);
        }
    }

    float rsn[MT];
    if (NORM && SUMS) {
#pragma unroll
        for (int r = 0; r < MT; r++) {
            const int rr = (NORM && SUMS) ? r : 0;
            float a = (p4[rr][0] + p4[rr][1]) + (p4[rr][2] + p4[rr][3]);
            if (r < rows)
                for (int i = lane + 256; i < sumsq_parts; i += 64) a += sumsq_in[(int64_t)r * sumsq_parts + i];
            rsn[r] = 1.0f / sqrtf(wave_sum_dpp(a) / (float)K + eps);
        }
    } else if (NORM) {
#pragma unroll
        for (int r = 0; r < MT; r++) {
            float ss = 0.0f;
#pragma unroll
            for (int i = 0; i < NV; i++) {
                const float4 v = nv[NORM ? r : 0][i];
                ss = fmaf(v.x, v.x, ss);
                ss = fmaf(v.y, v.y, ss);
                ss = fmaf(v.z, v.z, ss);
                ss = fmaf(v.w, v.w, ss);
            }
            if (r < rows) {  // rows longer than the preloaded part
                for (int64_t e = ((int64_t)NV * NW * 64 + threadIdx.x) * 4; e < K; e += NW * 64 * 4) {
                    const float4 v = *reinterpret_cast<const float4*>(x + (int64_t)r * K + e);
                    ss = fmaf(v.x, v.x, ss);
                    ss = fmaf(v.y, v.y, ss);
                    ss = fmaf(v.z, v.z, ss);
                    ss = fmaf(v.w, v.w, ss);
                }
            }
            ss = wave_sum_dpp(ss);
            if (lane == 0) nred[NORM ? wave : 0][r] = ss;
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < MT; r++) {
            float tot = 0.0f;
#pragma unroll
            for (int w = 0; w < NW; w++) tot += nred[NORM ? w : 0][r];
            rsn[r] = 1.0f / sqrtf(tot / (float)K + eps);
        }
    }

    if constexpr (G == 128) {
#define LLMOPS_BLOCK(ST, J)                                                                           \
    _Pragma("unroll") for (int r = 0; r < MT; r++) if (r < rows) {                                    \
        const Slot* slot = &xs[wave][r];                                                              \
        int acc[4];                                                                                   \
        if constexpr (HALF) dot_half_step(ST, slot->codes + (J) * 128, lane, acc);                    \
        else dot_step<G>(ST, slot->codes + (J) * 128, lane, acc);                                     \
        const float2 sc = slot->scale[J];                                                             \
        fold(f[r], acc, ST.dh, ST.mh, sc.x, first_row ? sc.y : 0.0f);                                 \
    }
        for (int tp = tr.t0; tp < tr.t1; tp += 2) {
#pragma unroll
            for (int r = 0; r < MT; r++) {
                if (r < rows) {
                    float4 v = xv[r];
                    if (NORM) {
                        v.x = v.x * rsn[r] * wv.x;
                        v.y = v.y * rsn[r] * wv.y;
                        v.z = v.z * rsn[r] * wv.z;
                        v.w = v.w * rsn[r] * wv.w;
                    }
                    if (GLUIN) {  // silu(gate)*up, the arithmetic of silu_mul_kernel
                        const float4 u = uv[GLUIN ? r : 0];
                        v.x = u.x * (v.x * (1.0f / (1.0f + expf(-v.x))));
                        v.y = u.y * (v.y * (1.0f / (1.0f + expf(-v.y))));
                        v.z = u.z * (v.z * (1.0f / (1.0f + expf(-v.z))));
                        v.w = u.w * (v.w * (1.0f / (1.0f + expf(-v.w))));
                    }
                    quantize_pair(v, &xs[wave][r], lane);
                }
            }
            __builtin_amdgcn_wave_barrier();  // LDS writes stay ahead of the reads below
            LLMOPS_BLOCK(cur, 0)
            if (tp + 1 < tr.t1) {
                LLMOPS_BLOCK(nxt, 1)
            }
            __builtin_amdgcn_wave_barrier();  // reads stay ahead of the next pair's writes
            // Most shapes give a wave one pair; a longer run asks for the next pair only now, which keeps
            // the registers of the pair in flight and of the pair in use from overlapping (64 in all).
            if (tp + 2 < tr.t1) {
                LLMOPS_LOAD_PAIR(tp + 2);
                LLMOPS_LOAD_BLOCK(cur, tp + 2);
                if (tp + 3 < tr.t1) LLMOPS_LOAD_BLOCK(nxt, tp + 3);
            }
        }
#undef LLMOPS_BLOCK
    } else {
        for (int t = tr.t0; t < tr.t1; t++) {
            if (t + 1 < tr.t1) {
                load_step<G>(nxt, strip, t + 1, Kg, lane);
#pragma unroll
                for (int r = 0; r < MT; r++)
                    if (r < rows) {
                        load_x<G>(xnxt[r], x + (int64_t)r * xstride, t + 1, K, lane);
                        if (GLUIN) load_x<G>(unxt[GLUIN ? r : 0], x + (int64_t)r * xstride + K, t + 1, K, lane);
                    }
                if (NORM) load_x<G>(wnxt, norm_w, t + 1, K, lane);
            }
#pragma unroll
            for (int r = 0; r < MT; r++) {
                if (r < rows) {
                    if (NORM) xcur[r].v[0] = xcur[r].v[0] * rsn[r] * wcur.v[0];
                    if (GLUIN) {  // silu(gate)*up, the arithmetic of silu_mul_kernel
                        const float g = xcur[r].v[0];
                        xcur[r].v[0] = ucur[GLUIN ? r : 0].v[0] * (g * (1.0f / (1.0f + expf(-g))));
                    }
                    Slot* slot = &xs[wave][r];
                    quantize_step<G>(xcur[r], slot, lane);
                    __builtin_amdgcn_wave_barrier();  // LDS writes stay ahead of the reads below
                    if (cur.valid) {
                        int acc[4];
                        dot_step<G>(cur, slot->codes, lane, acc);
                        const float2 sc = slot->scale[rs >> 2];
                        fold(f[r], acc, cur.dh, cur.mh, sc.x, first_row ? sc.y : 0.0f);
                    }
                    __builtin_amdgcn_wave_barrier();  // reads stay ahead of the next step's writes
                }
            }
            cur = nxt;
#pragma unroll
            for (int r = 0; r < MT; r++) xcur[r] = xnxt[r];
            if (GLUIN) {
#pragma unroll
                for (int r = 0; r < MT; r++) ucur[GLUIN ? r : 0] = unxt[GLUIN ? r : 0];
            }
            if (NORM) wcur = wnxt;
        }
    }
#undef LLMOPS_LOAD_PAIR
#undef LLMOPS_LOAD_BLOCK

    if (HALF) {
        finish_half_strip<MT, NW>(f, red, tr.nb, half, (int)(gridDim.x / 2), rows, N, y, residual, sumsq_out);
        return;
    }
    if (!GLU) {
        finish_strip<MT, NW>(f, red, &ticket_sh, tr.nb, tr.s, S, rows, N, y, part, counters, residual, sumsq_out);
        return;
    }
    // gate/up epilogue: sum row slots, then the two halves of the workgroup, then silu(gate)*up
    const int quad = lane & 7;
#pragma unroll
    for (int r = 0; r < MT; r++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            float v = f[r][j];
            v += dpp<kRowRor8>(v);
            v += __shfl_xor(v, 16, 64);
            v += __shfl_xor(v, 32, 64);
            f[r][j] = v;
        }
    if (rs == 0) {
#pragma unroll
        for (int r = 0; r < MT; r++)
#pragma unroll
            for (int j = 0; j < 4; j++) red[wave][r][quad * 4 + j] = f[r][j];
    }
    __syncthreads();
    const int trow = threadIdx.x >> 5, tn = threadIdx.x & 31;
    if (trow < MT && trow < rows) {
        float g = 0.0f, u = 0.0f;
#pragma unroll
        for (int w = 0; w < NWS; w++) {
            g += red[w][trow][tn];
            u += red[GLU ? w + NWS : w][trow][tn];
        }
        const int64_t n = (int64_t)blockIdx.x * kGroupN + tn;  // N = number of output columns (F)
        if (n < N) y[(int64_t)trow * N + n] = u * (g * (1.0f / (1.0f + expf(-g))));
    }
}

// Integer core only: acc[r][n][kb] (int32).  One wavefront per step, same loads and same dot
// code as the streaming kernels; the row slots of a block are summed with xor-shuffles.
template <int G>
__global__ __launch_bounds__(64) void fc_gemv_partials_kernel(const uint8_t* __restrict__ weiq,
                                                               const int8_t* __restrict__ xq, int32_t* __restrict__ out,
                                                               int Kg, int rows) {
    constexpr int BPS = Step<G>::kBlocksPerStep;
    const int lane = threadIdx.x;
    const int quad = lane & 7, rs = lane >> 3;
    const int T = (Kg + BPS - 1) / BPS;
    const int nb = blockIdx.x / T, t = blockIdx.x % T;
    const uint8_t* strip = weiq + (int64_t)nb * Kg * block_bytes(G);
    const int64_t Kp = (int64_t)Kg * G;
    const int64_t Np = (int64_t)(gridDim.x / T) * kGroupN;
    Step<G> st;
    load_step<G>(st, strip, t, Kg, lane);
    for (int r = 0; r < rows; r++) {
        int acc[4] = {0, 0, 0, 0};
        if (st.valid) dot_step<G>(st, xq + r * Kp + (int64_t)t * Step<G>::kK, lane, acc);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            int v = acc[j];
            v += __shfl_xor(v, 8, 64);
            v += __shfl_xor(v, 16, 64);
            if (G == 128) v += __shfl_xor(v, 32, 64);
            acc[j] = v;
        }
        const bool writer = (G == 128) ? (rs == 0) : ((rs & 3) == 0);
        const int kb = (G == 128) ? t : t * 2 + (rs >> 2);
        if (writer && st.valid) {
#pragma unroll
            for (int j = 0; j < 4; j++) out[((int64_t)r * Np + nb * kGroupN + quad * 4 + j) * Kg + kb] = acc[j];
        }
    }
}

static int g_target_workgroups = 256;  // split-K planner aims for this many workgroups
static int g_waves_per_workgroup = 0;  // 0 = choose per shape (pre-quantized variant only)

static int g_half_strips = 1;  // 0: never split strips into column halves

struct GemvPlan {
    int S, steps_per_split, NW;
    bool half;  // two workgroups per strip, 16 columns each, no split-K
};

static GemvPlan plan_gemv(int64_t rows, int64_t Ng, int64_t Kg, int G, bool fused) {
    const int bps = (G == 128) ? 1 : 2;
    const int T = (int)((Kg + bps - 1) / bps);
    int NW = fused ? 0 : g_waves_per_workgroup;
    if (NW == 0) NW = 16;
    if (rows > 4 && NW > 8) NW = 8;  // one (row, column) finaliser thread per output of the strip
    int S = (int)((g_target_workgroups + Ng - 1) / Ng);
    if ((T + NW - 1) / NW <= 2) S = 1;    // a wave already has only 1-2 blocks: splitting buys nothing
    const int max_s = (T + NW - 1) / NW;  // at least one step per wave
    if (S > max_s) S = max_s;
    if (S < 1) S = 1;
    int sps = (T + S - 1) / S;
    S = (T + sps - 1) / sps;  // drop empty splits
    return {S, sps, NW, false};
}

size_t gemv_workspace_bytes(int64_t rows, int64_t Ng, int64_t Kg, int G) {
    // upper bound over every plan the tuning knobs can produce: S never exceeds the step count
    const int bps = (G == 128) ? 1 : 2;
    const int64_t T = (Kg + bps - 1) / bps;
    int64_t S = (4096 + Ng - 1) / Ng;
    if (S > T) S = T;
    return (size_t)S * rows * Ng * kGroupN * sizeof(float);
}

struct FusedOps {
    const float* residual;  // y += residual
    const float* norm_w;    // x = rmsnorm(x, norm_w, eps) first
    float eps;
    bool glu;               // interleaved gate/up strips, y = silu(gate)*up
    bool glu_in;            // x is a gate|up row of 2K floats, the input is silu(gate)*up
    const float* sumsq_in;  // per-part sums of squares of x (instead of reading the row for the rmsnorm)
    int sumsq_parts;
    float* sumsq_out;       // per-strip sums of squares of y [rows, Ng]
};

template <int G, int MT, int NW>
static void launch_fused_t(const uint8_t* w, const float* x, float* y, float* part, unsigned* counters, int64_t Ng,
                           int64_t Kg, int64_t N, int rows, GemvPlan p, const FusedOps& o, hipStream_t st) {
    const int64_t K = Kg * G;
#define LLMOPS_FUSED(MODE, GRID)                                                                                      \
    fc_gemv_fused_kernel<G, MT, NW, MODE><<<(unsigned)(GRID), NW * 64, 0, st>>>(                                      \
        w, x, y, part, counters, (int)Kg, K, N, rows, p.S, p.steps_per_split, o.residual, o.norm_w, o.eps, o.sumsq_in, \
        o.sumsq_parts, o.sumsq_out)
    const bool sums = o.norm_w != nullptr && o.sumsq_in != nullptr;
    if constexpr (G == 128) {
        if (p.half) {
            if (o.glu_in) LLMOPS_FUSED(kGluIn | kHalf, Ng * 2);
            else if (sums) LLMOPS_FUSED(kNorm | kSums | kHalf, Ng * 2);
            else if (o.norm_w) LLMOPS_FUSED(kNorm | kHalf, Ng * 2);
            else LLMOPS_FUSED(kHalf, Ng * 2);
            return;
        }
    }
    if (o.glu_in) {
        LLMOPS_FUSED(kGluIn, Ng * p.S);
    } else if (o.glu) {
        if (sums) LLMOPS_FUSED(kNorm | kGlu | kSums, Ng / 2);
        else if (o.norm_w) LLMOPS_FUSED(kNorm | kGlu, Ng / 2);
        else LLMOPS_FUSED(kGlu, Ng / 2);
    } else {
        if (sums) LLMOPS_FUSED(kNorm | kSums, Ng * p.S);
        else if (o.norm_w) LLMOPS_FUSED(kNorm, Ng * p.S);
        else LLMOPS_FUSED(0, Ng * p.S);
    }
#undef LLMOPS_FUSED
}

// raw fp32 activations, quantized inside the kernel (+ optional rmsnorm / residual / gate-up epilogue)
int launch_gemv_fused(const uint8_t* w, const float* x, float* y, float* part, unsigned* counters, int64_t rows, int64_t Ng,
                      int64_t Kg, int G, int64_t N, const float* residual, const float* norm_w, float eps, int glu,
                      const float* sumsq_in, int sumsq_parts, float* sumsq_out, hipStream_t st) {
    GemvPlan p = plan_gemv(rows, Ng, Kg, G, true);
    if (glu == 1) p.S = 1;
    // Tensors with fewer strips than compute units and a K that gives a wave one pair of blocks: column
    // halves give every unit a workgroup without the split-K hand-off (4096x4096: 4.8 against 5.2 us).  With
    // a longer K the second quantization of every activation group costs what the hand-off does (4096x11008:
    // 9.4 against 9.1 us), so those keep split-K.
    if (g_half_strips && G == 128 && glu != 1 && Ng % 8 == 0 && Ng >= 96 && Ng < 256 && Kg <= 2 * p.NW) {
        p.half = true;
        p.S = 1;
    }
    const FusedOps o{residual, norm_w, eps, glu == 1, glu == 2, sumsq_in, sumsq_parts, sumsq_out};
#define LLMOPS_CASE(GG, MT, NWW) launch_fused_t<GG, MT, NWW>(w, x, y, part, counters, Ng, Kg, N, (int)rows, p, o, st)
    if (G == 128) {
        if (rows == 1) LLMOPS_CASE(128, 1, 16);
        else if (rows == 2) LLMOPS_CASE(128, 2, 16);
        else if (rows <= 4) LLMOPS_CASE(128, 4, 16);
        else LLMOPS_CASE(128, 8, 8);
    } else {
        if (rows == 1) LLMOPS_CASE(32, 1, 16);
        else if (rows == 2) LLMOPS_CASE(32, 2, 16);
        else if (rows <= 4) LLMOPS_CASE(32, 4, 16);
        else LLMOPS_CASE(32, 8, 8);
    }
#undef LLMOPS_CASE
    LLMOPS_LAUNCH_CHECK();
    return LLMOPS_OK;
}

template <int G, int MT, int NW>
static void launch_gemv_t(const uint8_t* w, const int8_t* xq, const float* xd, const float* gs, float* y, float* part,
                          unsigned* counters, int64_t Ng, int64_t Kg, int64_t N, int rows, GemvPlan p, hipStream_t st) {
    fc_gemv_kernel<G, MT, NW><<<(unsigned)(Ng * p.S), NW * 64, 0, st>>>(w, xq, xd, gs, y, part, counters, (int)Kg, N, rows,
                                                                      p.S, p.steps_per_split, nullptr);
}

template <int G, int MT>
static void launch_gemv_nw(const uint8_t* w, const int8_t* xq, const float* xd, const float* gs, float* y, float* part,
                           unsigned* counters, int64_t Ng, int64_t Kg, int64_t N, int rows, GemvPlan p, hipStream_t st) {
    if (p.NW >= 16 && MT <= 4)
        launch_gemv_t<G, MT, (MT <= 4 ? 16 : 8)>(w, xq, xd, gs, y, part, counters, Ng, Kg, N, rows, p, st);
    else if (p.NW >= 8)
        launch_gemv_t<G, MT, 8>(w, xq, xd, gs, y, part, counters, Ng, Kg, N, rows, p, st);
    else
        launch_gemv_t<G, MT, 4>(w, xq, xd, gs, y, part, counters, Ng, Kg, N, rows, p, st);
}

// activations already quantized by llmops_FC_dynamic_quantize_x
int launch_gemv(const uint8_t* w, const int8_t* xq, const float* xd, const float* gs, float* y, float* part,
                unsigned* counters, int64_t rows, int64_t Ng, int64_t Kg, int G, int64_t N, hipStream_t st) {
    const GemvPlan p = plan_gemv(rows, Ng, Kg, G, false);
#define LLMOPS_GEMV_CASE(GG, MT) launch_gemv_nw<GG, MT>(w, xq, xd, gs, y, part, counters, Ng, Kg, N, (int)rows, p, st)
    if (G == 128) {
        if (rows == 1) LLMOPS_GEMV_CASE(128, 1);
        else if (rows == 2) LLMOPS_GEMV_CASE(128, 2);
        else if (rows <= 4) LLMOPS_GEMV_CASE(128, 4);
        else LLMOPS_GEMV_CASE(128, 8);
    } else {
        if (rows == 1) LLMOPS_GEMV_CASE(32, 1);
        else if (rows == 2) LLMOPS_GEMV_CASE(32, 2);
        else if (rows <= 4) LLMOPS_GEMV_CASE(32, 4);
        else LLMOPS_GEMV_CASE(32, 8);
    }
#undef LLMOPS_GEMV_CASE
    LLMOPS_LAUNCH_CHECK();
    return LLMOPS_OK;
}

int launch_gemv_partials(const uint8_t* w, const int8_t* xq, int32_t* acc, int64_t rows, int64_t Ng, int64_t Kg, int G,
                         hipStream_t st) {
    const int bps = (G == 128) ? 1 : 2;
    const int64_t T = (Kg + bps - 1) / bps;
    if (G == 128)
        fc_gemv_partials_kernel<128><<<(unsigned)(Ng * T), 64, 0, st>>>(w, xq, acc, (int)Kg, (int)rows);
    else
        fc_gemv_partials_kernel<32><<<(unsigned)(Ng * T), 64, 0, st>>>(w, xq, acc, (int)Kg, (int)rows);
    LLMOPS_LAUNCH_CHECK();
    return LLMOPS_OK;
}

}  // namespace llmops

extern "C" void llmops_fc_set_half_strips(int on) { llmops::g_half_strips = on != 0; }

extern "C" void llmops_fc_set_tuning(int target_workgroups, int waves_per_workgroup) {
    if (target_workgroups > 0) llmops::g_target_workgroups = target_workgroups > 4096 ? 4096 : target_workgroups;
    if (waves_per_workgroup >= 0) llmops::g_waves_per_workgroup = waves_per_workgroup;
}

