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

template <int G, int NW, int PASS = 1>
__device__ __forceinline__ TileRange tile_range(int Kg, int S, int steps_per_split, int wave) {
    constexpr int BPS = Step<G>::kBlocksPerStep;
    TileRange r;
    if (S == 1) {  // no division for the common cases (a division is ~25 instructions in front of the first load)
        r.nb = blockIdx.x;
        r.s = 0;
    } else if (S == 2) {
        r.nb = blockIdx.x >> 1;
        r.s = blockIdx.x & 1;
    } else {
        r.nb = blockIdx.x / S;
        r.s = blockIdx.x % S;
    }
    const int T = (int)((unsigned)(Kg + BPS - 1) / BPS);  // steps in a strip
    const int t_lo = r.s * steps_per_split;
    const int t_hi = min(T, t_lo + steps_per_split);
    // (unsigned: every wave runs this before it can ask for its first byte, and a signed division by NW costs
    // three scalar instructions more)
    if constexpr (PASS == 1) {
        const int per_wave = (int)((unsigned)(t_hi - t_lo + NW - 1) / NW);
        r.t0 = min(t_hi, t_lo + wave * per_wave);
        r.t1 = min(t_hi, r.t0 + per_wave);
    } else {
        // The kernel that quantizes on the fly works in passes of PASS steps, and a pass costs its quantization
        // whether all of its steps are wanted or one: whole passes are dealt out, the first `rem` waves one more
        // than the others (43 blocks of a split: 22 passes = 6 waves with two and 10 with one, instead of 14 waves
        // with a full and a half-empty pass each).
        const unsigned np = (unsigned)(t_hi - t_lo + PASS - 1) / PASS;
        const unsigned q = np / NW, rem = np % NW;
        const unsigned first = (unsigned)wave * q + min((unsigned)wave, rem);
        const unsigned count = q + ((unsigned)wave < rem ? 1u : 0u);
        r.t0 = min(t_hi, t_lo + (int)(first * PASS));
        r.t1 = min(t_hi, r.t0 + (int)(count * PASS));
    }
    return r;
}

// Sum of squares of a strip's 32 outputs (threads tr*32 .. tr*32+31 hold them, zeros for padding):
// the next FC's rmsnorm adds these per-strip sums instead of re-reading the whole row.
__device__ __forceinline__ void strip_sumsq(float out, bool mine, int tr, int nb, int strips, float* __restrict__ sumsq_out) {
    float sq = out * out;
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) sq += __shfl_xor(sq, o, 64);
    if (mine && (lane_id_now() & 31) == 0) sumsq_out[(int64_t)tr * strips + nb] = sq;
}

// Sum the lanes' running sums over row slots, waves and k-splits and store the strip's outputs.
template <int MT, int NW>
__device__ __forceinline__ void finish_strip(float f[MT][4], float (*red)[MT][kGroupN], unsigned* ticket_sh, int wave, int nb, int s,
                                             int S, int rows, int64_t N, float* __restrict__ y, float* part,
                                             unsigned* counters, bool has_residual, float residual_value,
                                             float* __restrict__ sumsq_out = nullptr, unsigned long long* slots = nullptr) {
    const int lane = lane_id_now(), tid = wave * 64 + lane;  // `wave` is uniform (a scalar register)
    const int quad = lane & 7, rs = lane >> 3;
    // sum the 8 row slots (lane bits 3..5)
#pragma unroll
    for (int r = 0; r < MT; r++) rowslot_sum4(f[r]);
    if (rs == 0) {
#pragma unroll
        for (int r = 0; r < MT; r++)
#pragma unroll
            for (int j = 0; j < 4; j++) red[wave][r][quad * 4 + j] = f[r][j];
    }
    __syncthreads();

    const int tr = tid >> 5, tn = tid & 31;  // (row, column) this thread finalises
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
        const float out = (mine && n < N) ? (has_residual ? v + residual_value : v) : 0.0f;
        if (mine && n < N) y[(int64_t)tr * N + n] = out;
        if (sumsq_out != nullptr) strip_sumsq(out, mine, tr, nb, (int)(gridDim.x / S), sumsq_out);
        return;
    }
    // Two k-splits: the hand-off is one 64-bit exchange per output.  A slot is empty (0) or holds (1 << 32 | value bits); whoever finds the other split's
    // value there adds the two (a + b: the same bits whichever came first), stores the output and empties
    // the slot for the next launch; whoever finds it empty has parked its own value and is done.  The value
    // travels inside the atomic, so there is nothing to order, and the cost is one round trip to memory
    // instead of three (store and acknowledgement, ticket, loads).
    if (slots != nullptr) {
        float done = 0.0f;  // the finished output if this thread is the one that finished it, else 0
        if (mine && n < N) {
            unsigned long long* slot = slots + ((int64_t)tr * Np + n);
            const unsigned long long parked = (1ull << 32) | (unsigned long long)__float_as_uint(v);
            const unsigned long long old = __hip_atomic_exchange(slot, parked, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if ((old >> 32) != 0ull) {
                const float both = v + __uint_as_float((unsigned)(old & 0xFFFFFFFFull));
                done = has_residual ? both + residual_value : both;
                y[(int64_t)tr * N + n] = done;
                __hip_atomic_store(slot, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        if (sumsq_out == nullptr) return;
        // The strip's sum of squares: each of the two workgroups knows the squares of the outputs it finished;
        // the two partial sums meet through one more exchange per (row, strip), in slots behind the outputs'
        // (p0 + p1: the same bits whichever came first).
        float sq = done * done;
#pragma unroll
        for (int o = 16; o > 0; o >>= 1) sq += __shfl_xor(sq, o, 64);
        if (mine && (lane_id_now() & 31) == 0) {
            const int64_t strips = (int64_t)gridDim.x / S;
            unsigned long long* slot = slots + (int64_t)rows * Np + ((int64_t)tr * strips + nb);
            const unsigned long long parked = (1ull << 32) | (unsigned long long)__float_as_uint(sq);
            const unsigned long long old = __hip_atomic_exchange(slot, parked, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if ((old >> 32) != 0ull) {
                sumsq_out[(int64_t)tr * strips + nb] = sq + __uint_as_float((unsigned)(old & 0xFFFFFFFFull));
                __hip_atomic_store(slot, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
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
    if (tid == 0)
        *ticket_sh = __hip_atomic_fetch_add(&counters[nb], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (*ticket_sh != (unsigned)(S - 1)) return;
    float out = 0.0f;
    if (mine && n < N) {
        float acc = 0.0f;
        for (int i = 0; i < S; i++)
            acc += __hip_atomic_load(&part[((int64_t)i * rows + tr) * Np + n], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        out = has_residual ? acc + residual_value : acc;
        y[(int64_t)tr * N + n] = out;
    }
    if (sumsq_out != nullptr) strip_sumsq(out, mine, tr, nb, (int)(gridDim.x / S), sumsq_out);
    if (tid == 0) __hip_atomic_store(&counters[nb], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // next launch
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
    finish_strip<MT, NW>(f, red, &ticket_sh, wave, tr.nb, tr.s, S, rows, N, y, part, counters, false, 0.0f);
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
//   kDump: test build of the loop: besides the outputs it stores what it quantized (codes, scales, raw
//          group sums of every pass) and the int32 dot product of every (row, column, k-group), so that the
//          kernel's own quantizer and integer core can be compared bit for bit with the reference's
//          (llmops_test_fc_decode_dump).  Every workgroup stores the activations it quantized: all of them
//          must agree.
//   kAttnIn: the activation row is the output of decode attention, not yet merged: per head up to
//          kAttnRecChunks chunk records (max, sum, weighted V sum over the chunk's cache rows) as
//          llmops_attention_rope_decode_records leaves them.  A lane needs four consecutive elements of one head:
//          it fetches the head's statistics and its 16 bytes of every record, forms the chunk weights
//          exp(m_c - M) and the merged, normalised output -- the work of attn_merge_kernel -- and quantizes that.
//          One row only (group 128).  Saves the merge launch between attention and the o projection.
constexpr int kNorm = 1, kGlu = 2, kSums = 4, kGluIn = 8, kDump = 16, kAttnIn = 32;
constexpr int kAttnRecChunks = 8;  // as in attn.hip
struct AttnRecs {
    const float* stats;  // [rows*H][kAttnRecChunks][2]
    const float* outs;   // [rows*H][kAttnRecChunks][128]
    int chunks;          // records per head that were written (<= kAttnRecChunks)
};


// The lane's four elements of the attention output from the chunk records of its head: weights exp(m_c - M)
// over the chunks that hold rows (sum > 0), out = sum_c w_c o_c / sum_c w_c s_c (the arithmetic of
// attn_merge_kernel).  st[c/2] holds (m, s) of chunks c and c+1; a record that was not asked for reads as zeros.
__device__ __forceinline__ float4 merge_attn_records(const float4 (&ro)[kAttnRecChunks], const float4 (&st)[kAttnRecChunks / 2],
                                                     int chunks) {
    float m[kAttnRecChunks], sm[kAttnRecChunks];
#pragma unroll
    for (int c = 0; c < kAttnRecChunks / 2; c++) {  // (the statistics come in pairs: the second of the last pair may not exist)
        m[2 * c] = st[c].x, sm[2 * c] = st[c].y;
        m[2 * c + 1] = st[c].z, sm[2 * c + 1] = (2 * c + 1 < chunks) ? st[c].w : 0.0f;
    }
    float M = -3.402823466e+38f;
#pragma unroll
    for (int c = 0; c < kAttnRecChunks; c++) M = fmaxf(M, sm[c] == 0.0f ? -3.402823466e+38f : m[c]);
    float den = 0.0f;
    float4 num = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int c = 0; c < kAttnRecChunks; c++) {
        const float w = (sm[c] == 0.0f) ? 0.0f : expf(m[c] - M);
        den = fmaf(w, sm[c], den);
        num.x = fmaf(w, ro[c].x, num.x);
        num.y = fmaf(w, ro[c].y, num.y);
        num.z = fmaf(w, ro[c].z, num.z);
        num.w = fmaf(w, ro[c].w, num.w);
    }
    const float inv = 1.0f / den;
    return make_float4(num.x * inv, num.y * inv, num.z * inv, num.w * inv);
}

// One activation row needs few registers; asking for eight waves per SIMD (two workgroups of 16 waves
// per CU) keeps every variant at or below 64 registers, so that grids of 257..512 workgroups are
// resident at once.  (The second launch-bound argument counts waves per SIMD.)
//
// The kernel is bound by vector-ALU issue as much as by memory (a wave64 instruction occupies its SIMD
// for 4 cycles; at ~130-200 instructions per 2 KB block a CU streams 20-30 GB/s), so the loop is written
// for instruction count: a wave quantizes 256 activations with one pass of all 64 lanes (group 128: lanes
// 0-31 the first block's group, lanes 32-63 the second's; group 32: eight groups of 8 lanes) and uses the
// weight buffers of the pass in place, without register copies.
template <int G, int MT, int NW, int MODE>
__global__ __launch_bounds__(NW * 64, (MT == 1 ? ((MODE & kAttnIn) ? NW / 4 : NW / 2) : 1)) void fc_gemv_fused_kernel(const uint8_t* __restrict__ weiq, const float* __restrict__ x,
                                                                 int Kg, int S, int steps_per_split, int rows, int N, int sumsq_parts,
                                                                 const float* __restrict__ residual,
                                                                 const float* __restrict__ sumsq_in,
                                                                 const float* __restrict__ norm_w, float eps,
                                                                 float* __restrict__ y, float* part, unsigned* counters,
                                                                 float* __restrict__ sumsq_out, int exchange, const DumpBufs dump,
                                                                 const AttnRecs recs) {
    constexpr bool NORM = (MODE & kNorm) != 0, GLU = (MODE & kGlu) != 0, SUMS = (MODE & kSums) != 0;
    constexpr bool GLUIN = (MODE & kGluIn) != 0, DUMP = (MODE & kDump) != 0, ATTN = (MODE & kAttnIn) != 0;
    static_assert(!ATTN || (G == 128 && MT == 1 && !NORM && !GLU && !GLUIN), "chunk records: one row, group 128, plain input");
    static_assert(!(GLUIN && NORM), "the gate|up input has no rmsnorm");
    // (argument order: the first 14 dwords of a kernel's arguments arrive in scalar registers together with the
    // wave (the library is built with kernel-argument preload), so everything the first loads need -- tensor,
    // activations, the plan, the residual and the handed-over sums -- comes first: a wave then asks for its
    // data without a round trip to the argument buffer in front of it)
    const int64_t K = (int64_t)Kg * G;
    const int64_t xstride = GLUIN ? 2 * K : K;  // floats between activation rows
    constexpr int NWS = GLU ? NW / 2 : NW;  // waves per strip
    __shared__ float red[NW][MT][kGroupN];
    using Slot = XPairSlot;  // codes and scales of one pass (256 k-values)
    __shared__ __align__(16) Slot xs[NW][MT];
    __shared__ float nred[NORM ? NW : 1][MT];
    __shared__ unsigned ticket_sh;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int rs = lane >> 3;
    TileRange tr;
    if (GLU) {  // S == 1: blockIdx.x is the strip pair, each half of the workgroup owns one strip
        constexpr int BPS = Step<G>::kBlocksPerStep;
        const int T = (Kg + BPS - 1) / BPS;
        const int per_wave = (T + NWS - 1) / NWS;
        tr.nb = blockIdx.x * 2 + wave / NWS;
        tr.s = 0;
        tr.t0 = min(T, (wave % NWS) * per_wave);
        tr.t1 = min(T, tr.t0 + per_wave);
    } else {
        tr = tile_range<G, NW, (G == 128) ? 2 : 4>(Kg, S, steps_per_split, wave);  // passes of 256 k-values
    }
    // (a tensor has fewer than 2^32 blocks: one 32-bit product, then one widening multiplication)
    const uint8_t* strip = weiq + (uint64_t)((uint32_t)tr.nb * (uint32_t)Kg) * (uint32_t)block_bytes(G);
    const bool first_row = (G == 128) ? (rs == 0) : ((rs & 3) == 0);
    // The residual element this thread will add at the very end (thread = (row, column) of the strip) is
    // asked for now: at the end it would put a memory round trip behind the last barrier.  (With the
    // rmsnorm prologue the main loop has no register to spare; there it is asked for after the loop.)
    float resv = 0.0f;
#define LLMOPS_LOAD_RESIDUAL(TID)                                                          \
    if (!GLU && residual != nullptr) {                                                     \
        const int fr_ = (TID) >> 5;                                                        \
        const int64_t n_ = (int64_t)tr.nb * kGroupN + ((TID) & 31);                        \
        if (fr_ < MT && fr_ < rows && n_ < N) resv = residual[(int64_t)fr_ * N + n_];      \
    }
    if (!NORM) {
        LLMOPS_LOAD_RESIDUAL(threadIdx.x)
    }

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
    if (NORM && SUMS) {  // at most 256 parts (the launcher sees to it); what lies beyond a row's parts reads as 0
#pragma unroll
        for (int r = 0; r < MT; r++) {
            const buffer_rsrc ss_rs = make_rsrc(sumsq_in + (int64_t)r * sumsq_parts, r < rows ? (uint32_t)sumsq_parts * 4u : 0u);
#pragma unroll
            for (int u = 0; u < 4; u++) p4[(NORM && SUMS) ? r : 0][u] = buf_ldf1(ss_rs, (uint32_t)(lane + 64 * u) * 4u, 0u);
        }
        __builtin_amdgcn_sched_barrier(0);  // asked for first, used after everything else has been asked for
    }
    // A wave works in passes of 256 k-values: SPP steps (group 128: two blocks, one per step; group 32: four
    // steps of two blocks each) whose weights are in flight together with the pass's activations (and norm
    // weights), four per lane.  A wave's tile range is rounded to whole passes by its owner: steps
    // TP .. TP+SPP-1 of a pass that lie at or beyond t1 belong to nobody here and are not asked for.
    constexpr int SPP = (G == 128) ? 2 : 4;
    struct PairBuf {
        Step<G> s[SPP];
        float4 xv[MT], uv[GLUIN ? MT : 1], wv;
        float4 ro[ATTN ? kAttnRecChunks : 1], rs[ATTN ? kAttnRecChunks / 2 : 1];  // chunk records: outputs, (max, sum) pairs
    };
    PairBuf P0;
    const int lane_step = lane / (64 / SPP);  // which step of the pass this lane's four activations belong to
    // the pass's 256 activations are contiguous: uniform base + lane*16 bytes; activations are asked for
    // before the weights (loads return in issue order and the quantization comes first); all loads go
    // through buffer descriptors (scalar base + scalar block offset + lane offset)
    const buffer_rsrc strip_rs = make_rsrc(strip, (uint32_t)Kg * (uint32_t)block_bytes(G));
    const buffer_rsrc x_rs = make_rsrc(x, (uint32_t)rows * (uint32_t)xstride * 4u);
    const buffer_rsrc nw_rs = make_rsrc(NORM ? norm_w : x, NORM ? (uint32_t)K * 4u : 0u);
    // chunk records: K / 128 heads; a pass of 256 k-values covers two heads (lanes 0-31 the first, 32-63 the second)
    const buffer_rsrc ro_rs = make_rsrc(ATTN ? recs.outs : x, ATTN ? (uint32_t)(K / 128) * (uint32_t)(kAttnRecChunks * 128 * 4) : 0u);
    const buffer_rsrc rt_rs = make_rsrc(ATTN ? recs.stats : x, ATTN ? (uint32_t)(K / 128) * (uint32_t)(kAttnRecChunks * 2 * 4) : 0u);
    if constexpr (NORM && !SUMS) {
        // the row for the statistic, four floats per thread and slice of NW*256: asked for unconditionally (a
        // slice beyond K at an offset that returns 0) and first, so that the statistic waits for these only
#pragma unroll
        for (int r = 0; r < MT; r++)
#pragma unroll
            for (int i = 0; i < NV; i++) {
                const int64_t e = ((int64_t)i * NW * 64 + threadIdx.x) * 4;
                nv[NORM ? r : 0][i] = buf_ldf4(x_rs, (r < rows && e < K) ? (uint32_t)threadIdx.x * 16u : kNoLoad,
                                               (uint32_t)(r * K + (int64_t)i * NW * 256) * 4u);
            }
        __builtin_amdgcn_sched_barrier(0);
    }
#define LLMOPS_LOAD_PAIR(P, TP, WANT)                                                                            \
    do { /* branch-free: what is not wanted is asked for at an offset that returns 0 (see kNoLoad) */            \
        const bool ok_ = (WANT) && (TP) + lane_step < tr.t1 && (uint32_t)(TP) * Step<G>::kK + lane * 4 < (uint32_t)K; \
        const uint32_t so_ = (uint32_t)(TP) * (uint32_t)(Step<G>::kK * 4);                                       \
        if constexpr (ATTN) { /* head = (TP) + (lane >> 5): statistics first (the weights need them), then the outputs */ \
            const uint32_t hs_ = (uint32_t)(TP) * (uint32_t)(kAttnRecChunks * 2 * 4);                            \
            const uint32_t ho_ = (uint32_t)(TP) * (uint32_t)(kAttnRecChunks * 128 * 4);                          \
            _Pragma("unroll") for (int c_ = 0; c_ < kAttnRecChunks / 2; c_++)                                    \
                P.rs[ATTN ? c_ : 0] = buf_ldf4(rt_rs, (ok_ && 2 * c_ < recs.chunks) ? (uint32_t)(lane >> 5) * (uint32_t)(kAttnRecChunks * 8) + (uint32_t)c_ * 16u : kNoLoad, hs_); \
            _Pragma("unroll") for (int c_ = 0; c_ < kAttnRecChunks; c_++)                                        \
                P.ro[ATTN ? c_ : 0] = buf_ldf4(ro_rs, (ok_ && c_ < recs.chunks) ? (uint32_t)(lane >> 5) * (uint32_t)(kAttnRecChunks * 512) + (uint32_t)(lane & 31) * 16u + (uint32_t)c_ * 512u : kNoLoad, ho_); \
        } else {                                                                                                 \
        _Pragma("unroll") for (int r = 0; r < MT; r++) {                                                         \
            const uint32_t ro_ = so_ + (uint32_t)r * (uint32_t)xstride * 4u;                                     \
            const uint32_t lo_ = (ok_ && (MT == 1 || r < rows)) ? (uint32_t)lane * 16u : kNoLoad; /* MT == 1: one row */ \
            P.xv[r] = buf_ldf4(x_rs, lo_, ro_);                                                                  \
            if (GLUIN) P.uv[GLUIN ? r : 0] = buf_ldf4(x_rs, lo_, ro_ + (uint32_t)K * 4u);                        \
        }                                                                                                        \
        }                                                                                                        \
        if (NORM) P.wv = buf_ldf4(nw_rs, ok_ ? (uint32_t)lane * 16u : kNoLoad, so_);                             \
        __builtin_amdgcn_sched_barrier(0); /* the compiler's scheduler must not move the weights ahead */       \
        _Pragma("unroll") for (int i_ = 0; i_ < SPP; i_++) {                                                     \
            if constexpr (G == 128) load_step_buf(P.s[i_], strip_rs, (TP) + i_, lane, (WANT) && (TP) + i_ < tr.t1); \
            else load_step_buf(P.s[i_], strip_rs, (TP) + i_, Kg, lane, (WANT) && (TP) + i_ < tr.t1);             \
        }                                                                                                        \
        __builtin_amdgcn_sched_barrier(0);                                                                       \
    } while (0)
    // The first pass is asked for inside the region that uses it (below), so that loads, statistic and
    // loop stay in one block in this order; only the statistic that needs a workgroup barrier (rmsnorm
    // from the row) must run in every wave, and its loads are issued here.
    constexpr bool kBarrierStat = NORM && !SUMS;
    if constexpr (kBarrierStat) LLMOPS_LOAD_PAIR(P0, tr.t0, tr.t0 < tr.t1);

    float rsn[MT];
    // statistic from the handed-over sums; the empty statement the partial sums pass through keeps the
    // compiler from adding them up, and therefore waiting for them, before the loads issued after them
#define LLMOPS_SUMS_STAT                                                                                         \
    _Pragma("unroll") for (int r = 0; r < MT; r++) {                                                             \
        const int rr = (NORM && SUMS) ? r : 0;                                                                   \
        asm volatile("" : "+v"(p4[rr][0]), "+v"(p4[rr][1]), "+v"(p4[rr][2]), "+v"(p4[rr][3])::"memory");        \
        const float a = (p4[rr][0] + p4[rr][1]) + (p4[rr][2] + p4[rr][3]);                                       \
        rsn[r] = 1.0f / sqrtf(wave_sum_dpp(a) / (float)K + eps);                                                 \
    }
    if (NORM && SUMS) {
#pragma unroll
        for (int r = 0; r < MT; r++) rsn[r] = 0.0f;
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

#define LLMOPS_BLOCK(ST, J)                                                                           \
    _Pragma("unroll") for (int r = 0; r < MT; r++) if (r < rows) {                                    \
        const Slot* slot = &xs[wave][r];                                                              \
        int acc[4];                                                                                   \
        dot_step<G>(ST, slot->codes + (J) * Step<G>::kK, lane, acc);                                  \
        const float2 sc = slot->scale[(G == 128) ? (J) : (J) * 2 + (rs >> 2)];                        \
        fold(f[r], acc, ST.dh, ST.mh, sc.x, first_row ? sc.y : 0.0f);                                 \
        if constexpr (DUMP) { /* the block's sums over its k8-rows (lane bits 3.. of the block) */    \
            const int kb_ = (G == 128) ? tp_ + (J) : (tp_ + (J)) * 2 + (rs >> 2);                     \
            _Pragma("unroll") for (int j = 0; j < 4; j++) {                                           \
                int v_ = acc[j];                                                                      \
                v_ += __shfl_xor(v_, 8, 64);                                                          \
                v_ += __shfl_xor(v_, 16, 64);                                                         \
                if (G == 128) v_ += __shfl_xor(v_, 32, 64);                                           \
                if (first_row && kb_ < Kg)                                                            \
                    dump.acc[((int64_t)r * ((int64_t)gridDim.x / S * kGroupN) + tr.nb * kGroupN + (lane & 7) * 4 + j) * Kg + kb_] = v_; \
            }                                                                                         \
        }                                                                                             \
    }
#define LLMOPS_PAIR(P, TP)                                                                            \
    do {                                                                                              \
        const int tp_ = (TP);                                                                         \
        _Pragma("unroll") for (int r = 0; r < MT; r++) if (r < rows) {                                \
            float4 v = P.xv[r];                                                                       \
            if constexpr (ATTN) v = merge_attn_records(P.ro, P.rs, recs.chunks);                      \
            if (NORM) {                                                                               \
                v.x = v.x * rsn[r] * P.wv.x;                                                          \
                v.y = v.y * rsn[r] * P.wv.y;                                                          \
                v.z = v.z * rsn[r] * P.wv.z;                                                          \
                v.w = v.w * rsn[r] * P.wv.w;                                                          \
            }                                                                                         \
            if (GLUIN) { /* silu(gate)*up, the arithmetic of silu_mul_kernel */                       \
                const float4 u = P.uv[GLUIN ? r : 0];                                                 \
                v.x = silu_times(v.x, u.x);                                                           \
                v.y = silu_times(v.y, u.y);                                                           \
                v.z = silu_times(v.z, u.z);                                                           \
                v.w = silu_times(v.w, u.w);                                                           \
            }                                                                                         \
            if constexpr (G == 128) quantize_pair(v, &xs[wave][r], lane);                             \
            else quantize_pass32(v, &xs[wave][r], lane);                                              \
        }                                                                                             \
        __builtin_amdgcn_wave_barrier(); /* LDS writes stay ahead of the reads below */               \
        if constexpr (DUMP) {                                                                         \
            _Pragma("unroll") for (int r = 0; r < MT; r++) if (r < rows) {                            \
                const Slot* slot = &xs[wave][r];                                                      \
                const int64_t k_ = (int64_t)tp_ * Step<G>::kK + lane * 4;                             \
                if (tp_ + lane_step < tr.t1 && k_ < K)                                                \
                    *reinterpret_cast<uint32_t*>(dump.xq + (int64_t)r * Kg * G + k_) =                \
                        *reinterpret_cast<const uint32_t*>(&slot->codes[lane * 4]);                   \
                constexpr int kBlocksPerPass = 256 / G;                                               \
                const int kb_ = tp_ * Step<G>::kBlocksPerStep + lane;                                 \
                if (lane < kBlocksPerPass && tp_ + lane / Step<G>::kBlocksPerStep < tr.t1 && kb_ < Kg) { \
                    dump.xd[(int64_t)r * Kg + kb_] = slot->scale[lane].x;                             \
                    dump.gs[(int64_t)r * Kg + kb_] = slot->scale[lane].y;                             \
                }                                                                                     \
            }                                                                                         \
        }                                                                                             \
        LLMOPS_BLOCK(P.s[0], 0)                                                                       \
        _Pragma("unroll") for (int i_ = 1; i_ < SPP; i_++) {                                          \
            if ((TP) + i_ < tr.t1) {                                                                  \
                LLMOPS_BLOCK(P.s[i_], i_)                                                             \
            }                                                                                         \
        }                                                                                             \
        __builtin_amdgcn_wave_barrier(); /* reads stay ahead of the next pass's writes */             \
    } while (0)
    if (tr.t0 < tr.t1) {
        if constexpr (!kBarrierStat) {
            LLMOPS_LOAD_PAIR(P0, tr.t0, true);
            if constexpr (NORM && SUMS) {
                LLMOPS_SUMS_STAT
            }
        }
        // Most shapes give a wave one pass; a longer run asks for the next pass only when this one is done,
        // which keeps the registers of the two from overlapping (64 in all).
        for (int tp = tr.t0; tp < tr.t1; tp += SPP) {
            LLMOPS_PAIR(P0, tp);
            if (tp + SPP < tr.t1) LLMOPS_LOAD_PAIR(P0, tp + SPP, true);
        }
    }
#undef LLMOPS_PAIR
#undef LLMOPS_BLOCK
#undef LLMOPS_LOAD_PAIR
#undef LLMOPS_SUMS_STAT

    if (!GLU) {
        if (NORM) {
            LLMOPS_LOAD_RESIDUAL(wave * 64 + lane_id_now())
        }
#undef LLMOPS_LOAD_RESIDUAL
        // exchange: two k-splits meet through 64-bit slots (which `part` then points at) instead of the ticket
        finish_strip<MT, NW>(f, red, &ticket_sh, wave, tr.nb, tr.s, S, rows, N, y, part, counters, residual != nullptr, resv,
                             sumsq_out, exchange ? reinterpret_cast<unsigned long long*>(part) : nullptr);
        return;
    }
    // gate/up epilogue: sum row slots, then the two halves of the workgroup, then silu(gate)*up
    const int quad = lane & 7;
#pragma unroll
    for (int r = 0; r < MT; r++) rowslot_sum4(f[r]);
    if (rs == 0) {
#pragma unroll
        for (int r = 0; r < MT; r++)
#pragma unroll
            for (int j = 0; j < 4; j++) red[wave][r][quad * 4 + j] = f[r][j];
    }
    __syncthreads();
    const int tid = wave * 64 + lane_id_now();
    const int trow = tid >> 5, tn = tid & 31;
    if (trow < MT && trow < rows) {
        float g = 0.0f, u = 0.0f;
#pragma unroll
        for (int w = 0; w < NWS; w++) {
            g += red[w][trow][tn];
            u += red[GLU ? w + NWS : w][trow][tn];
        }
        const int64_t n = (int64_t)blockIdx.x * kGroupN + tn;  // N = number of output columns (F)
        if (n < N) y[(int64_t)trow * N + n] = silu_times(g, u);
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
static int g_exchange_handoff = 1;     // 0: two k-splits also meet through the arrival ticket
static int g_waves_per_workgroup = 0;  // 0 = choose per shape (pre-quantized variant only)

struct GemvPlan {
    int S, steps_per_split, NW;
};

static GemvPlan plan_gemv(int64_t rows, int64_t Ng, int64_t Kg, int G, bool fused) {
    const int bps = (G == 128) ? 1 : 2;
    const int T = (int)((Kg + bps - 1) / bps);
    int NW = fused ? 0 : g_waves_per_workgroup;
    if (NW == 0) NW = 16;
    if (rows > 4 && NW > 8) NW = 8;  // one (row, column) finaliser thread per output of the strip
    int S = (int)((g_target_workgroups + Ng - 1) / Ng);
    // a wave already has at most one pass of 256 k-values (2 steps at group 128, 4 at group 32 in the kernel
    // that quantizes on the fly): splitting would leave passes half empty (4096x4096 at group 32: 5.5 us
    // whole against 5.9 us in two splits)
    if ((T + NW - 1) / NW <= ((G == 32 && fused) ? 4 : 2)) S = 1;
    const int max_s = (T + NW - 1) / NW;  // at least one step per wave
    if (S > max_s) S = max_s;
    if (S < 1) S = 1;
    int sps = (T + S - 1) / S;
    S = (T + sps - 1) / sps;  // drop empty splits
    return {S, sps, NW};
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
    AttnRecs recs;          // stats != nullptr: the input is the chunk records of decode attention
};

template <int G, int MT, int NW>
static void launch_fused_t(const uint8_t* w, const float* x, float* y, float* part, unsigned* counters, int64_t Ng,
                           int64_t Kg, int64_t N, int rows, GemvPlan p, const FusedOps& o, hipStream_t st,
                           const DumpBufs* dump = nullptr) {
    // Two k-splits: the splits meet through one 64-bit exchange per output, in slots behind the arrival
    // counters in the zeroed head of the workspace (if they fit there).
    // (outputs' slots, then one slot per (row, strip) for the partial sums of squares)
    const int64_t slot_bytes = (int64_t)rows * Ng * kGroupN * 8 + (int64_t)rows * Ng * 8;
    const int exchange = g_exchange_handoff && p.S == 2 && !o.glu && slot_bytes <= LLMOPS_FC_COUNTER_BYTES - kTicketBytes;
    if (exchange) part = reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(counters) + kTicketBytes);
#define LLMOPS_FUSED(MODE, GRID)                                                                                      \
    fc_gemv_fused_kernel<G, MT, NW, MODE><<<(unsigned)(GRID), NW * 64, 0, st>>>(                                      \
        w, x, (int)Kg, p.S, p.steps_per_split, rows, (int)N, o.sumsq_parts, o.residual, o.sumsq_in, o.norm_w, o.eps, y,   \
        part, counters, o.sumsq_out, exchange, dump ? *dump : DumpBufs{nullptr, nullptr, nullptr, nullptr}, o.recs)
    // (the kernel reads up to 256 handed-over partial sums per row; with more, the statistic is recomputed)
    const bool sums = o.norm_w != nullptr && o.sumsq_in != nullptr && o.sumsq_parts <= 256;
    if (dump != nullptr) {  // plain fc_Q4A, or the chunk records of attention as input
        if (o.recs.stats == nullptr) LLMOPS_FUSED(kDump, Ng * p.S);
        else if constexpr (G == 128 && MT == 1) LLMOPS_FUSED(kDump | kAttnIn, Ng * p.S);
    } else if (o.recs.stats != nullptr) {
        if constexpr (G == 128 && MT == 1) LLMOPS_FUSED(kAttnIn, Ng * p.S);
    } else if (o.glu_in) {
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
                      const float* sumsq_in, int sumsq_parts, float* sumsq_out, hipStream_t st, const DumpBufs* dump,
                      const float* rec_stats, const float* rec_outs, int rec_chunks) {
    GemvPlan p = plan_gemv(rows, Ng, Kg, G, true);
    if (glu == 1) p.S = 1;
    if (N > INT32_MAX || Kg * G > INT32_MAX) return fail(LLMOPS_EINVAL, "fc_Q4A for up to 8 rows: N and K must fit 31 bits");
    if (dump != nullptr && (norm_w != nullptr || glu != 0)) return fail(LLMOPS_EINVAL, "the dump build runs the plain FC only");
    if (rec_stats != nullptr && (rows != 1 || G != 128 || norm_w != nullptr || glu != 0))
        return fail(LLMOPS_EINVAL, "chunk records as input: one row, group 128, no rmsnorm, no gate/up forms");
    const FusedOps o{residual, norm_w, eps, glu == 1, glu == 2, sumsq_in, sumsq_parts, sumsq_out, AttnRecs{rec_stats, rec_outs, rec_chunks}};
#define LLMOPS_CASE(GG, MT, NWW) launch_fused_t<GG, MT, NWW>(w, x, y, part, counters, Ng, Kg, N, (int)rows, p, o, st, dump)
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

extern "C" void llmops_test_fc_set_tuning(int target_workgroups, int waves_per_workgroup) {
    if (!llmops::test_hooks_enabled(__func__)) return;
    if (target_workgroups == -2 || target_workgroups == -3) {  // hand-off of two k-splits: -2 exchange slots, -3 ticket
        llmops::g_exchange_handoff = target_workgroups == -2;
        return;
    }
    if (target_workgroups > 0) llmops::g_target_workgroups = target_workgroups > 4096 ? 4096 : target_workgroups;
    if (waves_per_workgroup >= 0) llmops::g_waves_per_workgroup = waves_per_workgroup;
}

