// Q4_1 x Q8 fully-connected product for a handful of activation rows (decode): an HBM-streaming
// kernel built on v_dot4_i32_i8.
//
// Data movement.  The packed tensor [Ng][Kg][block] is a set of Ng independent strips (32 output
// columns each) whose blocks are contiguous in memory, so a strip is one linear stream.  Work is
// cut into (strip, k-range) tiles: one 256-thread workgroup per tile, each of its 4 wavefronts
// streaming a contiguous run of blocks with 16-byte loads per lane:
//
//   lane = rs*8 + quad,  rs = 0..7 (k8-row slot), quad = 0..7 (4 adjacent columns)
//   one wave-wide 16 B load = 8 k8-rows x 128 B = 64 k-values x 32 columns, perfectly coalesced
//   dword j of the load = column quad*4+j, k-values 8*row..8*row+7 (low nibbles k 0..3,
//   high nibbles k 4..7), so (dw & 0x0F0F0F0F) and ((dw>>4) & 0x0F0F0F0F) feed two v_dot4
//   against the lane's 8 activation codes with no shuffling.
//
// Each lane keeps fp32 running sums for its 4 columns (x rows); per block it folds its int32
// partial dot product in as (d*dx)*acc, and the lanes on a block's first k8-row add m*gsum.
// The 8 row slots are summed at the end with xor-shuffles, the 4 waves through LDS, and the
// k-splits of a strip through a scratch buffer: the workgroup that arrives last at the strip's
// counter adds the splits in index order, so results do not depend on scheduling.
//
// Follows fc_Q4A (/root/reference/ops/op_fc.hpp:286-426) for the arithmetic; the int32 partial
// sums are exact, the fp32 accumulation order differs from the reference's kb-sequential chain
// (bounded well inside the 1e-3 contract).
#include "common.h"

namespace llmops {

int launch_quant_x(const float* x, int64_t rows, int64_t K, int group_k, int8_t* xq, float* xd, float* gsum,
                   hipStream_t stream);

constexpr int kMaxGemvRows = 8;

__device__ __forceinline__ uint4 ldg16(const uint8_t* p) { return *reinterpret_cast<const uint4*>(p); }
__device__ __forceinline__ uint2 ldg8(const uint8_t* p) { return *reinterpret_cast<const uint2*>(p); }

// One "step" of a wavefront: G=128 -> one block (two 16 B loads per lane);
//                            G=32  -> two adjacent blocks, one per half-wave (one load per lane).
template <int G>
struct Step {
    static constexpr int kLoads = (G == 128) ? 2 : 1;
    static constexpr int kBlocksPerStep = (G == 128) ? 1 : 2;
    uint4 w[kLoads];
    uint2 dh, mh;  // 4 x fp16 d, 4 x fp16 m of the lane's columns
    bool valid;
};

template <int G>
__device__ __forceinline__ void load_step(Step<G>& st, const uint8_t* strip, int step, int kb_end, int lane) {
    const int quad = lane & 7, rs = lane >> 3;
    if (G == 128) {
        const uint8_t* blk = strip + (int64_t)step * block_bytes(128);
        st.valid = true;
        st.w[0] = ldg16(blk + lane * 16);
        st.w[Step<G>::kLoads - 1] = ldg16(blk + 1024 + lane * 16);
        st.dh = ldg8(blk + 2048 + quad * 8);
        st.mh = ldg8(blk + 2048 + 64 + quad * 8);
    } else {
        const int kb = step * 2 + (rs >> 2);
        st.valid = kb < kb_end;
        const uint8_t* blk = strip + (int64_t)kb * block_bytes(32);
        if (st.valid) {
            st.w[0] = ldg16(blk + (rs & 3) * kRowBytes + quad * 16);
            st.dh = ldg8(blk + 512 + quad * 8);
            st.mh = ldg8(blk + 512 + 64 + quad * 8);
        } else {
            st.w[0] = make_uint4(0, 0, 0, 0);
            st.dh = make_uint2(0, 0);
            st.mh = make_uint2(0, 0);
        }
    }
}

// int32 partial dot products of the lane's 4 columns over the lane's k8-rows of this step
template <int G>
__device__ __forceinline__ void dot_step(const Step<G>& st, const int8_t* xq_row, int step, int lane, int acc[4]) {
    const int rs = lane >> 3;
    const int2 xa = *reinterpret_cast<const int2*>(xq_row + (int64_t)step * (G == 128 ? 128 : 64) + rs * 8);
    const uint32_t* w0 = reinterpret_cast<const uint32_t*>(&st.w[0]);
#pragma unroll
    for (int j = 0; j < 4; j++) acc[j] = dot8_q4(w0[j], xa.x, xa.y, 0);
    if (G == 128) {
        const int2 xb = *reinterpret_cast<const int2*>(xq_row + (int64_t)step * 128 + 64 + rs * 8);
        const uint32_t* w1 = reinterpret_cast<const uint32_t*>(&st.w[Step<G>::kLoads - 1]);
#pragma unroll
        for (int j = 0; j < 4; j++) acc[j] = dot8_q4(w1[j], xb.x, xb.y, acc[j]);
    }
}

__device__ __forceinline__ void unpack_h4(uint2 h, float out[4]) {
    out[0] = f16_bits_to_f32((uint16_t)(h.x & 0xFFFFu));
    out[1] = f16_bits_to_f32((uint16_t)(h.x >> 16));
    out[2] = f16_bits_to_f32((uint16_t)(h.y & 0xFFFFu));
    out[3] = f16_bits_to_f32((uint16_t)(h.y >> 16));
}

template <int G, int MT>
__global__ __launch_bounds__(256) void fc_gemv_kernel(const uint8_t* __restrict__ weiq, const int8_t* __restrict__ xq,
                                                       const float* __restrict__ xd, const float* __restrict__ gs,
                                                       float* __restrict__ y, float* part, unsigned* counters, int Kg,
                                                       int64_t N, int rows, int S, int steps_per_split) {
    constexpr int BPS = Step<G>::kBlocksPerStep;
    __shared__ float red[4][MT][kGroupN];
    __shared__ unsigned ticket_sh;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nb = blockIdx.x / S, s = blockIdx.x % S;
    const int quad = lane & 7, rs = lane >> 3;
    const int T = (Kg + BPS - 1) / BPS;  // steps in a strip
    const int t_lo = s * steps_per_split;
    const int t_hi = min(T, t_lo + steps_per_split);
    const int per_wave = (t_hi - t_lo + 3) >> 2;
    const int t0 = min(t_hi, t_lo + wave * per_wave), t1 = min(t_hi, t0 + per_wave);
    const uint8_t* strip = weiq + (int64_t)nb * Kg * block_bytes(G);
    const int64_t Kp = (int64_t)Kg * G;  // padded K of the activation codes

    float f[MT][4];
#pragma unroll
    for (int r = 0; r < MT; r++)
#pragma unroll
        for (int j = 0; j < 4; j++) f[r][j] = 0.0f;

    Step<G> cur, nxt;
    if (t0 < t1) load_step<G>(cur, strip, t0, Kg, lane);
    for (int t = t0; t < t1; t++) {
        if (t + 1 < t1) load_step<G>(nxt, strip, t + 1, Kg, lane);
        // block index whose scales this lane applies
        const int kb = (G == 128) ? t : t * 2 + (rs >> 2);
        float d[4], m[4];
        unpack_h4(cur.dh, d);
        unpack_h4(cur.mh, m);
        const bool first_row = (G == 128) ? (rs == 0) : ((rs & 3) == 0);
#pragma unroll
        for (int r = 0; r < MT; r++) {
            if (r < rows && cur.valid) {
                int acc[4];
                dot_step<G>(cur, xq + r * Kp, t, lane, acc);
                const float dx = xd[(int64_t)r * Kg + kb];
                const float g = first_row ? gs[(int64_t)r * Kg + kb] : 0.0f;
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    f[r][j] = fmaf(d[j] * dx, (float)acc[j], f[r][j]);
                    f[r][j] = fmaf(m[j], g, f[r][j]);
                }
            }
        }
        cur = nxt;
    }

    // sum the 8 row slots (lane bits 3..5)
#pragma unroll
    for (int r = 0; r < MT; r++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            float v = f[r][j];
            v += __shfl_xor(v, 8, 64);
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
    const int64_t n = (int64_t)nb * kGroupN + tn;
    const int64_t Np = (int64_t)gridDim.x / S * kGroupN;
    float v = 0.0f;
    if (tr < MT && tr < rows) v = ((red[0][tr][tn] + red[1][tr][tn]) + red[2][tr][tn]) + red[3][tr][tn];
    if (S == 1) {
        if (tr < MT && tr < rows && n < N) y[(int64_t)tr * N + n] = v;
        return;
    }
    // Cross-workgroup hand-off without cache-wide fences: partial sums are written and read with
    // device-scope (write-through / cache-bypassing) accesses, and the arrival counter is a
    // device-scope atomic.  __syncthreads() waits for this workgroup's stores to be acknowledged
    // before thread 0 announces the arrival.  (A __threadfence() here makes every workgroup
    // write back and invalidate its whole L2 slice, which costs far more than the kernel itself.)
    if (tr < MT && tr < rows)
        __hip_atomic_store(&part[((int64_t)s * rows + tr) * Np + n], v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the write-through stores above have been acknowledged
    __syncthreads();
    if (threadIdx.x == 0)
        ticket_sh = __hip_atomic_fetch_add(&counters[nb], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (ticket_sh != (unsigned)(S - 1)) return;
    if (tr < MT && tr < rows && n < N) {
        float acc = 0.0f;
        for (int i = 0; i < S; i++)
            acc += __hip_atomic_load(&part[((int64_t)i * rows + tr) * Np + n], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        y[(int64_t)tr * N + n] = acc;
    }
    if (threadIdx.x == 0) __hip_atomic_store(&counters[nb], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // next launch
}

// Integer core only: acc[r][n][kb] (int32).  One wavefront per step, same loads and same dot
// code as fc_gemv_kernel; the row slots of a block are summed with xor-shuffles.
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
        if (st.valid) dot_step<G>(st, xq + r * Kp, t, lane, acc);
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

static int g_target_workgroups = 1024;

struct GemvPlan {
    int S, steps_per_split;
};

static GemvPlan plan_gemv(int64_t Ng, int64_t Kg, int G) {
    const int bps = (G == 128) ? 1 : 2;
    const int T = (int)((Kg + bps - 1) / bps);
    int S = (int)((g_target_workgroups + Ng - 1) / Ng);
    const int max_s = (T + 3) / 4;  // at least one step per wave
    if (S > max_s) S = max_s;
    if (S < 1) S = 1;
    int sps = (T + S - 1) / S;
    S = (T + sps - 1) / sps;  // drop empty splits
    return {S, sps};
}

size_t gemv_workspace_bytes(int64_t rows, int64_t Ng, int64_t Kg, int G) {
    const GemvPlan p = plan_gemv(Ng, Kg, G);
    return (size_t)p.S * rows * Ng * kGroupN * sizeof(float);
}

template <int G, int MT>
static void launch_gemv_t(const uint8_t* w, const int8_t* xq, const float* xd, const float* gs, float* y, float* part,
                          unsigned* counters, int64_t Ng, int64_t Kg, int64_t N, int rows, GemvPlan p, hipStream_t st) {
    fc_gemv_kernel<G, MT><<<(unsigned)(Ng * p.S), 256, 0, st>>>(w, xq, xd, gs, y, part, counters, (int)Kg, N, rows, p.S,
                                                                p.steps_per_split);
}

int launch_gemv(const uint8_t* w, const int8_t* xq, const float* xd, const float* gs, float* y, float* part,
                unsigned* counters, int64_t rows, int64_t Ng, int64_t Kg, int G, int64_t N, hipStream_t st) {
    const GemvPlan p = plan_gemv(Ng, Kg, G);
#define LLMOPS_GEMV_CASE(GG, MT) launch_gemv_t<GG, MT>(w, xq, xd, gs, y, part, counters, Ng, Kg, N, (int)rows, p, st)
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

// Development knob: number of workgroups the split-K planner aims for (default 1024).
extern "C" void llmops_fc_set_target_workgroups(int n) {
    if (n > 0) llmops::g_target_workgroups = n;
}
