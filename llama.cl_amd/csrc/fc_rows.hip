// Q4_1 x Q8 fully-connected product for 3..32 activation rows (group 128): weight streaming like
// the one-row kernel, inner product on the int8 matrix cores.
//
// With this few rows the FC is still bound by the weight stream, so the work is cut like the
// decode kernel's: one workgroup per strip of 32 output columns, its 8 or 16 waves split K into
// contiguous runs of k-groups, every wave reads each packed weight byte once, and the waves'
// fp32 results meet in LDS.  Nothing is staged through LDS on the way in: a lane fetches exactly
// the two dwords per (64-k half, 16-column tile) that make up its B operand of
// v_mfma_i32_16x16x64_i8 (dword (k8-row r, column n) of a block holds k = 8r..8r+7 of that
// column; lane (g, j) of the MFMA needs k = 16g..16g+15 of column j), unpacks them with two ANDs
// and a shift, and takes its A operand (16 int8 codes of one activation row) straight from the
// quantized activations in L2.  Per k-group and output element the fp32 fold is the reference's
// (ops/op_fc.hpp:381-412): f = fma(d*dx, float(acc), f); f = fma(m, gsum, f).
//
// The activations come pre-quantized (llmops_FC_dynamic_quantize_x_rows, with the (scale, sum)
// pairs transposed to [Kg][rows]); the int32 sums are the same as in every other path.
#include "common.h"
#include "gemv_device.h"

namespace llmops {

typedef int v4i_r __attribute__((ext_vector_type(4)));
typedef float v4f_r __attribute__((ext_vector_type(4)));

static int g_rows_split = 1;  // 0: never cut K in two for tensors with few strips
constexpr int kRowsBlk = 2176;

template <int RT>
struct RowsStage {
    uint32_t w[2][2][2];  // [64-k half][16-column tile][k8-row of the pair]
    uint32_t d[2], m[2];  // the dword that holds the fp16 scale / min of the lane's column in either tile
    v4i_r a[RT][2];       // activation codes: row tile, 64-k half
    float2 xs[RT][4];     // (dx, gsum) of the 4 rows this lane holds results for
};

// Loads of one k-group through buffer descriptors (scalar base + scalar offset + 32-bit lane offset).
// A stage that is not wanted (past the wave's last k-group) is asked for through descriptors of size 0,
// which return 0 without touching memory, instead of being branched around: loads complete in issue
// order and are counted, so only a loop whose every iteration issues the same loads lets the wave wait
// for exactly the stage it is about to use while the next one is still in flight.
struct RowsBufs {
    const void *w_base, *xq_base, *xs_base;
    uint32_t w_bytes, xq_bytes, xs_bytes;
    uint32_t lane_w, lane_s, lane_a[2], lane_x[2];  // lane offsets (bytes); RT <= 2
};

template <int RT>
__device__ __forceinline__ void rows_load(RowsStage<RT>& st, const RowsBufs& bf, int kb, int rows, bool wanted) {
    const uint32_t sw = (uint32_t)kb * (uint32_t)kRowsBlk;
    // (the size is chosen with scalar instructions; per-lane offsets stay loop invariants)
    const buffer_rsrc rw = make_rsrc(bf.w_base, wanted ? bf.w_bytes : 0u);
    const buffer_rsrc rq = make_rsrc(bf.xq_base, wanted ? bf.xq_bytes : 0u);
    const buffer_rsrc rx = make_rsrc(bf.xs_base, wanted ? bf.xs_bytes : 0u);
    const uint32_t lw = bf.lane_w, ls = bf.lane_s;
#pragma unroll
    for (int h = 0; h < 2; h++)
#pragma unroll
        for (int tau = 0; tau < 2; tau++)
#pragma unroll
            for (int p = 0; p < 2; p++)
                st.w[h][tau][p] = __builtin_amdgcn_raw_buffer_load_b32(rw, lw, sw + (uint32_t)((8 * h + p) * kRowBytes + 64 * tau), 2);
#pragma unroll
    for (int tau = 0; tau < 2; tau++) {
        st.d[tau] = __builtin_amdgcn_raw_buffer_load_b32(rw, ls, sw + 2048u + 32u * tau, 0);
        st.m[tau] = __builtin_amdgcn_raw_buffer_load_b32(rw, ls, sw + 2048u + 64u + 32u * tau, 0);
    }
#pragma unroll
    for (int t = 0; t < RT; t++) {
        const uint32_t la = bf.lane_a[t];
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rq, la, (uint32_t)kb * 128u + 64u * h, 0);
            st.a[t][h] = v4i_r{(int)v.x, (int)v.y, (int)v.z, (int)v.w};
        }
        // the (scale, sum) pairs of the lane's 4 rows are contiguous: two 16-byte loads.  Rows past `rows`
        // read the next k-group's pairs (or 0 past the end of the buffer); their results are never stored.
        const uint32_t lx = bf.lane_x[t];
#pragma unroll
        for (int v2 = 0; v2 < 2; v2++) {
            const u32x4 q = __builtin_amdgcn_raw_buffer_load_b128(rx, lx, (uint32_t)kb * (uint32_t)rows * 8u + 16u * v2, 0);
            st.xs[t][2 * v2] = make_float2(__uint_as_float(q.x), __uint_as_float(q.y));
            st.xs[t][2 * v2 + 1] = make_float2(__uint_as_float(q.z), __uint_as_float(q.w));
        }
    }
}

// DUMP: test build that stores the int32 sums of every (row, column, k-group) into `dump`
// ([rows][Ng*32][Kg]) instead of the outputs (llmops_fc_Q4A_partials with use_mfma = 3).
template <int RT, int NW, bool DUMP = false>
__global__ __launch_bounds__(NW * 64, RT == 2 ? 3 : 4) void fc_rows_mfma_kernel(const uint8_t* __restrict__ weiq,
                                                                         const int8_t* __restrict__ xq,
                                                                         const float2* __restrict__ xsT,
                                                                         unsigned long long* slots, int Kg, int rows,
                                                                         int64_t N, float* __restrict__ y,
                                                                         const float* __restrict__ residual,
                                                                         int32_t* dump = nullptr) {
    // (argument order: what the first loads need comes in the first 14 dwords, which arrive in scalar registers
    // with the wave)
    __shared__ float red[DUMP ? 1 : NW][16 * RT][kGroupN];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // uniform: block offsets stay scalar
    const int g = lane >> 4, jj = lane & 15;
    // slots != nullptr: two workgroups per strip, each with half of K (tensors with fewer strips than the
    // chip has compute units); the halves meet through one 64-bit exchange per output (below)
    const int nb = slots ? blockIdx.x >> 1 : blockIdx.x, split = slots ? blockIdx.x & 1 : 0;
    const uint8_t* strip = weiq + (int64_t)nb * Kg * kRowsBlk;
    const int64_t Kp = (int64_t)Kg * 128;
    const int k_lo = slots ? (split * Kg) / 2 : 0, k_n = slots ? ((split + 1) * Kg) / 2 - k_lo : Kg;
    const int t0 = k_lo + (wave * k_n) / NW, t1 = k_lo + ((wave + 1) * k_n) / NW;  // this wave's k-groups

    v4f_r f[RT][2];
#pragma unroll
    for (int t = 0; t < RT; t++)
#pragma unroll
        for (int tau = 0; tau < 2; tau++) f[t][tau] = v4f_r{0.f, 0.f, 0.f, 0.f};

    RowsBufs bf;
    bf.w_base = strip, bf.w_bytes = (uint32_t)Kg * (uint32_t)kRowsBlk;
    bf.xq_base = xq, bf.xq_bytes = (uint32_t)rows * (uint32_t)Kp;
    bf.xs_base = xsT, bf.xs_bytes = DUMP ? 0u : (uint32_t)Kg * (uint32_t)rows * 8u;
    bf.lane_w = (uint32_t)(2 * g * kRowBytes + jj * 4);
    bf.lane_s = (uint32_t)((jj >> 1) * 4);  // the dword with this column's fp16 scale; half_sh picks the half
    const int half_sh = (jj & 1) * 16;
#pragma unroll
    for (int t = 0; t < RT; t++) {
        bf.lane_a[t] = (uint32_t)min(rows - 1, 16 * t + jj) * (uint32_t)Kp + 16u * g;
        bf.lane_x[t] = (uint32_t)(16 * t + 4 * g) * 8u;
    }

    // Two stages used alternately (no register copies: a copy would have to wait for the loads it copies):
    // the k-group being multiplied waits for exactly its own loads while the next one's are in flight.
#define LLMOPS_ROWS_COMPUTE(ST, KB)                                                                          \
    do {                                                                                                     \
        v4i_r b[2][2];                                                                                       \
        _Pragma("unroll") for (int h = 0; h < 2; h++) _Pragma("unroll") for (int tau = 0; tau < 2; tau++) {  \
            const uint32_t pa = ST.w[h][tau][0], pb = ST.w[h][tau][1];                                       \
            b[h][tau] = v4i_r{(int)(pa & 0x0F0F0F0Fu), (int)((pa >> 4) & 0x0F0F0F0Fu), (int)(pb & 0x0F0F0F0Fu), \
                              (int)((pb >> 4) & 0x0F0F0F0Fu)};                                               \
        }                                                                                                    \
        _Pragma("unroll") for (int tau = 0; tau < 2; tau++) {                                                \
            const float d = f16_bits_to_f32((uint16_t)(ST.d[tau] >> half_sh));                               \
            const float m = f16_bits_to_f32((uint16_t)(ST.m[tau] >> half_sh));                               \
            _Pragma("unroll") for (int t = 0; t < RT; t++) {                                                 \
                v4i_r acc = v4i_r{0, 0, 0, 0};                                                               \
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(ST.a[t][0], b[0][tau], acc, 0, 0, 0);            \
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(ST.a[t][1], b[1][tau], acc, 0, 0, 0);            \
                if constexpr (DUMP) {                                                                        \
                    const int64_t Np_ = (int64_t)(slots ? gridDim.x / 2 : gridDim.x) * kGroupN;              \
                    _Pragma("unroll") for (int v = 0; v < 4; v++) {                                          \
                        const int row_ = 16 * t + 4 * g + v;                                                 \
                        if (row_ < rows && (KB) < t1)                                                        \
                            dump[((int64_t)row_ * Np_ + nb * kGroupN + 16 * tau + jj) * Kg + (KB)] = acc[v]; \
                    }                                                                                        \
                }                                                                                            \
                _Pragma("unroll") for (int v = 0; v < 4; v++) {                                              \
                    f[t][tau][v] = fmaf(d * ST.xs[t][v].x, (float)acc[v], f[t][tau][v]);                     \
                    f[t][tau][v] = fmaf(m, ST.xs[t][v].y, f[t][tau][v]);                                     \
                }                                                                                            \
            }                                                                                                \
        }                                                                                                    \
    } while (0)
    // Four k-groups per pass, two stages in flight, nothing loaded is live across the loop's back edge (a
    // value that is would be copied there by the register allocator, and the copy waits for its load).  A
    // hidden size of 4096 gives a wave exactly one pass; longer runs start each pass with a fresh pair.
    RowsStage<RT> sa, sb;
    for (int kb = t0; kb < t1; kb += 4) {
        rows_load<RT>(sa, bf, kb, rows, true);
        rows_load<RT>(sb, bf, kb + 1, rows, kb + 1 < t1);
        __builtin_amdgcn_sched_barrier(0);
        LLMOPS_ROWS_COMPUTE(sa, kb);
        __builtin_amdgcn_sched_barrier(0);
        rows_load<RT>(sa, bf, kb + 2, rows, kb + 2 < t1);
        __builtin_amdgcn_sched_barrier(0);
        LLMOPS_ROWS_COMPUTE(sb, kb + 1);  // (a stage that was not wanted holds zeros and adds nothing)
        __builtin_amdgcn_sched_barrier(0);
        rows_load<RT>(sb, bf, kb + 3, rows, kb + 3 < t1);
        __builtin_amdgcn_sched_barrier(0);
        // (the loads above are issued whatever the run's length; only the arithmetic on zeros is skipped)
        if (kb + 2 < t1) {
            LLMOPS_ROWS_COMPUTE(sa, kb + 2);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (kb + 3 < t1) {
            LLMOPS_ROWS_COMPUTE(sb, kb + 3);
        }
    }
#undef LLMOPS_ROWS_COMPUTE
    if constexpr (DUMP) return;

    // the waves' sums meet in LDS; one thread finishes each output
#pragma unroll
    for (int t = 0; t < RT; t++)
#pragma unroll
        for (int tau = 0; tau < 2; tau++)
#pragma unroll
            for (int v = 0; v < 4; v++) red[wave][16 * t + 4 * g + v][16 * tau + jj] = f[t][tau][v];
    __syncthreads();
#pragma unroll
    for (int i = 0; i < RT; i++) {
        const int idx = threadIdx.x + NW * 64 * i;
        const int row = idx >> 5, col = idx & 31;
        const int64_t n = (int64_t)nb * kGroupN + col;
        if (row < rows && n < N) {
            float v = 0.0f;
#pragma unroll
            for (int w = 0; w < NW; w++) v += red[w][row][col];
            if (slots != nullptr) {
                // A slot is empty (0) or holds (1 << 32 | value bits).  Whoever finds the other half's value
                // adds the two (a + b: the same bits whichever came first), stores the output and empties the
                // slot for the next launch; whoever finds it empty has parked its own value and is done.
                unsigned long long* slot = slots + ((int64_t)row * gridDim.x / 2 * kGroupN + n);
                const unsigned long long parked = (1ull << 32) | (unsigned long long)__float_as_uint(v);
                const unsigned long long old = __hip_atomic_exchange(slot, parked, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if ((old >> 32) == 0ull) continue;
                v += __uint_as_float((unsigned)(old & 0xFFFFFFFFull));
                __hip_atomic_store(slot, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            y[(int64_t)row * N + n] = residual ? v + residual[(int64_t)row * N + n] : v;
        }
    }
}

// rows <= 32 (two row tiles per wave from 17 on), group 128, activations already quantized (codes [rows, Kg*128], pairs [Kg][rows])
// `slots`: the zeroed exchange area of the FC workspace (`slot_bytes` of it), or nullptr
int launch_fc_rows(const uint8_t* w, const int8_t* xq, const float2* xsT, float* y, int64_t rows, int64_t Ng, int64_t Kg,
                   int64_t N, const float* residual, unsigned long long* slots, size_t slot_bytes, hipStream_t st) {
    if (rows > 32) return fail(LLMOPS_EINVAL, "the streaming MFMA kernel takes at most 32 rows, got %lld", (long long)rows);
    // fewer strips than compute units and a K worth cutting: two workgroups per strip
    const bool split = slots != nullptr && g_rows_split && Ng < 256 && Kg >= 16 && (size_t)rows * Ng * kGroupN * 8 <= slot_bytes;
    const unsigned grid = (unsigned)(split ? 2 * Ng : Ng);
    unsigned long long* sl = split ? slots : nullptr;
    // A wave has four k-groups in flight per pass: 8 waves cover 32 k-groups per workgroup in one pass (a hidden
    // size of 4096); longer runs take 16 waves rather than a second pass (4096x11008 in two halves, 16 rows:
    // 13.3 against 13.8 us; with 32 k-groups 16 waves are slower, 15.7 against 14.1 us at 11008x4096).
    // 17..32 rows: two row tiles per wave, 8 waves (16 would not have the registers).
    const int64_t k_per_wg = split ? (Kg + 1) / 2 : Kg;
    if (rows > 16)
        fc_rows_mfma_kernel<2, 8><<<grid, 512, 0, st>>>(w, xq, xsT, sl, (int)Kg, (int)rows, N, y, residual);
    else if (k_per_wg > 32)
        fc_rows_mfma_kernel<1, 16><<<grid, 1024, 0, st>>>(w, xq, xsT, sl, (int)Kg, (int)rows, N, y, residual);
    else
        fc_rows_mfma_kernel<1, 8><<<grid, 512, 0, st>>>(w, xq, xsT, sl, (int)Kg, (int)rows, N, y, residual);
    LLMOPS_LAUNCH_CHECK();
    return LLMOPS_OK;
}

// The same loop in its dump build, launched with the workgroup shape and K split that launch_fc_rows picks for
// these sizes.  The (scale, sum) pairs are not needed for the integer sums: their descriptor has size 0.
int launch_fc_rows_partials(const uint8_t* w, const int8_t* xq, int32_t* acc, int64_t rows, int64_t Ng, int64_t Kg,
                            hipStream_t st) {
    const bool split = g_rows_split && Ng < 256 && Kg >= 16;
    const unsigned grid = (unsigned)(split ? 2 * Ng : Ng);
    // only tested against nullptr in the dump build, never dereferenced
    unsigned long long* sl = split ? reinterpret_cast<unsigned long long*>(acc) : nullptr;
    const int64_t k_per_wg = split ? (Kg + 1) / 2 : Kg;
    if (rows > 16)
        fc_rows_mfma_kernel<2, 8, true><<<grid, 512, 0, st>>>(w, xq, nullptr, sl, (int)Kg, (int)rows, 0, nullptr, nullptr, acc);
    else if (k_per_wg > 32)
        fc_rows_mfma_kernel<1, 16, true><<<grid, 1024, 0, st>>>(w, xq, nullptr, sl, (int)Kg, (int)rows, 0, nullptr, nullptr, acc);
    else
        fc_rows_mfma_kernel<1, 8, true><<<grid, 512, 0, st>>>(w, xq, nullptr, sl, (int)Kg, (int)rows, 0, nullptr, nullptr, acc);
    LLMOPS_LAUNCH_CHECK();
    return LLMOPS_OK;
}

}  // namespace llmops

extern "C" void llmops_test_fc_rows_set_split(int on) {
    if (llmops::test_hooks_enabled(__func__)) llmops::g_rows_split = on != 0;
}
