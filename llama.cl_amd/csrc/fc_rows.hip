// Q4_1 x Q8 fully-connected product for 9..16 activation rows (group 128): weight streaming like
// the one-row kernel, inner product on the int8 matrix cores.
//
// With this few rows the FC is still bound by the weight stream, so the work is cut like the
// decode kernel's: one workgroup per strip of 32 output columns, its 8 waves split K into
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

namespace llmops {

typedef int v4i_r __attribute__((ext_vector_type(4)));
typedef float v4f_r __attribute__((ext_vector_type(4)));

constexpr int kRowsWaves = 8;
constexpr int kRowsBlk = 2176;

template <int RT>
struct RowsStage {
    uint32_t w[2][2][2];  // [64-k half][16-column tile][k8-row of the pair]
    uint16_t d[2], m[2];  // fp16 scale and min of the lane's column in either tile
    v4i_r a[RT][2];       // activation codes: row tile, 64-k half
    float2 xs[RT][4];     // (dx, gsum) of the 4 rows this lane holds results for
};

template <int RT>
__device__ __forceinline__ void rows_load(RowsStage<RT>& st, const uint8_t* __restrict__ strip, const int8_t* __restrict__ xq,
                                          const float2* __restrict__ xsT, int kb, int64_t Kp, int rows, int g, int jj) {
    const uint8_t* blk = strip + (int64_t)kb * kRowsBlk;
#pragma unroll
    for (int h = 0; h < 2; h++)
#pragma unroll
        for (int tau = 0; tau < 2; tau++)
#pragma unroll
            for (int p = 0; p < 2; p++)
                st.w[h][tau][p] = __builtin_nontemporal_load(
                    reinterpret_cast<const uint32_t*>(blk + (8 * h + 2 * g + p) * kRowBytes + (16 * tau + jj) * 4));
#pragma unroll
    for (int tau = 0; tau < 2; tau++) {
        st.d[tau] = *reinterpret_cast<const uint16_t*>(blk + 2048 + 2 * (16 * tau + jj));
        st.m[tau] = *reinterpret_cast<const uint16_t*>(blk + 2048 + 64 + 2 * (16 * tau + jj));
    }
#pragma unroll
    for (int t = 0; t < RT; t++) {
        const int ra = min(rows - 1, 16 * t + jj);
#pragma unroll
        for (int h = 0; h < 2; h++)
            st.a[t][h] = *reinterpret_cast<const v4i_r*>(xq + (int64_t)ra * Kp + (int64_t)kb * 128 + 64 * h + 16 * g);
#pragma unroll
        for (int v = 0; v < 4; v++) st.xs[t][v] = xsT[(int64_t)kb * rows + min(rows - 1, 16 * t + 4 * g + v)];
    }
}

template <int RT>
__global__ __launch_bounds__(kRowsWaves * 64, 4) void fc_rows_mfma_kernel(const uint8_t* __restrict__ weiq,
                                                                         const int8_t* __restrict__ xq,
                                                                         const float2* __restrict__ xsT,
                                                                         float* __restrict__ y, int Kg, int64_t N, int rows,
                                                                         const float* __restrict__ residual) {
    constexpr int NW = kRowsWaves;
    __shared__ float red[NW][16 * RT][kGroupN];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane >> 4, jj = lane & 15;
    const uint8_t* strip = weiq + (int64_t)blockIdx.x * Kg * kRowsBlk;
    const int64_t Kp = (int64_t)Kg * 128;
    const int t0 = (wave * Kg) / NW, t1 = ((wave + 1) * Kg) / NW;  // this wave's k-groups

    v4f_r f[RT][2];
#pragma unroll
    for (int t = 0; t < RT; t++)
#pragma unroll
        for (int tau = 0; tau < 2; tau++) f[t][tau] = v4f_r{0.f, 0.f, 0.f, 0.f};

    RowsStage<RT> cur, nxt;
    if (t0 < t1) rows_load<RT>(cur, strip, xq, xsT, t0, Kp, rows, g, jj);
    for (int kb = t0; kb < t1; kb++) {
        if (kb + 1 < t1) rows_load<RT>(nxt, strip, xq, xsT, kb + 1, Kp, rows, g, jj);
        v4i_r b[2][2];
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int tau = 0; tau < 2; tau++) {
                const uint32_t pa = cur.w[h][tau][0], pb = cur.w[h][tau][1];
                b[h][tau] = v4i_r{(int)(pa & 0x0F0F0F0Fu), (int)((pa >> 4) & 0x0F0F0F0Fu), (int)(pb & 0x0F0F0F0Fu),
                                  (int)((pb >> 4) & 0x0F0F0F0Fu)};
            }
#pragma unroll
        for (int tau = 0; tau < 2; tau++) {
            const float d = f16_bits_to_f32(cur.d[tau]), m = f16_bits_to_f32(cur.m[tau]);
#pragma unroll
            for (int t = 0; t < RT; t++) {
                v4i_r acc = v4i_r{0, 0, 0, 0};
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(cur.a[t][0], b[0][tau], acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(cur.a[t][1], b[1][tau], acc, 0, 0, 0);
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    f[t][tau][v] = fmaf(d * cur.xs[t][v].x, (float)acc[v], f[t][tau][v]);
                    f[t][tau][v] = fmaf(m, cur.xs[t][v].y, f[t][tau][v]);
                }
            }
        }
        cur = nxt;
    }

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
        const int64_t n = (int64_t)blockIdx.x * kGroupN + col;
        if (row < rows && n < N) {
            float v = 0.0f;
#pragma unroll
            for (int w = 0; w < NW; w++) v += red[w][row][col];
            y[(int64_t)row * N + n] = residual ? v + residual[(int64_t)row * N + n] : v;
        }
    }
}

// rows <= 16, group 128, activations already quantized (codes [rows, Kg*128], pairs [Kg][rows])
int launch_fc_rows(const uint8_t* w, const int8_t* xq, const float2* xsT, float* y, int64_t rows, int64_t Ng, int64_t Kg,
                   int64_t N, const float* residual, hipStream_t st) {
    if (rows > 16) return fail(LLMOPS_EINVAL, "the streaming MFMA kernel takes at most 16 rows, got %lld", (long long)rows);
    fc_rows_mfma_kernel<1><<<(unsigned)Ng, kRowsWaves * 64, 0, st>>>(w, xq, xsT, y, (int)Kg, N, (int)rows, residual);
    LLMOPS_LAUNCH_CHECK();
    return LLMOPS_OK;
}

}  // namespace llmops
