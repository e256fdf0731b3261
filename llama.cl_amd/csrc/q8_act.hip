// Per-group Q8 dynamic activation quantization (FC_dynamic_quantize_x,
// /root/reference/ops/op_fc.hpp:221-272).
//
// One wavefront quantizes one (row, k-group): the lanes hold the group's G floats in registers,
// the absolute maximum is a wave reduction (order independent, hence exact), codes are
// v_rndne (round half to even, like vroundps imm 0 in ops/utils.hpp:207) saturated to int8, and
// the raw group sum is accumulated left to right from lane registers so that it carries the
// same rounding as the reference's scalar loop (ops/op_fc.hpp:262-268).
#include "common.h"

namespace llmops {

__device__ __forceinline__ float lane_value(float v, int lane) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}

__device__ __forceinline__ int q8_code(float v, float id) {
    const float t = v * id;
    if (t != t) return -128;  // cvtps2dq(NaN) = INT_MIN, which the saturating packs turn into -128
    return (int)fminf(127.0f, fmaxf(-128.0f, rintf(t)));
}
// the last len % 8 values of a short group go through the reference's scalar tail, which rounds half away from
// zero (std::round, ops/utils.hpp:217-219) instead of half to even
__device__ __forceinline__ int q8_code_tail(float v, float id) { return (int)(int8_t)roundf(v * id); }

// EXACT_SUM: raw group sum accumulated left to right (bit-equal to the reference); otherwise a
// tree sum, which is what the prefill FC uses (the sum only feeds its fp32 output).
// xsT (optional): the same scale and sum again as float2 [Kg][rows] for the GEMM's tile loads.
template <int G, bool EXACT_SUM>
__global__ __launch_bounds__(256) void quant_x_kernel(const float* __restrict__ x, int64_t rows, int64_t K, int64_t Kg,
                                                       int8_t* __restrict__ xq, float* __restrict__ xd,
                                                       float* __restrict__ gsum, float2* __restrict__ xsT) {
    constexpr int E = (G >= 64) ? G / 64 : 1;  // elements per lane
    constexpr int LANES = G / E;               // lanes that hold data
    const int lane = threadIdx.x & 63;
    const int64_t item = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (item >= rows * Kg) return;  // whole wave leaves together
    const int64_t r = item / Kg, kb = item % Kg;
    const float* raw = x + r * K + kb * G;
    const int64_t left = K - kb * G;
    const int len = (int)(left < G ? left : G);

    const int vec = len & ~7;  // values the reference quantizes eight at a time; the rest take its scalar tail
    float v[E];
#pragma unroll
    for (int j = 0; j < E; j++) {
        const int e = lane * E + j;
        v[j] = (lane < LANES && e < len) ? raw[e] : 0.0f;
    }
    float amax = 0.0f;
#pragma unroll
    for (int j = 0; j < E; j++) amax = fmaxf(amax, fabsf(v[j]));
    amax = wave_max(amax);
    const float d = amax / 127.0f;
    const float id = (d != 0.0f) ? (1.0f / d) : 0.0f;

    if (lane < LANES) {
        int8_t* q = xq + (r * Kg + kb) * G + lane * E;
        if (E == 2) {
            const int e = lane * E;
            const uint32_t c0 = (uint32_t)(e < vec ? q8_code(v[0], id) : q8_code_tail(v[0], id)) & 0xFFu;
            const uint32_t c1 = (uint32_t)(e + 1 < vec ? q8_code(v[E - 1], id) : q8_code_tail(v[E - 1], id)) & 0xFFu;
            // padding beyond len is zero (ops/op_fc.hpp:259-261)
            *reinterpret_cast<uint16_t*>(q) = (uint16_t)((e < len ? c0 : 0u) | ((e + 1 < len ? c1 : 0u) << 8));
        } else {
            q[0] = (lane < len) ? (int8_t)(lane < vec ? q8_code(v[0], id) : q8_code_tail(v[0], id)) : (int8_t)0;
        }
    }

    float s = 0.0f;
    if (EXACT_SUM) {
        // left-to-right fp32 sum of the raw group, computed redundantly by every lane
#pragma unroll
        for (int i = 0; i < G; i++) {
            if (i < len) s += lane_value(v[i % E], i / E);
        }
    } else {
#pragma unroll
        for (int j = 0; j < E; j++) s += v[j];
        s = wave_sum(s);
    }
    if (lane == 0) {
        xd[r * Kg + kb] = d;
        gsum[r * Kg + kb] = s;
        if (xsT != nullptr) xsT[kb * rows + r] = make_float2(d, s);
    }
}

// Prefill variant (many rows): G/4 threads per group, each with one 16-byte load and one packed
// 4-code store per group, so a workgroup quantizes 256/(G/4) groups at a time with fully coalesced traffic.
// With many groups a team of G/4 threads takes U consecutive ones and asks for all of them before it uses
// the first (more bytes in flight per thread).  Codes and scales are the same bits as above; the raw group
// sum is a tree sum (it only feeds the fp32 output).  Whole groups only (K == Kg*G), so group i starts at
// float i*G of the dense [rows, K] array.
template <int G, int U>
__global__ __launch_bounds__(256) void quant_x_rows_kernel(const float* __restrict__ x, int64_t items, int64_t Kg,
                                                            int64_t rows, int8_t* __restrict__ xq, float* __restrict__ xd,
                                                            float* __restrict__ gsum, float2* __restrict__ xsT) {
    constexpr int TPG = G / 4;        // threads per group
    constexpr int GPW = 256 / TPG;    // teams per workgroup
    const int sub = threadIdx.x % TPG;
    const int64_t first = ((int64_t)blockIdx.x * GPW + threadIdx.x / TPG) * U;
    // a team's threads are all live or all idle for a group: the shuffles below stay inside a team
    float4 v[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
        const int64_t it = first + u < items ? first + u : items - 1;
        v[u] = *reinterpret_cast<const float4*>(x + it * G + sub * 4);
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
        const int64_t item = first + u;
        float amax = fmaxf(fmaxf(fabsf(v[u].x), fabsf(v[u].y)), fmaxf(fabsf(v[u].z), fabsf(v[u].w)));
        float s = (v[u].x + v[u].y) + (v[u].z + v[u].w);
#pragma unroll
        for (int o = TPG / 2; o > 0; o >>= 1) {
            amax = fmaxf(amax, __shfl_xor(amax, o, 64));
            s += __shfl_xor(s, o, 64);
        }
        const float d = amax / 127.0f;
        const float id = (d != 0.0f) ? (1.0f / d) : 0.0f;
        const uint32_t c = ((uint32_t)q8_code(v[u].x, id) & 0xFFu) | (((uint32_t)q8_code(v[u].y, id) & 0xFFu) << 8) |
                           (((uint32_t)q8_code(v[u].z, id) & 0xFFu) << 16) | (((uint32_t)q8_code(v[u].w, id) & 0xFFu) << 24);
        if (item < items) {
            *reinterpret_cast<uint32_t*>(xq + item * G + sub * 4) = c;
            if (sub == 0) {
                xd[item] = d;
                gsum[item] = s;
                if (xsT != nullptr) xsT[(item % Kg) * rows + item / Kg] = make_float2(d, s);
            }
        }
    }
}

// The form the group-128 prefill FC runs: only the codes and the transposed (scale, sum) pairs [Kg][rows] that
// its kernels read are written.  A workgroup takes 8 consecutive rows x U consecutive k-groups (a team of 32
// threads per row): a team reads U*512 contiguous bytes and writes U*128 contiguous bytes of codes, and the 8
// teams' pairs of one k-group are 64 contiguous bytes -- with one row per workgroup every pair was an 8-byte
// store into a line of its own, 16 KB from the next.  Codes and scales as in quant_x_rows_kernel.
// GLU: x is [rows, 2*Kg*G], a row holding the gate and the up projection side by side, and what is quantized is
// silu(gate) * up (silu_mul_kernel's expression, so the codes are those of the two launches it replaces).
template <int U, bool GLU = false>
__global__ __launch_bounds__(256) void quant_x_tile128_kernel(const float* __restrict__ x, int rows, int Kg, int kparts,
                                                               int8_t* __restrict__ xq, float* __restrict__ gsum,
                                                               float2* __restrict__ xsT) {
    constexpr int G = 128;
    const int sub = threadIdx.x & 31, team = threadIdx.x >> 5;
    const int rb = blockIdx.x / kparts, kp = blockIdx.x - rb * kparts;
    const int row = rb * 8 + team, kb0 = kp * U;
    const bool row_ok = row < rows;
    const int64_t rbase = (int64_t)(row_ok ? row : rows - 1) * Kg;
    float4 v[U];
    if (GLU) {
        float4 gt[U], up[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const float* p = x + (2 * rbase + min(kb0 + u, Kg - 1)) * G + sub * 4;
            gt[u] = *reinterpret_cast<const float4*>(p);
            up[u] = *reinterpret_cast<const float4*>(p + (int64_t)Kg * G);
        }
#pragma unroll
        for (int u = 0; u < U; u++)
            v[u] = make_float4(silu_times(gt[u].x, up[u].x), silu_times(gt[u].y, up[u].y), silu_times(gt[u].z, up[u].z),
                               silu_times(gt[u].w, up[u].w));
    } else {
#pragma unroll
        for (int u = 0; u < U; u++) v[u] = *reinterpret_cast<const float4*>(x + (rbase + min(kb0 + u, Kg - 1)) * G + sub * 4);
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
        float amax = fmaxf(fmaxf(fabsf(v[u].x), fabsf(v[u].y)), fmaxf(fabsf(v[u].z), fabsf(v[u].w)));
        float s = (v[u].x + v[u].y) + (v[u].z + v[u].w);
#pragma unroll
        for (int o = 16; o > 0; o >>= 1) {
            amax = fmaxf(amax, __shfl_xor(amax, o, 64));
            s += __shfl_xor(s, o, 64);
        }
        const float d = amax / 127.0f;
        const float id = (d != 0.0f) ? (1.0f / d) : 0.0f;
        const uint32_t c = ((uint32_t)q8_code(v[u].x, id) & 0xFFu) | (((uint32_t)q8_code(v[u].y, id) & 0xFFu) << 8) |
                           (((uint32_t)q8_code(v[u].z, id) & 0xFFu) << 16) | (((uint32_t)q8_code(v[u].w, id) & 0xFFu) << 24);
        const int kb = kb0 + u;
        if (row_ok && kb < Kg) {
            *reinterpret_cast<uint32_t*>(xq + (rbase + kb) * G + sub * 4) = c;
            if (sub == 0) {
                xsT[(int64_t)kb * rows + row] = make_float2(d, s);
                gsum[rbase + kb] = s;  // [row][kg] as well: the 256-row product kernel reads a row's sums eight at a time
            }
        }
    }
}

// rmsnorm and the quantization of its result in one pass over the row: one workgroup of 1024 threads per row, the
// row in registers as in rmsnorm_kernel (same statistic, same expression for the normalized value), and the G/4
// neighbouring threads that hold a k-group quantize it as quant_x_rows_kernel does (same reduction tree, same
// codes, scales and sums as rmsnorm_out followed by that kernel).  hidden % G == 0.
template <int VPT, int G>
__global__ __launch_bounds__(1024) void rmsnorm_quant_kernel(const float* __restrict__ x, int64_t hidden,
                                                              const float* __restrict__ w, float eps, int rows, int Kg,
                                                              int8_t* __restrict__ xq, float* __restrict__ xd,
                                                              float* __restrict__ gsum, float2* __restrict__ xsT) {
    constexpr int TPG = G / 4;
    __shared__ float red[16];
    const int row = blockIdx.x;
    float4 v[VPT];
    const float rs = rmsnorm_row_scale<VPT>(x + (int64_t)row * hidden, hidden, eps, v, red);
#pragma unroll
    for (int i = 0; i < VPT; i++) {
        const int64_t e = ((int64_t)i * 1024 + threadIdx.x) * 4;
        const bool live = e < hidden;  // the same for all threads of a team (hidden is a whole number of groups)
        float4 n = make_float4(0.f, 0.f, 0.f, 0.f);
        if (live) {
            const float4 ww = *reinterpret_cast<const float4*>(w + e);
            n = make_float4(v[i].x * rs * ww.x, v[i].y * rs * ww.y, v[i].z * rs * ww.z, v[i].w * rs * ww.w);
        }
        float amax = fmaxf(fmaxf(fabsf(n.x), fabsf(n.y)), fmaxf(fabsf(n.z), fabsf(n.w)));
        float s = (n.x + n.y) + (n.z + n.w);
#pragma unroll
        for (int o = TPG / 2; o > 0; o >>= 1) {
            amax = fmaxf(amax, __shfl_xor(amax, o, 64));
            s += __shfl_xor(s, o, 64);
        }
        const float d = amax / 127.0f;
        const float id = (d != 0.0f) ? (1.0f / d) : 0.0f;
        const uint32_t c = ((uint32_t)q8_code(n.x, id) & 0xFFu) | (((uint32_t)q8_code(n.y, id) & 0xFFu) << 8) |
                           (((uint32_t)q8_code(n.z, id) & 0xFFu) << 16) | (((uint32_t)q8_code(n.w, id) & 0xFFu) << 24);
        if (live) {
            *reinterpret_cast<uint32_t*>(xq + (int64_t)row * hidden + e) = c;
            if ((threadIdx.x % TPG) == 0) {
                const int64_t kb = e / G;
                xd[(int64_t)row * Kg + kb] = d;
                gsum[(int64_t)row * Kg + kb] = s;
                xsT[kb * rows + row] = make_float2(d, s);
            }
        }
    }
}

}  // namespace llmops

using namespace llmops;

namespace llmops {
// Quantization with the producer of the activations folded in (shared with fc.hip): norm_w != nullptr quantizes
// rmsnorm(x) * norm_w, glu_in quantizes silu(gate) * up of rows [gate | up] of 2K floats; one launch instead of the
// producer's launch, a round trip of its fp32 result through memory and the quantization launch.  Whole k-groups
// only; xd is written with norm_w only (the group-128 product kernels read xsT and gsum).
int launch_quant_x_fused(const float* x, int64_t rows, int64_t K, int group_k, const float* norm_w, float eps, bool glu_in,
                         int8_t* xq, float* xd, float* gsum, float2* xsT, hipStream_t stream) {
    const int64_t Kg = K / group_k;
    if (K != Kg * group_k || !aligned(x, 16) || !aligned(xq, 4) || rows >= ((int64_t)1 << 28))
        return fail(LLMOPS_EINVAL, "fused quantization: whole k-groups, 16-byte aligned rows, fewer than 2^28 rows");
    if (norm_w != nullptr) {
        if (glu_in || K > 16384 || !aligned(norm_w, 16))
            return fail(LLMOPS_EINVAL, "fused rmsnorm + quantization: rows of at most 16384 floats, 16-byte aligned weights, no glu");
#define LLMOPS_RQ(VPT)                                                                                                    \
    do {                                                                                                                  \
        if (group_k == 32)                                                                                                \
            rmsnorm_quant_kernel<VPT, 32><<<(unsigned)rows, 1024, 0, stream>>>(x, K, norm_w, eps, (int)rows, (int)Kg, xq, xd, \
                                                                               gsum, xsT);                                \
        else                                                                                                              \
            rmsnorm_quant_kernel<VPT, 128><<<(unsigned)rows, 1024, 0, stream>>>(x, K, norm_w, eps, (int)rows, (int)Kg, xq, xd, \
                                                                                gsum, xsT);                               \
    } while (0)
        if (K <= 4096) LLMOPS_RQ(1);
        else if (K <= 8192) LLMOPS_RQ(2);
        else LLMOPS_RQ(4);
#undef LLMOPS_RQ
        LLMOPS_LAUNCH_CHECK();
        return LLMOPS_OK;
    }
    if (!glu_in) return fail(LLMOPS_EINVAL, "fused quantization without a producer");
    const int64_t rblocks = (rows + 7) / 8;
    if (group_k != 128 || Kg >= ((int64_t)1 << 20) || rblocks * Kg >= ((int64_t)1 << 31))
        return fail(LLMOPS_EINVAL, "fused silu*up + quantization: group 128 only");
    if (rblocks * ((Kg + 3) / 4) >= 1024) {
        const int kparts = (int)((Kg + 3) / 4);
        quant_x_tile128_kernel<4, true><<<(unsigned)(rblocks * kparts), 256, 0, stream>>>(x, (int)rows, (int)Kg, kparts, xq, gsum, xsT);
    } else {
        quant_x_tile128_kernel<1, true><<<(unsigned)(rblocks * Kg), 256, 0, stream>>>(x, (int)rows, (int)Kg, (int)Kg, xq, gsum, xsT);
    }
    LLMOPS_LAUNCH_CHECK();
    return LLMOPS_OK;
}

// shared with fc.hip
int launch_quant_x(const float* x, int64_t rows, int64_t K, int group_k, int8_t* xq, float* xd, float* gsum, float2* xsT,
                   bool exact_sum, hipStream_t stream) {
    const int64_t Kg = (K + group_k - 1) / group_k;
    const int64_t items = rows * Kg;
    if (!exact_sum && xsT != nullptr && group_k == 128 && K == Kg * group_k && aligned(x, 16) && aligned(xq, 4) &&
        rows < ((int64_t)1 << 28) && Kg < ((int64_t)1 << 20) && ((rows + 7) / 8) * Kg < ((int64_t)1 << 31)) {  // (the grid)
        // the group-128 prefill kernels read only the codes, the transposed pairs and the sums: xd stays unwritten
        const int64_t rblocks = (rows + 7) / 8;
        if (rblocks * ((Kg + 3) / 4) >= 1024) {  // enough workgroups with four k-groups per team
            const int kparts = (int)((Kg + 3) / 4);
            quant_x_tile128_kernel<4><<<(unsigned)(rblocks * kparts), 256, 0, stream>>>(x, (int)rows, (int)Kg, kparts, xq, gsum, xsT);
        } else {
            quant_x_tile128_kernel<1><<<(unsigned)(rblocks * Kg), 256, 0, stream>>>(x, (int)rows, (int)Kg, (int)Kg, xq, gsum, xsT);
        }
        LLMOPS_LAUNCH_CHECK();
        return LLMOPS_OK;
    }
    if (!exact_sum && K == Kg * group_k && aligned(x, 16) && aligned(xq, 4)) {  // whole groups only: vector loads
        const int64_t teams = (group_k == 32) ? 32 : 8;  // per workgroup
        if (items >= 32768) {  // enough groups to fill the chip with four per team
            const unsigned grid = (unsigned)((items + teams * 4 - 1) / (teams * 4));
            if (group_k == 32) quant_x_rows_kernel<32, 4><<<grid, 256, 0, stream>>>(x, items, Kg, rows, xq, xd, gsum, xsT);
            else quant_x_rows_kernel<128, 4><<<grid, 256, 0, stream>>>(x, items, Kg, rows, xq, xd, gsum, xsT);
        } else {
            const unsigned grid = (unsigned)((items + teams - 1) / teams);
            if (group_k == 32) quant_x_rows_kernel<32, 1><<<grid, 256, 0, stream>>>(x, items, Kg, rows, xq, xd, gsum, xsT);
            else quant_x_rows_kernel<128, 1><<<grid, 256, 0, stream>>>(x, items, Kg, rows, xq, xd, gsum, xsT);
        }
        LLMOPS_LAUNCH_CHECK();
        return LLMOPS_OK;
    }
    const unsigned grid = (unsigned)((items + 3) / 4);
    if (group_k == 32) {
        if (exact_sum) quant_x_kernel<32, true><<<grid, 256, 0, stream>>>(x, rows, K, Kg, xq, xd, gsum, xsT);
        else quant_x_kernel<32, false><<<grid, 256, 0, stream>>>(x, rows, K, Kg, xq, xd, gsum, xsT);
    } else {
        if (exact_sum) quant_x_kernel<128, true><<<grid, 256, 0, stream>>>(x, rows, K, Kg, xq, xd, gsum, xsT);
        else quant_x_kernel<128, false><<<grid, 256, 0, stream>>>(x, rows, K, Kg, xq, xd, gsum, xsT);
    }
    LLMOPS_LAUNCH_CHECK();
    return LLMOPS_OK;
}
}  // namespace llmops

extern "C" int llmops_FC_dynamic_quantize_x(const float* x, int64_t rows, int64_t K, int group_k, int8_t* xq,
                                            float* xd, float* gsum, llmops_stream_t stream) {
    LLMOPS_REQUIRE(valid_group(group_k));
    LLMOPS_REQUIRE(x != nullptr && xq != nullptr && xd != nullptr && gsum != nullptr);
    LLMOPS_REQUIRE(rows > 0 && K > 0);
    LLMOPS_REQUIRE(aligned(xq, 2));
    const int64_t Kg = (K + group_k - 1) / group_k;
    LLMOPS_REQUIRE(rows * Kg < ((int64_t)1 << 33));
    return launch_quant_x(x, rows, K, group_k, xq, xd, gsum, nullptr, true, as_stream(stream));
}

extern "C" int llmops_FC_dynamic_quantize_x_rows(const float* x, int64_t rows, int64_t K, int group_k, int8_t* xq,
                                                 float* xd, float* gsum, llmops_stream_t stream) {
    LLMOPS_REQUIRE(valid_group(group_k));
    LLMOPS_REQUIRE(x != nullptr && xq != nullptr && xd != nullptr && gsum != nullptr);
    LLMOPS_REQUIRE(rows > 0 && K > 0 && (K % group_k) == 0);
    LLMOPS_REQUIRE(aligned(x, 16) && aligned(xq, 4));
    LLMOPS_REQUIRE(rows * (K / group_k) < ((int64_t)1 << 33));
    return launch_quant_x(x, rows, K, group_k, xq, xd, gsum, nullptr, false, as_stream(stream));
}
