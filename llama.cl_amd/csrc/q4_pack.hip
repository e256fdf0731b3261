// Q4_1 weight packing and unpacking on the device.
//
// One workgroup builds one packed block (32 columns x G k-values): thread (ni, r) owns the 8
// consecutive k-values 8r..8r+7 of column ni, i.e. exactly one dword of the block's nibble area
// (low nibbles = k 8r..8r+3, high nibbles = k 8r+4..8r+7).  The G/8 threads of a column sit in
// adjacent lanes, so the per-column min/max is a short xor-shuffle reduction.
//
// Arithmetic follows offline_FC_quant_Q4A (/root/reference/ops/op_fc.hpp:151-219) operation for
// operation so the packed bytes are identical: d=(max-min)/15, id=1/d (IEEE division), code =
// clamp(roundf((w-m)*id),0,15) with the *unrounded* fp32 d and m, and d, m stored as RNE fp16.
#include "common.h"

namespace llmops {

// min/max with the reference's "first occurrence wins" behaviour on equal values
// (get_min_max, ops/op_fc.hpp:112-122, compares strictly), which decides the sign of a zero.
template <int R>
__device__ __forceinline__ void column_min_max(float& vmin, float& vmax) {
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int o = 1; o < R; o <<= 1) {
        const float omin = __shfl_xor(vmin, o, 64);
        const float omax = __shfl_xor(vmax, o, 64);
        const bool partner_first = (lane ^ o) < lane;  // partner holds lower k
        if (omin < vmin || (omin == vmin && partner_first)) vmin = omin;
        if (omax > vmax || (omax == vmax && partner_first)) vmax = omax;
    }
}

template <int G>
__global__ __launch_bounds__(32 * (G / 8)) void quant_w_kernel(const float* __restrict__ wei, int64_t N, int64_t K,
                                                                int64_t ld, uint8_t* __restrict__ out, int64_t Kg) {
    constexpr int R = G / 8;
    const int kb = blockIdx.x, nb = blockIdx.y;
    const int r = threadIdx.x % R, ni = threadIdx.x / R;
    const int64_t n = (int64_t)nb * kGroupN + ni;
    const int64_t k0 = (int64_t)kb * G + r * 8;
    uint8_t* blk = out + ((int64_t)nb * Kg + kb) * block_bytes(G);
    const bool row_ok = n < N;

    float v[8];
    float vmin = __builtin_inff(), vmax = -__builtin_inff();
    bool first = true;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        v[j] = 0.0f;
        if (row_ok && k0 + j < K) {
            const float a = wei[n * ld + k0 + j];
            v[j] = a;
            if (first) {
                vmin = vmax = a;
                first = false;
            } else {
                if (vmax < a) vmax = a;
                if (vmin > a) vmin = a;
            }
        }
    }
    column_min_max<R>(vmin, vmax);

    uint32_t packed = 0;
    float d = 0.0f, m = 0.0f;
    if (row_ok) {
        d = (vmax - vmin) / 15.0f;
        m = vmin;
        const float id = (d != 0.0f) ? (1.0f / d) : 0.0f;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            uint32_t q = 0;
            if (k0 + j < K) {
                float t = roundf((v[j] - m) * id);  // half away from zero
                t = fminf(15.0f, fmaxf(t, 0.0f));
                q = (uint32_t)(int)t;
            }
            packed |= q << ((j & 3) * 8 + (j >> 2) * 4);
        }
    }
    *reinterpret_cast<uint32_t*>(blk + r * kRowBytes + ni * 4) = packed;
    if (r == 0) {
        uint16_t* wd = reinterpret_cast<uint16_t*>(blk + R * kRowBytes);
        wd[ni] = row_ok ? f32_to_f16_bits(d) : (uint16_t)0;
        wd[32 + ni] = row_ok ? f32_to_f16_bits(m) : (uint16_t)0;
    }
}

// out[n, k] = fp32(d)*q + fp32(m) (q4_1_block::get, ops/op_fc.hpp:49-61).  d has 11 significant
// bits and q 4, so the product is exact and contraction cannot change the result.
template <int G>
__global__ __launch_bounds__(32 * (G / 8)) void dequant_w_kernel(const uint8_t* __restrict__ weiq, int64_t Kg,
                                                                  float* __restrict__ out) {
    constexpr int R = G / 8;
    const int kb = blockIdx.x, nb = blockIdx.y;
    const int r = threadIdx.x % R, ni = threadIdx.x / R;
    const uint8_t* blk = weiq + ((int64_t)nb * Kg + kb) * block_bytes(G);
    const uint32_t w = *reinterpret_cast<const uint32_t*>(blk + r * kRowBytes + ni * 4);
    const uint16_t* wd = reinterpret_cast<const uint16_t*>(blk + R * kRowBytes);
    const float d = f16_bits_to_f32(wd[ni]);
    const float m = f16_bits_to_f32(wd[32 + ni]);
    float o[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const uint32_t q = (w >> ((j & 3) * 8 + (j >> 2) * 4)) & 0xFu;
        o[j] = d * (float)q + m;
    }
    float* dst = out + ((int64_t)nb * kGroupN + ni) * (Kg * G) + (int64_t)kb * G + r * 8;
    *reinterpret_cast<float4*>(dst) = make_float4(o[0], o[1], o[2], o[3]);
    *reinterpret_cast<float4*>(dst + 4) = make_float4(o[4], o[5], o[6], o[7]);
}

}  // namespace llmops

using namespace llmops;

extern "C" int64_t llmops_q4a_block_bytes(int group_k) { return valid_group(group_k) ? block_bytes(group_k) : 0; }

extern "C" int llmops_offline_FC_quant_Q4A(const float* wei, int64_t N, int64_t K, int64_t ld, int group_k,
                                           int8_t* weiq, llmops_stream_t stream) {
    LLMOPS_REQUIRE(valid_group(group_k));
    LLMOPS_REQUIRE(wei != nullptr && weiq != nullptr);
    LLMOPS_REQUIRE(N > 0 && K > 0 && ld >= K);
    LLMOPS_REQUIRE(aligned(weiq, 4));
    const int64_t Ng = (N + kGroupN - 1) / kGroupN, Kg = (K + group_k - 1) / group_k;
    LLMOPS_REQUIRE(Ng <= 65535 && Kg <= 0x7fffffff);
    dim3 grid((unsigned)Kg, (unsigned)Ng);
    uint8_t* out = reinterpret_cast<uint8_t*>(weiq);
    if (group_k == 32)
        quant_w_kernel<32><<<grid, 32 * 4, 0, as_stream(stream)>>>(wei, N, K, ld, out, Kg);
    else
        quant_w_kernel<128><<<grid, 32 * 16, 0, as_stream(stream)>>>(wei, N, K, ld, out, Kg);
    LLMOPS_LAUNCH_CHECK();
    return LLMOPS_OK;
}

extern "C" int llmops_offline_FC_dequant_Q4A(const int8_t* weiq, int64_t Ng, int64_t Kg, int group_k, float* out,
                                             llmops_stream_t stream) {
    LLMOPS_REQUIRE(valid_group(group_k));
    LLMOPS_REQUIRE(weiq != nullptr && out != nullptr);
    LLMOPS_REQUIRE(Ng > 0 && Kg > 0 && Ng <= 65535);
    LLMOPS_REQUIRE(aligned(weiq, 4) && aligned(out, 16));
    dim3 grid((unsigned)Kg, (unsigned)Ng);
    const uint8_t* in = reinterpret_cast<const uint8_t*>(weiq);
    if (group_k == 32)
        dequant_w_kernel<32><<<grid, 32 * 4, 0, as_stream(stream)>>>(in, Kg, out);
    else
        dequant_w_kernel<128><<<grid, 32 * 16, 0, as_stream(stream)>>>(in, Kg, out);
    LLMOPS_LAUNCH_CHECK();
    return LLMOPS_OK;
}
