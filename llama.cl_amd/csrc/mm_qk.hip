// Scaled query x key product over a KV cache: attn_w[b,h,pq,pk] = (q[b,h,pq,:] . k[b,h,pk,:]) / sqrt(S).
//
// The reference exports this product four times under benchmark names (mm_qk, mm_qk42, mm_qk81, mm_qk24:
// ops/op_attn.hpp:149-193, 195-298, 300-422, 424-515; bound at ops/main.cpp:163-166).  The four differ
// only in how the AVX loops are blocked; their results are the same product, so one kernel serves all.
//
// One workgroup = 4 wavefronts = 32 queries x 128 cache rows of one (batch, head); each wave owns a
// 32 x 32 tile of the output and walks S with v_mfma_f32_32x32x2_f32.  The matrix instruction takes, per
// lane, one A value (row = lane % 32, k = lane / 32) and one B value (column = lane % 32, k = lane / 32).
// Which s-index a k-slot stands for is free as long as A and B agree, so a lane reads its row in 16-byte
// pieces: piece j of lane-half h covers s = 8j + 4h .. 8j + 4h + 3, and the four multiplies of a piece pair
// take its four components.  Every byte of a 128-byte line a wave touches is used by that wave.
#include "common.h"

namespace llmops {

typedef float f32x16 __attribute__((ext_vector_type(16)));

__global__ __launch_bounds__(256) void mm_qk_kernel(const float* __restrict__ q, int64_t qs_b, int64_t qs_h, int64_t qs_q,
                                                    const float* __restrict__ kc, int64_t kmax, float* __restrict__ w,
                                                    int H, int qL, int kvLen, int S, float scale) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 31, hf = lane >> 5;
    const int bh = blockIdx.z, b = bh / H, h = bh - b * H;
    const int pq0 = blockIdx.y * 32, pk0 = blockIdx.x * 128 + wave * 32;
    if (pk0 >= kvLen) return;  // wave-uniform; no barrier follows
    // rows past the end are read from the last valid row and never stored
    const int pq = min(pq0 + r, qL - 1), pk = min(pk0 + r, kvLen - 1);
    const float4* qp = reinterpret_cast<const float4*>(q + b * qs_b + h * qs_h + (int64_t)pq * qs_q) + hf;
    const float4* kp = reinterpret_cast<const float4*>(kc + ((int64_t)bh * kmax + pk) * S) + hf;
    f32x16 acc = {0};
    const int pieces = S >> 3;
#pragma unroll 4
    for (int j = 0; j < pieces; j++) {
        const float4 a = qp[2 * j], c = kp[2 * j];
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, c.x, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, c.y, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.z, c.z, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.w, c.w, acc, 0, 0, 0);
    }
    // result layout: lane holds column lane % 32, rows 8g + 4(lane / 32) + i in acc[4g + i]
    const int col = pk0 + r;
    if (col < kvLen) {
        float* wp = w + ((int64_t)bh * qL) * kvLen + col;
#pragma unroll
        for (int g = 0; g < 4; g++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int row = pq0 + 8 * g + 4 * hf + i;
                if (row < qL) wp[(int64_t)row * kvLen] = acc[4 * g + i] * scale;
            }
    }
}

}  // namespace llmops

using namespace llmops;

extern "C" int llmops_mm_qk(const float* q, int64_t q_stride_b, int64_t q_stride_h, int64_t q_stride_q, const float* kcache,
                            int64_t kv_max, float* attn_w, int64_t B, int64_t H, int64_t qL, int64_t kvLen, int64_t S,
                            llmops_stream_t stream) {
    LLMOPS_REQUIRE(q != nullptr && kcache != nullptr && attn_w != nullptr);
    LLMOPS_REQUIRE(B > 0 && H > 0 && qL > 0 && kvLen > 0 && kvLen <= kv_max);
    LLMOPS_REQUIRE(S > 0 && (S % 8) == 0);  // ops/op_attn.hpp:205
    LLMOPS_REQUIRE(aligned(q, 16) && aligned(kcache, 16));
    LLMOPS_REQUIRE((q_stride_b % 4) == 0 && (q_stride_h % 4) == 0 && (q_stride_q % 4) == 0);
    LLMOPS_REQUIRE(B * H < 65536 && (qL + 31) / 32 < 65536 && qL < ((int64_t)1 << 31) && kvLen < ((int64_t)1 << 31) - 128);
    dim3 grid((unsigned)((kvLen + 127) / 128), (unsigned)((qL + 31) / 32), (unsigned)(B * H));
    mm_qk_kernel<<<grid, 256, 0, as_stream(stream)>>>(q, q_stride_b, q_stride_h, q_stride_q, kcache, kv_max, attn_w, (int)H,
                                                      (int)qL, (int)kvLen, (int)S, 1.0f / sqrtf((float)S));
    LLMOPS_LAUNCH_CHECK();
    return LLMOPS_OK;
}
