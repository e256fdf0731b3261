// Shared host/device helpers for the gfx950 llmops kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include <cstdarg>
#include <cstdio>
#include <string>

#include "../../include/llmops_hip.h"
#include "../../include/llmops_hip_test.h"

namespace llmops {

constexpr int kGroupN = 32;   // columns per packed strip (q4_1_block::group_n, ops/op_fc.hpp:17)
constexpr int kRowBytes = 128;  // one k8-row of a block: 32 columns x 4 bytes
// zeroed head of the FC workspace (LLMOPS_FC_COUNTER_BYTES): arrival counters of the k-splits, one per
// strip, then the exchange slots of the two-split hand-off
constexpr int kTicketBytes = 65536;

__host__ __device__ constexpr int64_t block_bytes(int G) { return (int64_t)(G / 8) * kRowBytes + 64 + 64; }

// where the dump build of the decode FC kernel stores what it quantized and its int32 sums
struct DumpBufs {
    int8_t* xq;    // [rows][Kg*G]
    float* xd;     // [rows][Kg]
    float* gs;     // [rows][Kg]
    int32_t* acc;  // [rows][Ng*32][Kg]
};

// ---- error reporting ------------------------------------------------------------------------
std::string& last_error();
int fail(int code, const char* fmt, ...);
// true if the process was started with LLMOPS_TEST_HOOKS=1; otherwise records why `hook` was refused (and says so
// once on stderr) and returns false
bool test_hooks_enabled(const char* hook);
#define LLMOPS_TEST_HOOK()                                                                            \
    do {                                                                                            \
        if (!::llmops::test_hooks_enabled(__func__)) return LLMOPS_EINVAL;                          \
    } while (0)

#define LLMOPS_REQUIRE(cond)                                                                        \
    do {                                                                                            \
        if (!(cond)) return ::llmops::fail(LLMOPS_EINVAL, "assert %s failed at %s:%d", #cond, __FILE__, __LINE__); \
    } while (0)

#define LLMOPS_HIP_CHECK(expr)                                                                      \
    do {                                                                                            \
        hipError_t e_ = (expr);                                                                     \
        if (e_ != hipSuccess)                                                                       \
            return ::llmops::fail(LLMOPS_EHIP, "%s failed: %s at %s:%d", #expr, hipGetErrorString(e_), __FILE__, __LINE__); \
    } while (0)

#define LLMOPS_LAUNCH_CHECK() LLMOPS_HIP_CHECK(hipGetLastError())

inline hipStream_t as_stream(llmops_stream_t s) { return reinterpret_cast<hipStream_t>(s); }
inline bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }
inline bool valid_group(int g) { return g == 32 || g == 128; }

// ---- device helpers -------------------------------------------------------------------------
#if defined(__HIPCC__)

// fp16 bits <-> fp32, IEEE round-to-nearest-even (v_cvt_f16_f32 / v_cvt_f32_f16)
__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) { return __half_as_ushort(__float2half_rn(f)); }
__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) { return __half2float(__ushort_as_half(h)); }

// signed 4 x int8 dot product with int32 accumulate (v_dot4_i32_i8)
__device__ __forceinline__ int dot4(int a, int b, int c) { return __builtin_amdgcn_sdot4(a, b, c, false); }

// 8 packed 4-bit codes in one dword (low nibbles = k 0..3, high nibbles = k 4..7 of one column)
// against 8 int8 activation codes (xlo = k 0..3, xhi = k 4..7)
__device__ __forceinline__ int dot8_q4(uint32_t w, int xlo, int xhi, int acc) {
    acc = dot4((int)(w & 0x0F0F0F0Fu), xlo, acc);
    acc = dot4((int)((w >> 4) & 0x0F0F0F0Fu), xhi, acc);
    return acc;
}

// silu(gate) * up (itrans "silu" + imul, ops/op_misc.hpp:83-138) as every fused form of it computes it:
// the sigmoid's reciprocal is the hardware's (1 ulp) rather than an IEEE division -- the reference's own
// uses the 12-bit rcpps (ops/utils.hpp:373-378) -- and all fused forms share this one expression so that
// they agree bit for bit.
__device__ __forceinline__ float silu_times(float gate, float up) {
    return up * (gate * __builtin_amdgcn_rcpf(1.0f + expf(-gate)));
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// rmsnorm's scale 1/sqrt(mean(x^2) + eps) of one row, computed by a workgroup of 1024 threads that keeps the
// row in registers (v[i] = floats 4*(1024*i + thread) .. +3, zeros beyond the row).  Every kernel that
// normalizes whole rows goes through this one function, so that they agree bit for bit.  red: 16 floats of LDS.
template <int VPT>
__device__ __forceinline__ float rmsnorm_row_scale(const float* __restrict__ row, int64_t hidden, float eps, float4 (&v)[VPT],
                                                   float* red) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float ss = 0.0f;
#pragma unroll
    for (int i = 0; i < VPT; i++) {
        const int64_t e = ((int64_t)i * 1024 + threadIdx.x) * 4;
        v[i] = e < hidden ? *reinterpret_cast<const float4*>(row + e) : make_float4(0.f, 0.f, 0.f, 0.f);
        ss = fmaf(v[i].x, v[i].x, ss);
        ss = fmaf(v[i].y, v[i].y, ss);
        ss = fmaf(v[i].z, v[i].z, ss);
        ss = fmaf(v[i].w, v[i].w, ss);
    }
    ss = wave_sum(ss);
    if (lane == 0) red[wave] = ss;
    __syncthreads();
    float tot = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; i++) tot += red[i];
    return 1.0f / sqrtf(tot / (float)hidden + eps);
}

#endif  // __HIPCC__

}  // namespace llmops
