// Device helpers shared by the decode FC kernels: the 16-byte weight "step" of a wavefront, its
// dot4 inner product against int8 activation codes, the fp32 fold of a block's scales, the DPP
// lane exchanges and the in-wave activation quantization (FC_dynamic_quantize_x,
// /root/reference/ops/op_fc.hpp:221-272).
#pragma once
#include "common.h"

namespace llmops {

// weights are read exactly once: non-temporal loads keep them from displacing the activations,
// scales and partial sums that are reused out of the caches
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 ldg16(const uint8_t* p) {
    const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint2 ldg8(const uint8_t* p) { return *reinterpret_cast<const uint2*>(p); }

// ---- lane exchanges on the VALU (DPP), no LDS round trips --------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), CTRL, 0xF, 0xF, false));
}
__device__ __forceinline__ float lane_bcast(float v, int lane) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}
constexpr int kQuadXor1 = 0xB1, kQuadXor2 = 0x4E, kRowHalfMirror = 0x141, kRowMirror = 0x140, kRowRor8 = 0x128;

// max and sum over each row of 16 lanes, result in every lane of the row
__device__ __forceinline__ void row16_max_sum(float& mx, float& sm) {
    mx = fmaxf(mx, dpp<kQuadXor1>(mx));
    sm += dpp<kQuadXor1>(sm);
    mx = fmaxf(mx, dpp<kQuadXor2>(mx));
    sm += dpp<kQuadXor2>(sm);
    mx = fmaxf(mx, dpp<kRowHalfMirror>(mx));
    sm += dpp<kRowHalfMirror>(sm);
    mx = fmaxf(mx, dpp<kRowMirror>(mx));
    sm += dpp<kRowMirror>(sm);
}

// One "step" of a wavefront: G=128 -> one block (two 16 B loads per lane);
//                            G=32  -> two adjacent blocks, one per half-wave (one load per lane).
template <int G>
struct Step {
    static constexpr int kLoads = (G == 128) ? 2 : 1;
    static constexpr int kBlocksPerStep = (G == 128) ? 1 : 2;
    static constexpr int kK = (G == 128) ? 128 : 64;  // k-values per step
    uint4 w[kLoads];
    uint2 dh, mh;  // 4 x fp16 d, 4 x fp16 m of the lane's columns
    bool valid;
};

template <int G>
__device__ __forceinline__ void load_step(Step<G>& st, const uint8_t* strip, int step, int kb_end, int lane) {
    const int quad = lane & 7, rs = lane >> 3;
    if (G == 128) {
        // uniform block address + 32-bit lane offsets: the loads take the (scalar base, vector offset) form
        const uint8_t* blk = strip + (int64_t)step * block_bytes(128);
        const uint32_t wo = (uint32_t)lane * 16u, so = (uint32_t)quad * 8u;
        st.valid = true;
        st.w[0] = ldg16(blk + wo);
        st.w[Step<G>::kLoads - 1] = ldg16(blk + 1024 + wo);
        st.dh = ldg8(blk + 2048 + so);
        st.mh = ldg8(blk + 2048 + 64 + so);
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

// The same group-128 step through a buffer descriptor: scalar base (the strip), scalar offset (the block)
// and one 32-bit lane offset, so that a loop over blocks keeps no 64-bit addresses in vector registers.
// Reads past the descriptor's size return 0.
typedef __amdgpu_buffer_rsrc_t buffer_rsrc;
__device__ __forceinline__ buffer_rsrc make_rsrc(const void* base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}
// weights: non-temporal (cache policy bit 1)
__device__ __forceinline__ uint4 buf_ldg16_nt(buffer_rsrc r, uint32_t voff, uint32_t soff) {
    const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 2);
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint2 buf_ldg8(buffer_rsrc r, uint32_t voff, uint32_t soff) {
    typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
    const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(r, voff, soff, 0);
    return make_uint2(v.x, v.y);
}
__device__ __forceinline__ float4 buf_ldf4(buffer_rsrc r, uint32_t voff, uint32_t soff) {
    const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 0);
    return make_float4(__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w));
}
__device__ __forceinline__ float buf_ldf1(buffer_rsrc r, uint32_t voff, uint32_t soff) {
    return __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0));
}
// A lane offset no descriptor covers: the load returns 0 without touching memory.  Loads that are not
// wanted are issued with it instead of being branched around: the hardware counts outstanding loads
// in issue order, and only a wave whose every path issues the same loads can wait for exactly the one
// it needs (a branch around a younger load makes the compiler wait for all of them).
constexpr uint32_t kNoLoad = 0xFFFFFF00u;
__device__ __forceinline__ void load_step_buf(Step<128>& st, buffer_rsrc strip, int step, int lane, bool wanted = true) {
    const uint32_t so = (uint32_t)step * (uint32_t)block_bytes(128);
    const uint32_t wo = wanted ? (uint32_t)lane * 16u : kNoLoad, qo = wanted ? (uint32_t)(lane & 7) * 8u : kNoLoad;
    st.valid = true;
    // constant parts go to the scalar offset: the lane offsets stay two registers for the whole loop
    st.w[0] = buf_ldg16_nt(strip, wo, so);
    st.w[1] = buf_ldg16_nt(strip, wo, so + 1024u);
    st.dh = buf_ldg8(strip, qo, so + 2048u);
    st.mh = buf_ldg8(strip, qo, so + 2048u + 64u);
}

// A group-32 step (two adjacent blocks, lane = rs*8 + quad, rs>>2 = block of the step, rs&3 = k8-row)
// through a buffer descriptor.  A block past the strip's last (odd block count) or an unwanted step is
// asked for at kNoLoad: zeros, which add nothing.
__device__ __forceinline__ void load_step_buf(Step<32>& st, buffer_rsrc strip, int step, int kb_end, int lane, bool wanted = true) {
    const int rs = lane >> 3, quad = lane & 7;
    const bool ok = wanted && step * 2 + (rs >> 2) < kb_end;
    const uint32_t so = (uint32_t)step * 2u * (uint32_t)block_bytes(32);
    const uint32_t bo = (uint32_t)(rs >> 2) * (uint32_t)block_bytes(32);
    const uint32_t wo = ok ? bo + (uint32_t)(rs & 3) * kRowBytes + (uint32_t)quad * 16u : kNoLoad;
    const uint32_t qo = ok ? bo + (uint32_t)quad * 8u : kNoLoad;
    st.valid = true;
    st.w[0] = buf_ldg16_nt(strip, wo, so);
    st.dh = buf_ldg8(strip, qo, so + 512u);
    st.mh = buf_ldg8(strip, qo, so + 512u + 64u);
}

// int32 partial dot products of the lane's 4 columns over the lane's k8-rows of this step;
// `codes` points at the step's activation codes (Step<G>::kK of them)
template <int G>
__device__ __forceinline__ void dot_step(const Step<G>& st, const int8_t* codes, int lane, int acc[4]) {
    const int rs = lane >> 3;
    const int2 xa = *reinterpret_cast<const int2*>(codes + rs * 8);
    const uint32_t* w0 = reinterpret_cast<const uint32_t*>(&st.w[0]);
#pragma unroll
    for (int j = 0; j < 4; j++) acc[j] = dot8_q4(w0[j], xa.x, xa.y, 0);
    if (G == 128) {
        const int2 xb = *reinterpret_cast<const int2*>(codes + 64 + rs * 8);
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

// The lane id computed on the spot (2 instructions) instead of kept in a register since the kernel began:
// the epilogue of a kernel that is short of registers in its main loop uses this.
__device__ __forceinline__ int lane_id_now() {
    int l;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(l));
    return l;
}

// f[r][j] += d*(dx*acc) + m*gsum for the lane's 4 columns (d and m enter the fused multiply-adds as
// fp16 operands: no separate conversions)
__device__ __forceinline__ void fold(float f[4], const int acc[4], uint2 dh, uint2 mh, float dx, float g) {
    float d[4], m[4];
    unpack_h4(dh, d);
    unpack_h4(mh, m);
#pragma unroll
    for (int j = 0; j < 4; j++) {
        f[j] = fmaf(d[j], dx * (float)acc[j], f[j]);
        f[j] = fmaf(m[j], g, f[j]);
    }
}

// Sum over the 8 row slots of a wave (lane bits 3, 4, 5), result in every lane: one DPP-fused add inside the
// rows of 16 lanes, then the rows pairwise (v_permlane16_swap) and the wave's halves (v_permlane32_swap).
__device__ __forceinline__ void rowslot_sum4(float f[4]) {
    asm("s_nop 1\n\t"
        "v_add_f32_dpp %0, %0, %0 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
        "v_add_f32_dpp %1, %1, %1 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
        "v_add_f32_dpp %2, %2, %2 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
        "v_add_f32_dpp %3, %3, %3 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1"
        : "+v"(f[0]), "+v"(f[1]), "+v"(f[2]), "+v"(f[3]));
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(f[j]), __float_as_uint(f[j]), false, false);
        const float v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
        const auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
        f[j] = __uint_as_float(b[0]) + __uint_as_float(b[1]);
    }
}

// ---- raw fp32 activations, quantized by the wavefront that consumes them ---------------------
template <int G>
struct XRaw {
    float v[(G == 128) ? 2 : 1];
};

template <int G>
__device__ __forceinline__ void load_x(XRaw<G>& xr, const float* xrow, int step, int64_t K, int lane) {
    if (G == 128) {
        const float2 t = *reinterpret_cast<const float2*>(xrow + (int64_t)step * 128 + lane * 2);
        xr.v[0] = t.x;
        xr.v[(G == 128) ? 1 : 0] = t.y;
    } else {
        const int64_t k = (int64_t)step * 64 + lane;
        xr.v[0] = k < K ? xrow[k] : 0.0f;
    }
}

__device__ __forceinline__ int q8_code_rne(float v, float id) {
    const float t = v * id;
    if (t != t) return -128;  // what the reference's cvtps2dq + saturating packs give for NaN
    return (int)fminf(127.0f, fmaxf(-128.0f, rintf(t)));
}

// Per-step record in LDS: the step's int8 codes followed by (dx, gsum) per block of the step
template <int G>
struct XSlot {
    int8_t codes[Step<G>::kK];
    float2 scale[Step<G>::kBlocksPerStep];
};

// The same for a pass of 256 k-values quantized at once: two blocks of group 128 or eight of group 32
struct XPairSlot {
    int8_t codes[256];
    float2 scale[8];
};

// FC_dynamic_quantize_x for one step (/root/reference/ops/op_fc.hpp:246-268): amax -> d = amax/127 ->
// id = 1/d -> RNE codes; raw sum of the group
template <int G>
__device__ __forceinline__ void quantize_step(const XRaw<G>& xr, XSlot<G>* slot, int lane) {
    if (G == 128) {
        float amax = fmaxf(fabsf(xr.v[0]), fabsf(xr.v[(G == 128) ? 1 : 0]));
        float sum = xr.v[0] + xr.v[(G == 128) ? 1 : 0];
        row16_max_sum(amax, sum);
        amax = fmaxf(fmaxf(lane_bcast(amax, 0), lane_bcast(amax, 16)), fmaxf(lane_bcast(amax, 32), lane_bcast(amax, 48)));
        sum = (lane_bcast(sum, 0) + lane_bcast(sum, 16)) + (lane_bcast(sum, 32) + lane_bcast(sum, 48));
        const float d = amax / 127.0f;
        const float id = (d != 0.0f) ? (1.0f / d) : 0.0f;
        const uint32_t c0 = (uint32_t)q8_code_rne(xr.v[0], id) & 0xFFu;
        const uint32_t c1 = (uint32_t)q8_code_rne(xr.v[(G == 128) ? 1 : 0], id) & 0xFFu;
        *reinterpret_cast<uint16_t*>(&slot->codes[lane * 2]) = (uint16_t)(c0 | (c1 << 8));
        if (lane == 0) slot->scale[0] = make_float2(d, sum);
    } else {
        float amax = fabsf(xr.v[0]);
        float sum = xr.v[0];
        row16_max_sum(amax, sum);
        // the two half-waves hold two different groups
        const float a_lo = fmaxf(lane_bcast(amax, 0), lane_bcast(amax, 16)), a_hi = fmaxf(lane_bcast(amax, 32), lane_bcast(amax, 48));
        const float s_lo = lane_bcast(sum, 0) + lane_bcast(sum, 16), s_hi = lane_bcast(sum, 32) + lane_bcast(sum, 48);
        const bool hi = lane >= 32;
        const float d = (hi ? a_hi : a_lo) / 127.0f;
        const float id = (d != 0.0f) ? (1.0f / d) : 0.0f;
        slot->codes[lane] = (int8_t)q8_code_rne(xr.v[0], id);
        if ((lane & 31) == 0) slot->scale[(G == 128) ? 0 : (lane >> 5)] = make_float2(d, hi ? s_hi : s_lo);
    }
}

// max and sum over each row of 16 lanes with the lane exchange folded into the arithmetic instruction
// (one instruction per level and quantity).  A DPP operand must not be read within two wait states of
// the instruction that wrote it: the two chains alternate and an s_nop fills the remaining slot.
__device__ __forceinline__ void row16_max_sum_fused(float& mx, float& sm) {
    asm("s_nop 1\n\t"
        "v_max_f32_dpp %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
        "v_add_f32_dpp %1, %1, %1 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 0\n\t"
        "v_max_f32_dpp %0, %0, %0 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
        "v_add_f32_dpp %1, %1, %1 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 0\n\t"
        "v_max_f32_dpp %0, %0, %0 row_half_mirror row_mask:0xf bank_mask:0xf\n\t"
        "v_add_f32_dpp %1, %1, %1 row_half_mirror row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 0\n\t"
        "v_max_f32_dpp %0, %0, %0 row_mirror row_mask:0xf bank_mask:0xf\n\t"
        "v_add_f32_dpp %1, %1, %1 row_mirror row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1"
        : "+v"(mx), "+v"(sm));
}

// The same for two groups of 128 at once: lanes 0-31 hold the first group (four consecutive values per
// lane), lanes 32-63 the second.  Same operations per value as the reference (amax -> d = amax/127 ->
// id = 1/d -> round to nearest even, clamp), written for instruction count: the rows of 16 lanes are
// combined pairwise with v_permlane16_swap, rounding and conversion are one addition of 1.5*2^23 (whose
// low byte is then the two's-complement code), four codes are packed with two byte permutes.  The raw
// group sum is a tree sum.
__device__ __forceinline__ void quantize_pair(const float4& v, XPairSlot* slot, int lane) {
    float amax;
    float sum = (v.x + v.y) + (v.z + v.w);
    asm("v_max3_f32 %0, |%1|, |%2|, |%3|\n\t"
        "v_max_f32_e64 %0, %0, |%4|"
        : "=&v"(amax)
        : "v"(v.x), "v"(v.y), "v"(v.z), "v"(v.w));
    row16_max_sum_fused(amax, sum);
    // rows (0,1) -> lanes 0-31, rows (2,3) -> lanes 32-63: after the swap one register holds rows
    // [0,0,2,2] and the other [1,1,3,3]
    const auto ra = __builtin_amdgcn_permlane16_swap(__float_as_uint(amax), __float_as_uint(amax), false, false);
    const auto rs = __builtin_amdgcn_permlane16_swap(__float_as_uint(sum), __float_as_uint(sum), false, false);
    amax = __uint_as_float(ra[0] > ra[1] ? ra[0] : ra[1]);  // non-negative floats order like their bit patterns
    sum = __uint_as_float(rs[0]) + __uint_as_float(rs[1]);
    const float d = amax / 127.0f;
    const float id = (d != 0.0f) ? (1.0f / d) : 0.0f;
    constexpr float kRound = 12582912.0f;  // 1.5 * 2^23
    const uint32_t u0 = __float_as_uint(__builtin_amdgcn_fmed3f(v.x * id, -128.0f, 127.0f) + kRound);
    const uint32_t u1 = __float_as_uint(__builtin_amdgcn_fmed3f(v.y * id, -128.0f, 127.0f) + kRound);
    const uint32_t u2 = __float_as_uint(__builtin_amdgcn_fmed3f(v.z * id, -128.0f, 127.0f) + kRound);
    const uint32_t u3 = __float_as_uint(__builtin_amdgcn_fmed3f(v.w * id, -128.0f, 127.0f) + kRound);
    const uint32_t lo = __builtin_amdgcn_perm(u1, u0, 0x0c0c0400u), hi = __builtin_amdgcn_perm(u3, u2, 0x04000c0cu);
    *reinterpret_cast<uint32_t*>(&slot->codes[lane * 4]) = lo | hi;
    slot->scale[lane >> 5] = make_float2(d, sum);  // every lane of the half writes the same pair
}

// Eight groups of 32 at once (group g = lanes 8g..8g+7, four consecutive values per lane): the same
// operations per value; the reduction stays inside the 8 lanes of a group (three DPP levels).
__device__ __forceinline__ void quantize_pass32(const float4& v, XPairSlot* slot, int lane) {
    float amax;
    float sum = (v.x + v.y) + (v.z + v.w);
    asm("v_max3_f32 %0, |%1|, |%2|, |%3|\n\t"
        "v_max_f32_e64 %0, %0, |%4|"
        : "=&v"(amax)
        : "v"(v.x), "v"(v.y), "v"(v.z), "v"(v.w));
    asm("s_nop 1\n\t"
        "v_max_f32_dpp %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
        "v_add_f32_dpp %1, %1, %1 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 0\n\t"
        "v_max_f32_dpp %0, %0, %0 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
        "v_add_f32_dpp %1, %1, %1 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 0\n\t"
        "v_max_f32_dpp %0, %0, %0 row_half_mirror row_mask:0xf bank_mask:0xf\n\t"
        "v_add_f32_dpp %1, %1, %1 row_half_mirror row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1"
        : "+v"(amax), "+v"(sum));
    const float d = amax / 127.0f;
    const float id = (d != 0.0f) ? (1.0f / d) : 0.0f;
    constexpr float kRound = 12582912.0f;  // 1.5 * 2^23
    const uint32_t u0 = __float_as_uint(__builtin_amdgcn_fmed3f(v.x * id, -128.0f, 127.0f) + kRound);
    const uint32_t u1 = __float_as_uint(__builtin_amdgcn_fmed3f(v.y * id, -128.0f, 127.0f) + kRound);
    const uint32_t u2 = __float_as_uint(__builtin_amdgcn_fmed3f(v.z * id, -128.0f, 127.0f) + kRound);
    const uint32_t u3 = __float_as_uint(__builtin_amdgcn_fmed3f(v.w * id, -128.0f, 127.0f) + kRound);
    const uint32_t lo = __builtin_amdgcn_perm(u1, u0, 0x0c0c0400u), hi = __builtin_amdgcn_perm(u3, u2, 0x04000c0cu);
    *reinterpret_cast<uint32_t*>(&slot->codes[lane * 4]) = lo | hi;
    slot->scale[lane >> 3] = make_float2(d, sum);  // every lane of the group writes the same pair
}

__device__ __forceinline__ float wave_sum_dpp(float v) {
    asm("s_nop 1\n\t"
        "v_add_f32_dpp %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_add_f32_dpp %0, %0, %0 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_add_f32_dpp %0, %0, %0 row_half_mirror row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_add_f32_dpp %0, %0, %0 row_mirror row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1"
        : "+v"(v));
    return (lane_bcast(v, 0) + lane_bcast(v, 16)) + (lane_bcast(v, 32) + lane_bcast(v, 48));
}

}  // namespace llmops
