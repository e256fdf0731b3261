// Rotary embedding, KV-cache update and attention over the cache
// (attention_rope2 / attention_rope, /root/reference/ops/op_attn.hpp:721-1029 and :518-718).
//
// Three launches per call:
//   1. attn_prep_kernel   rotate q and k in place (rope_embed, ops/op_attn.hpp:44-94), write the
//                         rotated k and the v rows into the cache at slots[p] (:764-773), and
//                         record which cache rows were written by which token of this call.
//   2. attn_split_kernel  split-KV attention: one workgroup per (b, h, query, chunk of C cache
//                         rows) streams its K and V rows exactly once with 16-byte loads (all
//                         issued before the first use so a whole chunk is in flight), computes
//                         the chunk's scores, their max, exp and sum, and the chunk's weighted
//                         V sum.  Chunks make up for the low head count (B*H = 32 in decode).
//   3. attn_merge_kernel  merges the chunks of a query with the usual max/sum rescaling and
//                         overwrites q with the result (:1018-1025).
// The cache element type is fp32 (reference layout) or fp16 (all arithmetic still fp32).
//
// In-chunk causal mask (:1007-1011): for query token pq, cache row slots[p'] is excluded for
// every p' in (pq, qL).  Excluded rows get weight exactly 0, as the reference's exp() returns 0
// for lowest()-max.
#include <float.h>
#include <limits.h>

#include "common.h"

namespace llmops {

// ---- rope ------------------------------------------------------------------------------------
// theta = inv_freq[i] * (float)pos, cosf/sinf in fp32 (CosSin_cache::update, ops/op_attn.hpp:25-32)
__device__ __forceinline__ void rope_pair(float& x0, float& x1, float inv_freq, int pos) {
    const float xita = inv_freq * (float)pos;
    const float c = cosf(xita), s = sinf(xita);
    const float y0 = c * x0 - s * x1;
    const float y1 = s * x0 + c * x1;
    x0 = y0;
    x1 = y1;
}

// x [B,H,L,S] in place; one thread per rotated pair
__global__ void rope_kernel(float* __restrict__ x, int64_t BH, int64_t L, int64_t S, const float* __restrict__ inv_freq,
                            int64_t half, int position_id) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= BH * L * half) return;
    const int64_t p = i % half, l = (i / half) % L, bh = i / (half * L);
    float* px = x + (bh * L + l) * S;
    float x0 = px[p], x1 = px[p + half];
    rope_pair(x0, x1, inv_freq[p], (int)l + position_id);
    px[p] = x0;
    px[p + half] = x1;
}

template <typename T>
__device__ __forceinline__ void store_cache(T* dst, float v);
template <>
__device__ __forceinline__ void store_cache<float>(float* dst, float v) {
    *dst = v;
}
template <>
__device__ __forceinline__ void store_cache<__half>(__half* dst, float v) {
    *dst = __float2half_rn(v);
}

// q,k,v [B,qL,H,S].  One workgroup per (b, l, h); thread i handles element i (and i+half).
template <typename T>
__global__ void attn_prep_kernel(float* __restrict__ q, float* __restrict__ k, const float* __restrict__ v, int64_t qL,
                                 int64_t H, int64_t S, const float* __restrict__ inv_freq, int64_t half,
                                 T* __restrict__ kc, T* __restrict__ vc, int64_t maxlen, const int32_t* __restrict__ slots,
                                 int position_id, int32_t* __restrict__ row_token) {
    const int64_t h = blockIdx.x % H, l = (blockIdx.x / H) % qL, b = blockIdx.x / (H * qL);
    const int64_t base = ((b * qL + l) * H + h) * S;
    const int slot = slots[l];
    // slots live in device memory and cannot be validated on the host: a slot outside the cache is
    // dropped (q and k are still rotated) rather than written through
    const bool slot_ok = slot >= 0 && slot < maxlen;
    T* kdst = kc + ((b * H + h) * maxlen + (slot_ok ? slot : 0)) * S;
    T* vdst = vc + ((b * H + h) * maxlen + (slot_ok ? slot : 0)) * S;
    if (blockIdx.x < qL && threadIdx.x == 0) {
        const int s0 = slots[blockIdx.x];
        if (s0 >= 0 && s0 < maxlen) row_token[s0] = (int32_t)blockIdx.x;
    }
    for (int64_t i = threadIdx.x; i < S; i += blockDim.x) {
        if (i < half) {
            float q0 = q[base + i], q1 = q[base + i + half];
            float k0 = k[base + i], k1 = k[base + i + half];
            const float f = inv_freq[i];
            rope_pair(q0, q1, f, (int)l + position_id);
            rope_pair(k0, k1, f, (int)l + position_id);
            q[base + i] = q0;
            q[base + i + half] = q1;
            k[base + i] = k0;
            k[base + i + half] = k1;
            if (slot_ok) {
                store_cache(kdst + i, k0);
                store_cache(kdst + i + half, k1);
            }
        } else if (i >= 2 * half && slot_ok) {
            store_cache(kdst + i, k[base + i]);
        }
        if (slot_ok) store_cache(vdst + i, v[base + i]);
    }
}

__global__ void fill_i32_kernel(int32_t* p, int64_t n, int32_t v) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

// ---- split-KV attention ----------------------------------------------------------------------
__device__ __forceinline__ float4 load4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 load4(const __half* p) {
    const uint2 u = *reinterpret_cast<const uint2*>(p);
    const __half2 a = *reinterpret_cast<const __half2*>(&u.x), b = *reinterpret_cast<const __half2*>(&u.y);
    const float2 fa = __half22float2(a), fb = __half22float2(b);
    return make_float4(fa.x, fa.y, fb.x, fb.y);
}

__device__ __forceinline__ float2 load2(const float* p) { return *reinterpret_cast<const float2*>(p); }
__device__ __forceinline__ float2 load2(const __half* p) {
    const uint32_t u = *reinterpret_cast<const uint32_t*>(p);
    return __half22float2(*reinterpret_cast<const __half2*>(&u));
}

// Per-chunk record in the workspace: [max, sum, out[S]]
// Workgroup = 4 waves; wave w owns rows w*PW .. w*PW+PW-1 of the chunk (C = 4*PW rows);
// lane = 32*hf + e: row parity hf, elements 4e..4e+3 (S == 128).
template <typename T, int PW>
__global__ __launch_bounds__(256) void attn_split_kernel(const float* __restrict__ q, const T* __restrict__ kc,
                                                          const T* __restrict__ vc, int64_t qL, int64_t H, int64_t maxlen,
                                                          int64_t kvLen, const int32_t* __restrict__ row_token,
                                                          float* __restrict__ part, int nchunks) {
    constexpr int S = 128, C = 4 * PW, NL = PW / 2;
    __shared__ float sc[C];
    __shared__ float osh[4][2][S];
    __shared__ float stat[2];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int hf = lane >> 5, e = lane & 31;
    const int chunk = blockIdx.x % nchunks;
    const int64_t bhq = blockIdx.x / nchunks;  // ((b*H)+h)*qL + pq
    const int64_t pq = bhq % qL, h = (bhq / qL) % H, b = bhq / (qL * H);
    const int64_t p0 = (int64_t)chunk * C;
    const T* kbase = kc + (b * H + h) * maxlen * S;
    const T* vbase = vc + (b * H + h) * maxlen * S;

    // issue every K and V load of this wave before anything is consumed
    float4 kv[NL], vv[NL];
#pragma unroll
    for (int i = 0; i < NL; i++) {
        const int64_t p = p0 + wave * PW + i * 2 + hf;
        const int64_t pc = p < kvLen ? p : kvLen - 1;
        kv[i] = load4(kbase + pc * S + e * 4);
        vv[i] = load4(vbase + pc * S + e * 4);
    }
    const float4 qv = load4(q + ((b * qL + pq) * H + h) * S + e * 4);
    const float d_scale = 1.0f / sqrtf((float)S);

#pragma unroll
    for (int i = 0; i < NL; i++) {
        float s = qv.x * kv[i].x;
        s = fmaf(qv.y, kv[i].y, s);
        s = fmaf(qv.z, kv[i].z, s);
        s = fmaf(qv.w, kv[i].w, s);
#pragma unroll
        for (int o = 16; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
        const int r = wave * PW + i * 2 + hf;
        const int64_t p = p0 + r;
        bool live = p < kvLen;
        if (live && qL > 1) live = !(row_token[p] > (int32_t)pq);  // written by a later token of this call
        if (e == 0) sc[r] = live ? s * d_scale : -FLT_MAX;
    }
    __syncthreads();
    if (wave == 0) {
        float v = lane < C ? sc[lane] : -FLT_MAX;
        const float mx = wave_max(v);
        // a row counts only if it is live; a chunk with no live row reports sum 0
        float ex = (lane < C && v != -FLT_MAX) ? expf(v - mx) : 0.0f;
        if (lane < C) sc[lane] = ex;
        const float sum = wave_sum(ex);
        if (lane == 0) {
            stat[0] = mx;
            stat[1] = sum;
        }
    }
    __syncthreads();
    float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int i = 0; i < NL; i++) {
        const float w = sc[wave * PW + i * 2 + hf];
        o.x = fmaf(w, vv[i].x, o.x);
        o.y = fmaf(w, vv[i].y, o.y);
        o.z = fmaf(w, vv[i].z, o.z);
        o.w = fmaf(w, vv[i].w, o.w);
    }
    *reinterpret_cast<float4*>(&osh[wave][hf][e * 4]) = o;
    __syncthreads();
    float* rec = part + ((int64_t)bhq * nchunks + chunk) * (S + 2);
    if (threadIdx.x < S) {
        float a = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; w++) a += osh[w][0][threadIdx.x] + osh[w][1][threadIdx.x];
        rec[2 + threadIdx.x] = a;
    }
    if (threadIdx.x == 0) {
        rec[0] = stat[0];
        rec[1] = stat[1];
    }
}

// Merge of the chunk records of one query: out = sum_c exp(m_c - M) o_c / sum_c exp(m_c - M) s_c.
// LOAD fetches one float of a record.
template <typename LOAD>
__device__ __forceinline__ float merge_chunks(const float* rec, int nchunks, int tid, LOAD load) {
    constexpr int S = 128, CB = 32;
    float M = -FLT_MAX, den = 0.0f, num = 0.0f;
    // every thread reads the (few) chunk statistics itself, so all loads of a batch of chunks are
    // independent and in flight together; batches are folded in with the running-max rescaling
    for (int c0 = 0; c0 < nchunks; c0 += CB) {
        float m[CB], sm[CB], o[CB];
#pragma unroll
        for (int u = 0; u < CB; u++) {
            const bool ok = c0 + u < nchunks;
            const float* r = rec + (int64_t)(ok ? c0 + u : c0) * (S + 2);
            m[u] = ok ? load(r) : -FLT_MAX;
            sm[u] = ok ? load(r + 1) : 0.0f;
            o[u] = ok ? load(r + 2 + tid) : 0.0f;
        }
        float Mb = M;
#pragma unroll
        for (int u = 0; u < CB; u++) Mb = fmaxf(Mb, m[u]);
        const float rescale = (den == 0.0f) ? 0.0f : expf(M - Mb);
        den *= rescale;
        num *= rescale;
#pragma unroll
        for (int u = 0; u < CB; u++) {
            const float sc = (sm[u] == 0.0f) ? 0.0f : expf(m[u] - Mb);
            den = fmaf(sc, sm[u], den);
            num = fmaf(sc, o[u], num);
        }
        M = Mb;
    }
    return num * (1.0f / den);
}

// `nchunks` records per query are laid out; with pos_dev (decode graphs) only the first
// ceil(min(pos_dev[0] + 1, maxlen) / chunk_rows) of them were written by this call.
__global__ __launch_bounds__(128) void attn_merge_kernel(float* __restrict__ q, const float* __restrict__ part, int64_t qL,
                                                          int64_t H, int nchunks, int chunk_rows = 1,
                                                          const int32_t* __restrict__ pos_dev = nullptr, int64_t maxlen = 0) {
    constexpr int S = 128;
    __shared__ float wsh[2][64];
    const int64_t bhq = blockIdx.x;
    const int64_t pq = bhq % qL, h = (bhq / qL) % H, b = bhq / (qL * H);
    const float* rec = part + (int64_t)bhq * nchunks * (S + 2);
    if (pos_dev != nullptr) nchunks = (int)((min((int64_t)pos_dev[0] + 1, maxlen) + chunk_rows - 1) / chunk_rows);
    float r;
    if (nchunks <= 64) {
        // The chunk weights exp(m_c - M) / sum are the same for all 128 output elements: each wave computes
        // them once, one chunk per lane (one expf per lane instead of one per chunk and thread), and every
        // thread then only accumulates its element over the chunks.  Loads in order of use (statistics, then
        // the partial outputs, the first 32 in flight together with the statistics), addresses clamped instead of branched around.
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
        const float* rc = rec + (int64_t)min(lane, nchunks - 1) * (S + 2);
        const float m = rc[0], sm0 = rc[1];
        // (the first 32 partial outputs do not depend on the weights: asked for before the weights are computed)
        float o0[32];
#pragma unroll
        for (int u = 0; u < 32; u++) o0[u] = rec[(int64_t)min(u, nchunks - 1) * (S + 2) + 2 + threadIdx.x];
        __builtin_amdgcn_sched_barrier(0);
        float acc = 0.0f;
        const float mm = lane < nchunks ? m : -FLT_MAX;
        const float sm = lane < nchunks ? sm0 : 0.0f;
        const float M = wave_max(mm);
        const float w = (sm == 0.0f) ? 0.0f : expf(mm - M);
        const float den = wave_sum(w * sm);
        wsh[wave][lane] = w * (1.0f / den);
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int u = 0; u < 32; u++) acc = fmaf(u < nchunks ? wsh[wave][u] : 0.0f, o0[u], acc);
        for (int c0 = 32; c0 < nchunks; c0 += 16) {
            float o[16];
#pragma unroll
            for (int u = 0; u < 16; u++) o[u] = rec[(int64_t)min(c0 + u, nchunks - 1) * (S + 2) + 2 + threadIdx.x];
#pragma unroll
            for (int u = 0; u < 16; u++) acc = fmaf(c0 + u < nchunks ? wsh[wave][c0 + u] : 0.0f, o[u], acc);
        }
        r = acc;
    } else {
        r = merge_chunks(rec, nchunks, threadIdx.x, [](const float* p) { return *p; });
    }
    q[((b * qL + pq) * H + h) * S + threadIdx.x] = r;
}

// ---- decode attention (one query token) ------------------------------------------------------
// attention_rope2 for qL == 1: every workgroup rotates q itself (cos/sin of the position computed once
// per workgroup, one angle per lane), the workgroup whose chunk holds the new token's cache row rotates
// k, writes the rotated k back in place and k, v into the cache, and attends to the new row from
// registers.  The chunk records (max, sum, weighted V sum) are merged by attn_merge_kernel, a second
// launch.  (Merging inside this kernel, by whichever workgroup of a head takes the last arrival ticket, was
// measured slower at every size: the record stores must be acknowledged before the ticket is taken and the
// last workgroup then fetches the records, three round trips to memory against one launch -- kv 256: 9.2
// against 8.2 us, kv 2048: 25.4 against 19.0 us.  One workgroup of 16 wavefronts per head, which needs no
// merge, is bound by what one compute unit can fetch: kv 256 9.1 against 8.2 us, kv 512 with an fp16 cache 20.4
// against 9.4 us.)  A head with a single chunk (nchunks == 1) is finished here and written straight into q.
//
// A lane always fetches 16 bytes of a cache row: 4 floats or 8 halves.  A 128-element row is therefore
// LPR = 32 (fp32) or 16 (fp16) lanes wide and one wave-wide load covers RPW = 2 or 4 rows; a wave owns PW
// rows of the chunk, NL = PW / RPW loads per lane for K and as many for V.
//
// The position may come from device memory (pos_dev != nullptr): a HIP graph of a decode step captures the
// launch once, for the largest kv length (the grid and the record layout are sized by `nchunks`), and every
// replay reads the current position; workgroups whose chunk lies beyond the current kv length leave at once.
template <typename T>
__device__ __forceinline__ float cache_round(float v);
template <>
__device__ __forceinline__ float cache_round<float>(float v) {
    return v;
}
template <>
__device__ __forceinline__ float cache_round<__half>(float v) {
    return __half2float(__float2half_rn(v));
}
template <typename T>
__device__ __forceinline__ void store4(T* dst, float4 v);
template <>
__device__ __forceinline__ void store4<float>(float* dst, float4 v) {
    *reinterpret_cast<float4*>(dst) = v;
}
template <>
__device__ __forceinline__ void store4<__half>(__half* dst, float4 v) {
    const __half2 a = __floats2half2_rn(v.x, v.y), b = __floats2half2_rn(v.z, v.w);
    uint2 u;
    u.x = *reinterpret_cast<const uint32_t*>(&a);
    u.y = *reinterpret_cast<const uint32_t*>(&b);
    *reinterpret_cast<uint2*>(dst) = u;
}

// rotate the lane's 4 elements (index e4 = first element) of a 128-wide head vector at `base`;
// cs = cos table [half], sn = sin table [half] of the current position (LDS)
__device__ __forceinline__ float4 rope4(const float* base, int e4, const float* cs, const float* sn, int half) {
    const float4 own = *reinterpret_cast<const float4*>(base + e4);
    if (e4 >= 2 * half) return own;
    const bool low = e4 < half;
    const float4 other = *reinterpret_cast<const float4*>(base + (low ? e4 + half : e4 - half));
    const int f0 = low ? e4 : e4 - half;
    float o[4] = {own.x, own.y, own.z, own.w}, p[4] = {other.x, other.y, other.z, other.w}, r[4];
#pragma unroll
    for (int c = 0; c < 4; c++) {
        // pair (x0 = element i, x1 = element i+half): y0 = c*x0 - s*x1, y1 = s*x0 + c*x1
        r[c] = low ? cs[f0 + c] * o[c] - sn[f0 + c] * p[c] : sn[f0 + c] * p[c] + cs[f0 + c] * o[c];
    }
    return make_float4(r[0], r[1], r[2], r[3]);
}

// the same on values already in registers: `own` = the lane's 4 elements at e4, `other` = their partners
__device__ __forceinline__ float4 rope4_regs(float4 own, float4 other, int e4, const float* cs, const float* sn, int half) {
    if (e4 >= 2 * half) return own;
    const bool low = e4 < half;
    const int f0 = low ? e4 : e4 - half;
    float o[4] = {own.x, own.y, own.z, own.w}, p[4] = {other.x, other.y, other.z, other.w}, r[4];
#pragma unroll
    for (int c = 0; c < 4; c++) r[c] = low ? cs[f0 + c] * o[c] - sn[f0 + c] * p[c] : sn[f0 + c] * p[c] + cs[f0 + c] * o[c];
    return make_float4(r[0], r[1], r[2], r[3]);
}
__device__ __forceinline__ int rope_partner(int e4, int half) {
    return e4 >= 2 * half ? e4 : (e4 < half ? e4 + half : e4 - half);
}

// 16 bytes of a cache row as they come from memory, and their widening to floats
template <typename T>
struct RowPiece;
template <>
struct RowPiece<float> {
    static constexpr int EPL = 4;  // elements per lane
    static __device__ __forceinline__ void widen(const uint4& r, float out[4]) {
        out[0] = __uint_as_float(r.x), out[1] = __uint_as_float(r.y), out[2] = __uint_as_float(r.z), out[3] = __uint_as_float(r.w);
    }
    // the 16 bytes as the cache stores them
    static __device__ __forceinline__ uint4 pack(const float4* v) {
        return make_uint4(__float_as_uint(v[0].x), __float_as_uint(v[0].y), __float_as_uint(v[0].z), __float_as_uint(v[0].w));
    }
};
template <>
struct RowPiece<__half> {
    static constexpr int EPL = 8;
    static __device__ __forceinline__ float lo(uint32_t w) { return __half2float(__ushort_as_half((unsigned short)(w & 0xFFFFu))); }
    static __device__ __forceinline__ float hi(uint32_t w) { return __half2float(__ushort_as_half((unsigned short)(w >> 16))); }
    static __device__ __forceinline__ void widen(const uint4& r, float out[8]) {
        out[0] = lo(r.x), out[1] = hi(r.x), out[2] = lo(r.y), out[3] = hi(r.y);
        out[4] = lo(r.z), out[5] = hi(r.z), out[6] = lo(r.w), out[7] = hi(r.w);
    }
    static __device__ __forceinline__ uint32_t pack2(float a, float b) {
        return (uint32_t)__half_as_ushort(__float2half_rn(a)) | ((uint32_t)__half_as_ushort(__float2half_rn(b)) << 16);
    }
    static __device__ __forceinline__ uint4 pack(const float4* v) {
        return make_uint4(pack2(v[0].x, v[0].y), pack2(v[0].z, v[0].w), pack2(v[1].x, v[1].y), pack2(v[1].z, v[1].w));
    }
};
// cache rows are read exactly once per call: non-temporal, so that they do not displace the records and the
// activations that are reused out of the caches
__device__ __forceinline__ uint4 load_row16(const void* p) {
    typedef unsigned int u32x4_a __attribute__((ext_vector_type(4)));
    const u32x4_a v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_a*>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}

//
// RECS: the chunk records are not merged here at all but handed to the FC that consumes the attention output
// (the o projection merges them as it loads its input, llmops_fc_Q4A_decode_attn): workgroups of NWV = 16
// wavefronts take 256 or 512 cache rows each, so that a head has at most kAttnRecChunks records, laid out as
// stats [B*H][kAttnRecChunks][2] (max, sum) and outs [B*H][kAttnRecChunks][128]; a chunk beyond the current kv
// length leaves an empty record (sum 0, zeros).  q is then left as it came in.
constexpr int kAttnRecChunks = 8;

template <typename T, int PW, int NWV = 4, bool RECS = false>
__global__ __launch_bounds__(NWV * 64) void attn_decode_kernel(const int32_t* __restrict__ pos_dev, int position_id, int nchunks,
                                                           int maxlen, T* kc, T* vc, const int32_t* __restrict__ slots,
                                                           float* q, float* k, const float* __restrict__ v,
                                                           const float* __restrict__ inv_freq, int half, float* part,
                                                           float* rec_stats = nullptr, float* rec_outs = nullptr) {
    // (argument order: the first 14 dwords arrive in scalar registers with the wave (kernel-argument preload);
    // they are what the position, the slot and the cache rows' addresses need)
    constexpr int S = 128, C = NWV * PW;
    constexpr int EPL = RowPiece<T>::EPL, LPR = S / EPL, RPW = 64 / LPR, NL = PW / RPW;
    static_assert(NL >= 1 && NL <= LPR, "rows per lane");
    __shared__ float sc[C];
    __shared__ float osh[NWV][RPW][S];
    __shared__ float stat[2];
    __shared__ float cs_sh[64], sn_sh[64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int rsel = lane / LPR, e = lane % LPR;  // which of the RPW rows of a wave-wide load, which 16 bytes of it
    // grid = (chunks, heads): no division, and 32-bit row arithmetic throughout -- every instruction in front of
    // the first cache row is paid once per wave before the memory system has anything to do
    const int chunk = blockIdx.x;
    const uint32_t bh = blockIdx.y;
    // One round trip for everything that did not come with the wave: the slot, the position (read through a
    // pointer that is always valid, so that there is no branch around the load) and the remaining arguments,
    // which the compiler would otherwise fetch one by one where the code first uses them.
    const int slot = slots[0];
    const int pos_loaded = (pos_dev != nullptr ? pos_dev : slots)[0];
    asm volatile("" ::"s"(slot), "s"(pos_loaded), "s"(k), "s"(v), "s"(inv_freq), "s"(half), "s"(rec_stats), "s"(rec_outs), "s"(part));
    if (pos_dev != nullptr) position_id = pos_loaded;
    const int kvLen = position_id < maxlen ? position_id + 1 : maxlen;
    const int nact = (int)((unsigned)(kvLen + C - 1) / C);  // chunks that hold rows at this position (none if kvLen <= 0)
    if (chunk >= nact || kvLen <= 0) {
        if (RECS) {  // an empty record: weight 0 whatever the others hold
            if (threadIdx.x < S) rec_outs[((size_t)bh * kAttnRecChunks + chunk) * S + threadIdx.x] = 0.0f;
            if (threadIdx.x == 0) {
                rec_stats[((size_t)bh * kAttnRecChunks + chunk) * 2] = -FLT_MAX;
                rec_stats[((size_t)bh * kAttnRecChunks + chunk) * 2 + 1] = 0.0f;
            }
        }
        return;
    }
    const int p0 = chunk * C;
    // a head's plane of the cache is below 4 GiB (checked by the launcher): uniform 64-bit base, 32-bit lane offsets
    T* kbase = kc + (size_t)bh * ((uint32_t)maxlen * (uint32_t)S);
    T* vbase = vc + (size_t)bh * ((uint32_t)maxlen * (uint32_t)S);
    const float* qrow = q + (size_t)bh * S;
    float* krow = k + (size_t)bh * S;
    const float* vrow = v + (size_t)bh * S;

    // Loads return in issue order and a wave can only wait for "all but the youngest n".  So the small
    // loads whose data the rotation needs go first, then the K rows, then the V rows: the cos/sin table,
    // the rotation of q (and k) and the scores are then computed while the rows behind them are still in
    // flight, instead of after the last V row has landed.
    const bool slot_ok = slot >= 0 && slot < maxlen;
    // the workgroup that owns the new token's row (or the last chunk, if the row lies beyond kvLen)
    const int owner = (slot_ok && slot / C < nact) ? slot / C : nact - 1;
    const int e0 = e * EPL;  // the lane's first element of the row
    const float freq = inv_freq[min((int)threadIdx.x, half - 1)];
    float4 q_own[EPL / 4], q_oth[EPL / 4];
#pragma unroll
    for (int u = 0; u < EPL / 4; u++) {
        q_own[u] = *reinterpret_cast<const float4*>(qrow + (uint32_t)(e0 + 4 * u));
        q_oth[u] = *reinterpret_cast<const float4*>(qrow + (uint32_t)rope_partner(e0 + 4 * u, half));
    }
    // The new token's k and v rows: only the owner uses them, but every workgroup asks for them (48-96 bytes per
    // lane out of L2): a branch around these loads would leave the registers with two definitions, and the copies
    // that merge them wait for the loads -- one memory round trip in front of the owner's first cache row.
    float4 kn[EPL / 4], k_oth[EPL / 4], vn[EPL / 4];
#pragma unroll
    for (int u = 0; u < EPL / 4; u++) {
        kn[u] = *reinterpret_cast<const float4*>(krow + (uint32_t)(e0 + 4 * u));
        k_oth[u] = *reinterpret_cast<const float4*>(krow + (uint32_t)rope_partner(e0 + 4 * u, half));
        vn[u] = *reinterpret_cast<const float4*>(vrow + (uint32_t)(e0 + 4 * u));
    }
    __builtin_amdgcn_sched_barrier(0);
    uint4 kraw[NL], vraw[NL];
#pragma unroll
    for (int i = 0; i < NL; i++) {
        const int pc = min(p0 + wave * PW + i * RPW + rsel, kvLen - 1);
        kraw[i] = load_row16(kbase + (uint32_t)(pc * S + e0));
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < NL; i++) {
        const int pc = min(p0 + wave * PW + i * RPW + rsel, kvLen - 1);
        vraw[i] = load_row16(vbase + (uint32_t)(pc * S + e0));
    }
    __builtin_amdgcn_sched_barrier(0);
    if (threadIdx.x < half) {
        const float xita = freq * (float)position_id;
        cs_sh[threadIdx.x] = cosf(xita);
        sn_sh[threadIdx.x] = sinf(xita);
    }
    __syncthreads();
    float qv[EPL];
#pragma unroll
    for (int u = 0; u < EPL / 4; u++) {
        const float4 r = rope4_regs(q_own[u], q_oth[u], e0 + 4 * u, cs_sh, sn_sh, half);
        qv[4 * u] = r.x, qv[4 * u + 1] = r.y, qv[4 * u + 2] = r.z, qv[4 * u + 3] = r.w;
    }
    // the new token's row as the cache holds it (rounded to T): it is attended to from registers
    uint4 knraw = make_uint4(0, 0, 0, 0), vnraw = knraw;
    if (chunk == owner) {
        // The new v row is only needed here, and its conversion to the cache's type must stay here: the compiler
        // otherwise moves it up into the block that loads the row, in front of the cache rows' loads, and the
        // owner workgroup then waits for one round trip before it asks for its first cache row.  Tying the values
        // to something read after the barrier keeps the conversion below it.
        const float after_barrier = cs_sh[0];
#pragma unroll
        for (int u = 0; u < EPL / 4; u++)
            asm volatile("" : "+v"(vn[u].x), "+v"(vn[u].y), "+v"(vn[u].z), "+v"(vn[u].w) : "v"(after_barrier));
#pragma unroll
        for (int u = 0; u < EPL / 4; u++) kn[u] = rope4_regs(kn[u], k_oth[u], e0 + 4 * u, cs_sh, sn_sh, half);
        knraw = RowPiece<T>::pack(kn);
        vnraw = RowPiece<T>::pack(vn);
        __syncthreads();  // every wave has read the raw k before it is overwritten
        if (wave == 0 && rsel == 0) {
#pragma unroll
            for (int u = 0; u < EPL / 4; u++) *reinterpret_cast<float4*>(krow + (uint32_t)(e0 + 4 * u)) = kn[u];
            if (slot_ok) {
                *reinterpret_cast<uint4*>(kbase + (uint32_t)(slot * S + e0)) = knraw;
                *reinterpret_cast<uint4*>(vbase + (uint32_t)(slot * S + e0)) = vnraw;
            }
        }
#pragma unroll
        for (int i = 0; i < NL; i++)
            if (p0 + wave * PW + i * RPW + rsel == slot) kraw[i] = knraw;
    }
    const float d_scale = 1.0f / sqrtf((float)S);
    // NL partial dot products per lane, each to be summed over the LPR lanes of a row.  Summing them one
    // by one takes log2(LPR) lane exchanges each; instead the lanes split the rows between them while they
    // add: at every exchange a lane keeps one half of its rows and hands the other half to its partner,
    // so NL rows cost NL/2 + NL/4 + .. + 1 exchanges plus one per remaining lane bit.
    float sp[NL];
#pragma unroll
    for (int i = 0; i < NL; i++) {
        float kf[EPL];
        RowPiece<T>::widen(kraw[i], kf);
        float s = 0.0f;
#pragma unroll
        for (int c = 0; c < EPL; c++) s = fmaf(qv[c], kf[c], s);
        sp[i] = s;
    }
    int row_of_lane = 0;  // which of the NL rows this lane ends up holding
    {
        int n = NL, off = LPR / 2;
#pragma unroll
        for (; n > 1; n >>= 1, off >>= 1) {
            const bool up = (e & off) != 0;
#pragma unroll
            for (int j = 0; j < NL / 2; j++) {
                if (j < n / 2) {
                    const float keep = up ? sp[j + n / 2] : sp[j];
                    const float send = up ? sp[j] : sp[j + n / 2];
                    sp[j] = keep + __shfl_xor(send, off, 64);
                }
            }
            row_of_lane = row_of_lane * 2 + (up ? 1 : 0);
        }
#pragma unroll
        for (; off > 0; off >>= 1) sp[0] += __shfl_xor(sp[0], off, 64);
    }
    {
        // lanes whose remaining (low) bits are zero write the row they hold
        constexpr int kLowMask = LPR / NL - 1;
        const int r = wave * PW + row_of_lane * RPW + rsel;
        if ((e & kLowMask) == 0) sc[r] = (p0 + r < kvLen) ? sp[0] * d_scale : -FLT_MAX;
    }
    __syncthreads();
    if (wave == 0) {
        float mx = -FLT_MAX;
#pragma unroll
        for (int u = 0; u < (C + 63) / 64; u++) mx = fmaxf(mx, lane + 64 * u < C ? sc[lane + 64 * u] : -FLT_MAX);
        mx = wave_max(mx);
        float sum = 0.0f;
#pragma unroll
        for (int u = 0; u < (C + 63) / 64; u++) {
            const int r = lane + 64 * u;
            if (r < C) {
                const float x = sc[r];
                const float ex = (x != -FLT_MAX) ? expf(x - mx) : 0.0f;
                sc[r] = ex;
                sum += ex;
            }
        }
        sum = wave_sum(sum);
        if (lane == 0) {
            stat[0] = mx;
            stat[1] = sum;
        }
    }
    __syncthreads();
    if (chunk == owner) {
#pragma unroll
        for (int i = 0; i < NL; i++)
            if (p0 + wave * PW + i * RPW + rsel == slot) vraw[i] = vnraw;
    }
    float o[EPL];
#pragma unroll
    for (int c = 0; c < EPL; c++) o[c] = 0.0f;
#pragma unroll
    for (int i = 0; i < NL; i++) {
        float vf[EPL];
        RowPiece<T>::widen(vraw[i], vf);
        const float w = sc[wave * PW + i * RPW + rsel];
#pragma unroll
        for (int c = 0; c < EPL; c++) o[c] = fmaf(w, vf[c], o[c]);
    }
#pragma unroll
    for (int u = 0; u < EPL / 4; u++)
        *reinterpret_cast<float4*>(&osh[wave][rsel][e0 + 4 * u]) = make_float4(o[4 * u], o[4 * u + 1], o[4 * u + 2], o[4 * u + 3]);
    __syncthreads();
    float* rec = part + ((size_t)bh * nchunks + chunk) * (S + 2);
    float mine = 0.0f;  // this thread's element of the chunk's weighted V sum (threads 0..127)
    if (threadIdx.x < S) {
#pragma unroll
        for (int w = 0; w < NWV; w++)
#pragma unroll
            for (int r = 0; r < RPW; r++) mine += osh[w][r][threadIdx.x];
    }
    if (RECS) {
        if (threadIdx.x < S) rec_outs[((size_t)bh * kAttnRecChunks + chunk) * S + threadIdx.x] = mine;
        if (threadIdx.x == 0) {
            rec_stats[((size_t)bh * kAttnRecChunks + chunk) * 2] = stat[0];
            rec_stats[((size_t)bh * kAttnRecChunks + chunk) * 2 + 1] = stat[1];
        }
        return;
    }
    if (nchunks == 1) {  // the workgroup saw every row of the head
        if (threadIdx.x < S) q[(size_t)bh * S + threadIdx.x] = mine * (1.0f / stat[1]);
        return;
    }
    if (threadIdx.x < S) rec[2 + threadIdx.x] = mine;
    if (threadIdx.x == 0) {
        rec[0] = stat[0];
        rec[1] = stat[1];
    }
}

// ---- prefill: tiled attention on the fp16 matrix cores, fp32 values carried as two halves -------
// Many query tokens share the K and V rows they look at, so the split kernel above (one workgroup
// per query and chunk) re-reads the cache qL times.  Here a workgroup owns 128 queries of one head
// and walks the cache in tiles of 32 rows that are staged once in LDS.  It has two sets of 4 waves
// (32 queries per wave, ONE QUERY PER LANE PAIR): both sets hold the same queries, set 0 takes the even
// tiles and set 1 the odd ones, each with its own online softmax, and the two results are merged through
// LDS at the end.  (A tile's chain -- stage, products, softmax, products -- is a sequence of latencies
// that one wave per SIMD cannot hide, and under the causal mask the last query tile of a head has 16
// times the tiles of the first; two sets halve the longest chain.)  Query tiles are dealt out from the
// last to the first, one workgroup per compute unit at a time.
//
// Arithmetic.  On this part v_mfma_f32_32x32x2_f32 runs at the vector ALU's rate and keeps the vector ALU
// busy while it runs (a wave's -- or its SIMD neighbour's -- vector instructions simply add to its time:
// measured), so an fp32-MFMA kernel pays for the softmax, the staging and the products one after the
// other.  The fp16 MFMAs are 16 times faster and leave the vector ALU free.  Every fp32 operand x is
// therefore split into two halves, hi = fp16(x) (rounded toward zero) and lo = fp16(x - hi), whose sum
// carries 22 bits of x, and a product a*b is computed as hi_a*hi_b + hi_a*lo_b + lo_a*hi_b: three
// v_mfma_f32_32x32x16_f16 with fp32 accumulation (each half-by-half product is exact in fp32; the dropped
// lo*lo term is 2^-22 of the product).  Results agree with fp32 arithmetic to about 1e-6 of the largest
// output, like two fp32 evaluations in different summation orders.  Values beyond the fp16 range
// (|x| >= 65504) are not representable this way; activations and cache rows of a transformer are far below.
// An fp16 cache has no low halves: two MFMAs per product.
//
//   S^T = K_tile * Q^T     8 steps of 16 head dims.  A = K[kv = lane%32][16i + 8*hf .. +7]: 16 bytes of the
//                          row's hi plane (and of its lo plane) in LDS.  B = the lane's own query row, same
//                          dims, split once into 64 registers.  The result puts query lane%32 into the
//                          lane, 16 cache rows 8j + 4*hf + v each.  hi*hi goes to one accumulator, the cross
//                          terms to another.
//   mask, online softmax   per lane, fp32, plus one exchange with lane^32 (the other 16 rows of the tile)
//   O^T += V_tile^T * P^T  2 steps of 16 cache rows x 4 blocks of 32 output columns.  B = the lane's 8
//                          probabilities 8b .. 8b+7 exactly as they sit in registers (rows 8j + 4*hf + v,
//                          j = 2b, 2b+1), split into halves.  A = V[those 8 rows][column 32c + lane%32]:
//                          the tile is staged transposed, with the rows of a column permuted so that these
//                          8 halves are 16 contiguous bytes.
//
// Everything a lane holds (running max, sum, 4 x 16 output values) belongs to its own query, so
// the rescaling needs no cross-lane traffic, and no probability ever goes through LDS.  Tiles that
// no query of a wave may see (in-chunk causal mask, ops/op_attn.hpp:1007-1011) are skipped.  K rows
// take 272 bytes per plane and V columns 80, so that the 16 lanes one phase of a 16-byte read serves
// touch 16 different 16-byte slots of the 256-byte bank line (17 and 5 are odd).
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));

// (a, b) -> packed halves hi and lo with a = hi.x + lo.x, b = hi.y + lo.y to 22 bits
__device__ __forceinline__ void split2(float a, float b, uint32_t& hi, uint32_t& lo) {
    const v2h h = __builtin_bit_cast(v2h, __builtin_amdgcn_cvt_pkrtz(a, b));
    hi = __builtin_bit_cast(uint32_t, h);
    lo = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(a - (float)h[0], b - (float)h[1]));
}
__device__ __forceinline__ uint32_t pack_hi(float a, float b) {
    return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(a, b));
}
union V8hBits {
    v8h h;
    uint32_t u[4];
    uint4 q;
};

// One tile in LDS (fp16 planes, the tile's tokens); each wave set has two of them; the merge at the end reuses the memory
template <bool LO>
struct PrefillSmem {
    static constexpr int S = 128, BK = 32, KSB = 272, VSB = 80;
    uint8_t k_hi[BK * KSB];
    uint8_t k_lo[LO ? BK * KSB : 16];
    uint8_t v_hi[S * VSB];
    uint8_t v_lo[LO ? S * VSB : 16];
    int tok[BK];
    int tok_range[4];  // smallest and largest token of the tile
};
constexpr size_t kPrefillMergeBytes = (size_t)66 * 256 * sizeof(float);  // set 1's (max, sum, 64 outputs) per lane
template <bool LO>
constexpr size_t prefill_smem_bytes() {
    return 4 * sizeof(PrefillSmem<LO>) > kPrefillMergeBytes ? 4 * sizeof(PrefillSmem<LO>) : kPrefillMergeBytes;
}

template <typename T>
__global__ __launch_bounds__(512) void attn_prefill_kernel(float* q, const T* __restrict__ kc, const T* __restrict__ vc,
                                                          int64_t qL, int64_t H, int64_t maxlen, int64_t kvLen,
                                                          const int32_t* __restrict__ row_token, int qtiles) {
    constexpr bool LO = sizeof(T) == 4;  // an fp16 cache holds no low halves
    constexpr int S = 128, BQ = 128, BK = 32, KSB = 272, VSB = 80;
    extern __shared__ __align__(16) uint8_t smem_raw[];
    const int lane = threadIdx.x & 63, wave8 = threadIdx.x >> 6;
    const int set = wave8 >> 2, wave = wave8 & 3, tid = threadIdx.x & 255;  // (wave, tid: within the set)
    // two tile buffers per set, used alternately: while a tile is multiplied the next one is written
    PrefillSmem<LO>* const sm2 = reinterpret_cast<PrefillSmem<LO>*>(smem_raw) + 2 * set;
    const int hf = lane >> 5, c32 = lane & 31;
    // late query tiles see the most cache rows: they are dealt out first so that they do not form the tail
    const int64_t bhs = gridDim.x / qtiles;
    const int qt = qtiles - 1 - (int)(blockIdx.x / bhs);
    const int64_t bh = blockIdx.x % bhs, b = bh / H, h = bh % H;
    // (32-bit arithmetic from here on: the launcher keeps qL and kvLen below 2^31 and a head's cache plane below 4 GiB)
    const int qLi = (int)qL, kvLeni = (int)kvLen;
    const int q_lo_wave = qt * BQ + wave * 32;
    const int pq = q_lo_wave + c32;  // this lane's query token
    const bool valid = pq < qLi;
    const int q_hi_wave = min(q_lo_wave + 31, qLi - 1);
    float* qrow = q + ((b * qL + (valid ? pq : qLi - 1)) * H + h) * S;
    const T* kbase = kc + bh * maxlen * S;
    const T* vbase = vc + bh * maxlen * S;

    // the lane's share of its query row as halves: step i covers dims 16i + 8*hf .. +7
    V8hBits qh[8], ql[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const float4 t0 = *reinterpret_cast<const float4*>(qrow + 16 * i + 8 * hf);
        const float4 t1 = *reinterpret_cast<const float4*>(qrow + 16 * i + 8 * hf + 4);
        split2(t0.x, t0.y, qh[i].u[0], ql[i].u[0]);
        split2(t0.z, t0.w, qh[i].u[1], ql[i].u[1]);
        split2(t1.x, t1.y, qh[i].u[2], ql[i].u[2]);
        split2(t1.z, t1.w, qh[i].u[3], ql[i].u[3]);
    }
    const float d_scale = 1.0f / sqrtf((float)S);
    float m_run = -FLT_MAX, l_run = 0.0f;
    v16f o[4];
#pragma unroll
    for (int c = 0; c < 4; c++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[c][r] = 0.0f;

    // Staging.  K: a thread moves 16 consecutive floats of one row (row = thread/8).  V is written transposed,
    // cache row r of the tile at position 16*(r/16) + 8*((r/4)%2) + 4*((r%16)/8) + r%4 of its column: a thread
    // moves the 8 rows that share an aligned run of 8 positions (rows 16b + 4h + w and 16b + 8 + 4h + w, w = 0..3;
    // (b, h) = the thread's wave) of two neighbouring columns, so that a column's share is one 16-byte store.
    // (Four rows of four columns per thread meant 8-byte stores 320 bytes apart: eight lanes on every bank.)
    // The next tile's global loads are issued before the current tile is computed on and land in registers
    // meanwhile.
    const int krow = tid >> 3, kseg = tid & 7;
    const int vb = wave >> 1, vh = wave & 1, vcp = lane;  // rows 16*vb + 8*(e/4) + 4*vh + e%4, columns 2*vcp, 2*vcp+1
    float4 kst[4];
    float2 vst[8];
    int tst = INT_MAX;
#define LLMOPS_STAGE_LOAD(KV0)                                                                          \
    do {                                                                                                \
        const uint32_t rk_ = (uint32_t)min((KV0) + krow, kvLeni - 1);                                   \
        _Pragma("unroll") for (int u = 0; u < 4; u++)                                                   \
            kst[u] = load4(kbase + (rk_ * (uint32_t)S + (uint32_t)(kseg * 16 + u * 4)));               \
        _Pragma("unroll") for (int e = 0; e < 8; e++) {                                                 \
            const uint32_t rv_ = (uint32_t)min((KV0) + 16 * vb + 8 * (e >> 2) + 4 * vh + (e & 3), kvLeni - 1); \
            vst[e] = load2(vbase + (rv_ * (uint32_t)S + (uint32_t)(vcp * 2)));                          \
        }                                                                                               \
        if (tid < BK) tst = ((KV0) + tid < kvLeni) ? row_token[(KV0) + tid] : INT_MAX;                  \
    } while (0)
    // The last cache row that any query of the workgroup may see bounds the walk (rows of later tokens and rows
    // beyond it are masked anyway; without the bound an early query tile would stage, barrier by barrier, all the
    // tiles that only later tiles need).
    int kv_end;
    {
        const int q_hi_wg = min((qt + 1) * BQ, qLi) - 1;
        int last = -1;
        for (int r = tid; r < kvLeni; r += 256)
            if (row_token[r] <= q_hi_wg) last = r;  // (r grows: the last hit is the largest; each set scans all rows)
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) last = max(last, __shfl_xor(last, off, 64));
        int* const red = sm2[1].tok;  // (the second buffer is first written at the end of the loop's first pass)
        if (lane == 0) red[wave] = last;
        __syncthreads();
        kv_end = max(max(red[0], red[1]), max(red[2], red[3])) + 1;
    }
    if (kv_end <= 0) kv_end = 1;  // no row is visible to anybody (cannot happen: a token sees its own row)
    // Writing a staged tile: halves of K row-major, halves of V transposed, the tile's tokens and their range.
#define LLMOPS_STAGE_STORE(SM)                                                                                  \
    do {                                                                                                        \
        uint32_t hi_[8], lo_[8];                                                                                \
        _Pragma("unroll") for (int u = 0; u < 4; u++) {                                                         \
            split2(kst[u].x, kst[u].y, hi_[2 * u], lo_[2 * u]);                                                 \
            split2(kst[u].z, kst[u].w, hi_[2 * u + 1], lo_[2 * u + 1]);                                         \
        }                                                                                                       \
        uint4* dh_ = reinterpret_cast<uint4*>(&(SM).k_hi[krow * KSB + kseg * 32]);                              \
        dh_[0] = make_uint4(hi_[0], hi_[1], hi_[2], hi_[3]);                                                    \
        dh_[1] = make_uint4(hi_[4], hi_[5], hi_[6], hi_[7]);                                                    \
        if (LO) {                                                                                               \
            uint4* dl_ = reinterpret_cast<uint4*>(&(SM).k_lo[krow * KSB + kseg * 32]);                          \
            dl_[0] = make_uint4(lo_[0], lo_[1], lo_[2], lo_[3]);                                                \
            dl_[1] = make_uint4(lo_[4], lo_[5], lo_[6], lo_[7]);                                                \
        }                                                                                                       \
        {                                                                                                       \
            uint32_t h_[2][4], l_[2][4]; /* [column][pair of rows] */                                           \
            _Pragma("unroll") for (int e2 = 0; e2 < 4; e2++) {                                                  \
                split2(vst[2 * e2].x, vst[2 * e2 + 1].x, h_[0][e2], l_[0][e2]);                                 \
                split2(vst[2 * e2].y, vst[2 * e2 + 1].y, h_[1][e2], l_[1][e2]);                                 \
            }                                                                                                   \
            _Pragma("unroll") for (int j = 0; j < 2; j++) {                                                     \
                const int at_ = (2 * vcp + j) * VSB + (16 * vb + 8 * vh) * 2;                                   \
                *reinterpret_cast<uint4*>(&(SM).v_hi[at_]) = make_uint4(h_[j][0], h_[j][1], h_[j][2], h_[j][3]); \
                if (LO) *reinterpret_cast<uint4*>(&(SM).v_lo[at_]) = make_uint4(l_[j][0], l_[j][1], l_[j][2], l_[j][3]); \
            }                                                                                                   \
        }                                                                                                       \
        if (wave == 0) {                                                                                        \
            /* the tile's token range, once for all waves: DPP steps inside the rows of 16 lanes, the two rows */ \
            /* that hold tokens (lanes 0..31) combined through scalar registers */                              \
            int mn_ = tst, mx_ = tst;                                                                           \
            LLMOPS_DPP_MINMAX(0xB1);  /* quad_perm [1,0,3,2] */                                                 \
            LLMOPS_DPP_MINMAX(0x4E);  /* quad_perm [2,3,0,1] */                                                 \
            LLMOPS_DPP_MINMAX(0x141); /* row_half_mirror */                                                     \
            LLMOPS_DPP_MINMAX(0x140); /* row_mirror */                                                          \
            const int lo2_ = min(__builtin_amdgcn_readlane(mn_, 0), __builtin_amdgcn_readlane(mn_, 16));        \
            const int hi2_ = max(__builtin_amdgcn_readlane(mx_, 0), __builtin_amdgcn_readlane(mx_, 16));        \
            if (lane < BK) (SM).tok[lane] = tst;                                                                \
            if (lane == 0) (SM).tok_range[0] = lo2_, (SM).tok_range[1] = hi2_;                                  \
        }                                                                                                       \
    } while (0)
#define LLMOPS_DPP_MINMAX(CTRL)                                                      \
    mn_ = min(mn_, __builtin_amdgcn_update_dpp(mn_, mn_, CTRL, 0xF, 0xF, false)); \
    mx_ = max(mx_, __builtin_amdgcn_update_dpp(mx_, mx_, CTRL, 0xF, 0xF, false))
    // Set 0 walks the tiles 0, 2, 4, ..., set 1 the tiles 1, 3, 5, ...: both make the same number of passes.  One
    // barrier per pass: behind it the pass's buffer is complete and nobody reads the other buffer any more, which
    // the pass then fills -- after its own products -- from the registers that the loads of the pass before filled.
    LLMOPS_STAGE_LOAD(set * BK);
    LLMOPS_STAGE_STORE(sm2[0]);
    if (2 * BK < kv_end) LLMOPS_STAGE_LOAD(set * BK + 2 * BK);
    for (int kv_pair = 0, pass = 0; kv_pair < kv_end; kv_pair += 2 * BK, pass++) {
        PrefillSmem<LO>& sm = sm2[pass & 1];
        const uint8_t* kp_hi = &sm.k_hi[c32 * KSB + 16 * hf];  // + 32 i
        const uint8_t* kp_lo = &sm.k_lo[LO ? c32 * KSB + 16 * hf : 0];
        const uint8_t* vp_hi = &sm.v_hi[c32 * VSB + 16 * hf];  // + 32 c * VSB + 32 b
        const uint8_t* vp_lo = &sm.v_lo[LO ? c32 * VSB + 16 * hf : 0];
        const int* tok = sm.tok;
        __syncthreads();
        // skip the tile if even the wave's last query may not see any of its rows; a tile that every query of the
        // wave sees whole (the usual case away from the diagonal) needs no masks
        const int tmin = sm.tok_range[0], tmax = sm.tok_range[1];
        if (q_lo_wave < qLi && tmin <= q_hi_wave) {
        const bool all_visible = tmax <= q_lo_wave && q_lo_wave + 31 < qLi;

        v16f s0, s1;
#pragma unroll
        for (int r = 0; r < 16; r++) s0[r] = 0.0f, s1[r] = 0.0f;
        {
            // operand reads run two steps ahead of the MFMAs that use them
            v8h ah[3], al[3];
            ah[0] = *reinterpret_cast<const v8h*>(kp_hi);
            ah[1] = *reinterpret_cast<const v8h*>(kp_hi + 32);
            if (LO) {
                al[0] = *reinterpret_cast<const v8h*>(kp_lo);
                al[1] = *reinterpret_cast<const v8h*>(kp_lo + 32);
            }
#pragma unroll
            for (int i = 0; i < 8; i++) {
                if (i + 2 < 8) {
                    ah[(i + 2) % 3] = *reinterpret_cast<const v8h*>(kp_hi + 32 * (i + 2));
                    if (LO) al[(i + 2) % 3] = *reinterpret_cast<const v8h*>(kp_lo + 32 * (i + 2));
                }
                __builtin_amdgcn_sched_barrier(0);
                s0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah[i % 3], qh[i].h, s0, 0, 0, 0);
                s1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah[i % 3], ql[i].h, s1, 0, 0, 0);
                if (LO) s1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(al[i % 3], qh[i].h, s1, 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        v16f sacc = s0 + s1;

        // scale, mask (rows written by later tokens of this call, rows beyond kvLen), running max
        float mx = -FLT_MAX;
        if (all_visible) {  // (the same for the whole wave)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                sacc[r] *= d_scale;
                mx = fmaxf(mx, sacc[r]);
            }
        } else {
            const int pq32 = valid ? pq : INT_MIN;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int4 t4 = *reinterpret_cast<const int4*>(&tok[8 * j + 4 * hf]);
                const int tt[4] = {t4.x, t4.y, t4.z, t4.w};
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    const float sv = (tt[v] <= pq32) ? sacc[4 * j + v] * d_scale : -FLT_MAX;
                    sacc[4 * j + v] = sv;
                    mx = fmaxf(mx, sv);
                }
            }
        }
        {  // the other half of the lane pair (lane ^ 32) holds the other 16 rows of the query's tile
            const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(mx), __float_as_uint(mx), false, false);
            mx = fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
        }
        const float m_new = fmaxf(m_run, mx);
        const float alpha = expf(m_run - m_new);  // 0 on the first visible tile, 1 while nothing is visible
        float psum = 0.0f;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            // e^x as 2^(x * log2 e) on the exponential unit: x <= 0, and wherever the result matters (|x| < 20)
            // the product's rounding moves it by less than 1e-6 of itself
            const float pv = (sacc[r] == -FLT_MAX) ? 0.0f : __builtin_amdgcn_exp2f((sacc[r] - m_new) * 1.44269504088896341f);
            sacc[r] = pv;
            psum += pv;
        }
        {
            const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(psum), __float_as_uint(psum), false, false);
            psum = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
        }
        l_run = l_run * alpha + psum;
        if (__any(m_new != m_run)) {  // (alpha is exactly 1 for a query whose maximum did not move)
#pragma unroll
            for (int c = 0; c < 4; c++)
#pragma unroll
                for (int r = 0; r < 16; r++) o[c][r] *= alpha;
        }
        m_run = m_new;

        // O^T += V^T P^T: step b takes the lane's probabilities 8b .. 8b+7 (cache rows 8j + 4*hf + v, j = 2b, 2b+1)
#pragma unroll
        for (int bb = 0; bb < 2; bb++) {
            V8hBits ph, pl;
#pragma unroll
            for (int e = 0; e < 4; e++) split2(sacc[8 * bb + 2 * e], sacc[8 * bb + 2 * e + 1], ph.u[e], pl.u[e]);
            v8h ah[4], al[4];
#pragma unroll
            for (int c = 0; c < 4; c++) {
                ah[c] = *reinterpret_cast<const v8h*>(vp_hi + 32 * c * VSB + 32 * bb);
                if (LO) al[c] = *reinterpret_cast<const v8h*>(vp_lo + 32 * c * VSB + 32 * bb);
            }
#pragma unroll
            for (int c = 0; c < 4; c++) o[c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah[c], ph.h, o[c], 0, 0, 0);
#pragma unroll
            for (int c = 0; c < 4; c++) o[c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah[c], pl.h, o[c], 0, 0, 0);
            if (LO) {
#pragma unroll
                for (int c = 0; c < 4; c++) o[c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(al[c], ph.h, o[c], 0, 0, 0);
            }
        }
        }  // (tile visible to the wave)
        if (kv_pair + 2 * BK < kv_end) {
            LLMOPS_STAGE_STORE(sm2[(pass + 1) & 1]);
            if (kv_pair + 4 * BK < kv_end) LLMOPS_STAGE_LOAD(kv_pair + set * BK + 4 * BK);
        }
    }

#undef LLMOPS_STAGE_STORE
#undef LLMOPS_DPP_MINMAX
#undef LLMOPS_STAGE_LOAD
    // Merge of the two sets: lane by lane (same query, same columns in both).  Set 1 leaves its running maximum, its
    // sum and its 64 outputs in LDS, value r of lane l of wave w at float r*256 + w*64 + l.
    __syncthreads();  // every wave is done with its tile
    float* mrg = reinterpret_cast<float*>(smem_raw) + wave * 64 + lane;
    if (set == 1) {
        mrg[0] = m_run;
        mrg[256] = l_run;
#pragma unroll
        for (int c = 0; c < 4; c++)
#pragma unroll
            for (int r = 0; r < 16; r++) mrg[(2 + 16 * c + r) * 256] = o[c][r];
    }
    __syncthreads();
    if (set == 1 || !valid) return;
    {
        const float m1 = mrg[0], l1 = mrg[256];
        const float mm = fmaxf(m_run, m1);
        const float a0 = expf(m_run - mm), a1 = expf(m1 - mm);  // (a set that saw no row has sum 0 and outputs 0)
        l_run = l_run * a0 + l1 * a1;
#pragma unroll
        for (int c = 0; c < 4; c++)
#pragma unroll
            for (int r = 0; r < 16; r++) o[c][r] = o[c][r] * a0 + mrg[(2 + 16 * c + r) * 256] * a1;
    }
    const float inv = 1.0f / l_run;
    // the lane holds columns 32c + 8j + 4*hf + v of its query's output row
#pragma unroll
    for (int c = 0; c < 4; c++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const float4 out = make_float4(o[c][4 * j] * inv, o[c][4 * j + 1] * inv, o[c][4 * j + 2] * inv, o[c][4 * j + 3] * inv);
            *reinterpret_cast<float4*>(qrow + 32 * c + 8 * j + 4 * hf) = out;
        }
}

// ---- softmax op (ops/op_misc.hpp:183-194): one workgroup per row ------------------------------
__global__ __launch_bounds__(256) void softmax_kernel(float* __restrict__ x, int64_t K) {
    __shared__ float red[4];
    float* row = x + (int64_t)blockIdx.x * K;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float mx = -FLT_MAX;
    for (int64_t i = threadIdx.x; i < K; i += 256) mx = fmaxf(mx, row[i]);
    mx = wave_max(mx);
    if (lane == 0) red[wave] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    __syncthreads();
    float sum = 0.0f;
    for (int64_t i = threadIdx.x; i < K; i += 256) {
        const float ex = expf(row[i] - mx);
        row[i] = ex;
        sum += ex;
    }
    sum = wave_sum(sum);
    if (lane == 0) red[wave] = sum;
    __syncthreads();
    const float scale = 1.0f / (((red[0] + red[1]) + red[2]) + red[3]);
    for (int64_t i = threadIdx.x; i < K; i += 256) row[i] *= scale;
}

static inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

static int g_prefill_min_tokens = 32;  // query tokens per call from which the tiled MFMA kernel is used

static int pick_pw(int64_t bhq, int64_t kvLen) {
    // smallest chunk count that still gives ~1024 workgroups; chunk = 4*PW rows
    for (int pw : {16, 8, 4}) {
        const int64_t chunks = (kvLen + 4 * pw - 1) / (4 * pw);
        if (bhq * chunks >= 1024 || pw == 4) return pw;
    }
    return 4;
}

// cache rows per chunk when the chunk records go to the consumer FC (at most kAttnRecChunks chunks per head): 0 = the
// cache is too long for that
static int records_chunk_rows(int64_t maxlen, bool half_cache) {
    if (maxlen <= kAttnRecChunks * 256) return 256;
    if (half_cache && maxlen <= kAttnRecChunks * 512) return 512;
    return 0;
}

// Decode (one query token): cache rows per wavefront (a chunk is 4 times that).  g_decode_pw forces it (tests,
// measurements); 0 = choose.
static int g_decode_pw = 0;
struct DecodePlan {
    int pw;
};
static DecodePlan plan_decode(int64_t bh, int64_t kv, bool half_cache, int64_t max_records) {
    // fp32 rows are 32 lanes wide (2 rows per wave-wide load), fp16 rows 16 lanes (4 rows): 2..8 loads per lane
    const int lo = half_cache ? 8 : 4, hi = half_cache ? 32 : 16;
    auto chunks = [&](int pw) { return (kv + 4 * pw - 1) / (4 * pw); };
    // Chunks of 4 wavefronts, merged by a second launch: the largest chunk that still gives 256
    // workgroups, and 512 for the two larger chunk sizes (measured, us, fp32: kv 256 -- 16/32/64-row chunks 8.6 / 8.2 /
    // 9.3; kv 512 -- 11.1 / 10.1 / 10.3; kv 1024 -- 15.1 / 13.3 / 13.1; kv 2048 -- 30.7 / 19.7 / 19.0)
    DecodePlan p{lo};
    for (int pw = hi; pw >= lo; pw >>= 1)
        if (bh * chunks(pw) >= (pw > 2 * lo ? 512 : 256)) {
            p.pw = pw;
            break;
        }
    if (g_decode_pw >= lo && g_decode_pw <= hi && (g_decode_pw & (g_decode_pw - 1)) == 0) p.pw = g_decode_pw;
    while (p.pw < hi && bh * chunks(p.pw) > max_records) p.pw <<= 1;  // the records must fit the workspace
    return p;
}

}  // namespace llmops

using namespace llmops;

extern "C" int llmops_rope_embed(float* x, int64_t B, int64_t H, int64_t L, int64_t S, const float* inv_freq,
                                 int64_t half, int position_id, llmops_stream_t stream) {
    LLMOPS_REQUIRE(x != nullptr && inv_freq != nullptr);
    LLMOPS_REQUIRE(B > 0 && H > 0 && L > 0 && S > 0 && half > 0 && 2 * half <= S);
    const int64_t total = B * H * L * half;
    rope_kernel<<<(unsigned)((total + 255) / 256), 256, 0, as_stream(stream)>>>(x, B * H, L, S, inv_freq, half, position_id);
    LLMOPS_LAUNCH_CHECK();
    return LLMOPS_OK;
}

extern "C" size_t llmops_attention_workspace_bytes(int64_t B, int64_t qL, int64_t H, int64_t S, int64_t maxlen) {
    if (B <= 0 || qL <= 0 || H <= 0 || S <= 0 || maxlen <= 0) return 0;
    // the planners use 64-row chunks (128 with an fp16 cache) unless that gives fewer than 1024 workgroups, and the
    // finer chunkings they then fall back to stay below 2048 workgroups; a plan that does not fit is coarsened
    const int64_t bhq = B * H * qL;
    int64_t records = bhq * ((maxlen + 63) / 64);
    if (records < 2048) records = 2048;
    return LLMOPS_ATTN_COUNTER_BYTES + align_up((size_t)maxlen * sizeof(int32_t), 256) +
           (size_t)records * (S + 2) * sizeof(float);
}

template <typename T>
static int attention_impl(float* q, float* k, const float* v, int64_t B, int64_t qL, int64_t H, int64_t S,
                          const float* inv_freq, int64_t half, T* cache, int64_t maxlen, const int32_t* slots,
                          int position_id, const int32_t* pos_dev, int layer_id, void* workspace, size_t workspace_bytes,
                          hipStream_t st, float* rec_stats = nullptr, float* rec_outs = nullptr) {
    constexpr bool kHalfCache = sizeof(T) == 2;
    T* kc = cache + (int64_t)(2 * layer_id + 0) * B * H * maxlen * S;
    T* vc = cache + (int64_t)(2 * layer_id + 1) * B * H * maxlen * S;
    uint8_t* wsb = reinterpret_cast<uint8_t*>(workspace);
    int32_t* row_token = reinterpret_cast<int32_t*>(wsb + LLMOPS_ATTN_COUNTER_BYTES);
    const size_t part_off = LLMOPS_ATTN_COUNTER_BYTES + align_up((size_t)maxlen * 4, 256);
    float* part = reinterpret_cast<float*>(wsb + part_off);
    const int64_t max_records = (int64_t)((workspace_bytes - part_off) / ((S + 2) * sizeof(float)));
    int64_t kvLen = (int64_t)position_id + qL;
    if (kvLen > maxlen) kvLen = maxlen;
    const int64_t bhq = B * H * qL;
    if (rec_stats != nullptr) {
        // decode with the merge left to the consumer: 16 wavefronts x 16 rows per chunk, or x 32 with an fp16 cache
        // longer than 2048 rows
        const int64_t kv_plan = pos_dev ? maxlen : kvLen;
        const int rows = records_chunk_rows(maxlen, kHalfCache);
        if (qL != 1 || (half % 4) != 0 || rows == 0) return fail(LLMOPS_EINVAL, "chunk records need one query token, half %% 4 == 0 and a cache of at most %d rows", kAttnRecChunks * (kHalfCache ? 512 : 256));
        const int nchunks = (int)((kv_plan + rows - 1) / rows);
        if (bhq > 65535 || maxlen * S * (int64_t)sizeof(T) >= ((int64_t)1 << 32))
            return fail(LLMOPS_EINVAL, "decode attention: at most 65535 heads in all and a cache plane per head below 4 GiB");
        const dim3 grid((unsigned)nchunks, (unsigned)bhq);
        if (rows == 256)
            attn_decode_kernel<T, 16, 16, true><<<grid, 1024, 0, st>>>(pos_dev, position_id, nchunks, (int)maxlen, kc, vc, slots, q, k, v,
                                                                       inv_freq, (int)half, nullptr, rec_stats, rec_outs);
        else if constexpr (kHalfCache)
            attn_decode_kernel<T, 32, 16, true><<<grid, 1024, 0, st>>>(pos_dev, position_id, nchunks, (int)maxlen, kc, vc, slots, q, k, v,
                                                                       inv_freq, (int)half, nullptr, rec_stats, rec_outs);
        LLMOPS_LAUNCH_CHECK();
        return LLMOPS_OK;
    }
    // (the decode kernels index heads with the grid's y dimension: more than 65535 heads in all take the general
    // path below, which the position in device memory cannot)
    if (qL == 1 && (half % 4) == 0 && (bhq <= 65535 || pos_dev != nullptr)) {
        // decode: rope, cache update and split-KV attention in one launch, then the merge of the chunk records
        // (none when a head has a single chunk).  With the position in device memory the launch is sized for a
        // full cache.
        const int64_t kv_plan = pos_dev ? maxlen : kvLen;
        const DecodePlan p = plan_decode(bhq, kv_plan, kHalfCache, max_records);
        const int nchunks = (int)((kv_plan + 4 * p.pw - 1) / (4 * p.pw));
        if ((int64_t)bhq * nchunks > max_records)
            return fail(LLMOPS_EWORKSPACE, "attention workspace too small for %lld chunk records", (long long)bhq * nchunks);
        if (bhq > 65535 || maxlen * S * (int64_t)sizeof(T) >= ((int64_t)1 << 32))
            return fail(LLMOPS_EINVAL, "decode attention: at most 65535 heads in all and a cache plane per head below 4 GiB");
        const dim3 grid((unsigned)nchunks, (unsigned)bhq);
#define LLMOPS_DECODE(PWV)                                                                                         \
    attn_decode_kernel<T, PWV><<<grid, 256, 0, st>>>(pos_dev, position_id, nchunks, (int)maxlen, kc, vc, slots, q, k, v, inv_freq, \
                                                     (int)half, part)
        switch (p.pw) {
            case 4: if constexpr (!kHalfCache) LLMOPS_DECODE(4); break;
            case 8: LLMOPS_DECODE(8); break;
            case 16: LLMOPS_DECODE(16); break;
            case 32: if constexpr (kHalfCache) LLMOPS_DECODE(32); break;
        }
#undef LLMOPS_DECODE
        LLMOPS_LAUNCH_CHECK();
        if (nchunks > 1) {
            attn_merge_kernel<<<(unsigned)bhq, 128, 0, st>>>(q, part, qL, H, nchunks, 4 * p.pw, pos_dev, maxlen);
            LLMOPS_LAUNCH_CHECK();
        }
        return LLMOPS_OK;
    }
    if (pos_dev != nullptr) return fail(LLMOPS_EINVAL, "a position in device memory needs one query token and half %% 4 == 0");
    const int pw = pick_pw(bhq, kvLen);
    const int nchunks = (int)((kvLen + 4 * pw - 1) / (4 * pw));
    const unsigned grid = (unsigned)(bhq * nchunks);
    if (qL > 1) {
        fill_i32_kernel<<<(unsigned)((maxlen + 255) / 256), 256, 0, st>>>(row_token, maxlen, -1);
        LLMOPS_LAUNCH_CHECK();
    }
    attn_prep_kernel<T><<<(unsigned)(B * qL * H), 64, 0, st>>>(q, k, v, qL, H, S, inv_freq, half, kc, vc, maxlen, slots,
                                                              position_id, row_token);
    LLMOPS_LAUNCH_CHECK();
    if (qL >= g_prefill_min_tokens) {
        // enough query tokens to share K/V tiles: the MFMA kernel reads the cache once per 128 queries
        if (maxlen * S * (int64_t)sizeof(T) >= ((int64_t)1 << 32))
            return fail(LLMOPS_EINVAL, "attention over 32 or more query tokens: a head's cache plane must be below 4 GiB");
        const int qtiles = (int)((qL + 127) / 128);
        constexpr size_t smem = prefill_smem_bytes<!kHalfCache>();
        static bool configured = false;  // opt in to more than 64 KiB of dynamic LDS once per kernel
        if (!configured) {
            LLMOPS_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_prefill_kernel<T>),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
            configured = true;
        }
        attn_prefill_kernel<T><<<(unsigned)(B * H * qtiles), 512, smem, st>>>(q, kc, vc, qL, H, maxlen, kvLen, row_token, qtiles);
        LLMOPS_LAUNCH_CHECK();
        return LLMOPS_OK;
    }
    if ((int64_t)bhq * nchunks > max_records) return fail(LLMOPS_EWORKSPACE, "attention workspace too small for %lld chunk records", (long long)bhq * nchunks);
    if (pw == 16)
        attn_split_kernel<T, 16><<<grid, 256, 0, st>>>(q, kc, vc, qL, H, maxlen, kvLen, row_token, part, nchunks);
    else if (pw == 8)
        attn_split_kernel<T, 8><<<grid, 256, 0, st>>>(q, kc, vc, qL, H, maxlen, kvLen, row_token, part, nchunks);
    else
        attn_split_kernel<T, 4><<<grid, 256, 0, st>>>(q, kc, vc, qL, H, maxlen, kvLen, row_token, part, nchunks);
    LLMOPS_LAUNCH_CHECK();
    attn_merge_kernel<<<(unsigned)bhq, 128, 0, st>>>(q, part, qL, H, nchunks);
    LLMOPS_LAUNCH_CHECK();
    return LLMOPS_OK;
}

static int attention_entry(float* q, float* k, const float* v, int64_t B, int64_t qL, int64_t H, int64_t S,
                           const float* inv_freq, int64_t half, void* kv_cache, int cache_dtype, int64_t planes,
                           int64_t maxlen, const int32_t* slots, int position_id, const int32_t* pos_dev, int layer_id,
                           void* workspace, size_t workspace_bytes, llmops_stream_t stream, float* rec_stats = nullptr,
                           float* rec_outs = nullptr) {
    LLMOPS_REQUIRE(q != nullptr && k != nullptr && v != nullptr && inv_freq != nullptr && kv_cache != nullptr);
    LLMOPS_REQUIRE(slots != nullptr && workspace != nullptr);
    LLMOPS_REQUIRE(B > 0 && qL > 0 && H > 0 && maxlen > 0);
    LLMOPS_REQUIRE(S == 128);  // head size of every supported model shape (the reference needs S % 16 == 0)
    LLMOPS_REQUIRE(half > 0 && 2 * half <= S);
    LLMOPS_REQUIRE(layer_id >= 0 && 2 * (int64_t)layer_id + 1 < planes);
    LLMOPS_REQUIRE(position_id >= 0);
    LLMOPS_REQUIRE(cache_dtype == LLMOPS_CACHE_F32 || cache_dtype == LLMOPS_CACHE_F16);
    LLMOPS_REQUIRE(aligned(q, 16) && aligned(k, 16) && aligned(v, 16) && aligned(kv_cache, 16) && aligned(workspace, 256));
    LLMOPS_REQUIRE(B * H * qL * ((maxlen + 63) / 64) < ((int64_t)1 << 31));
    const size_t need = llmops_attention_workspace_bytes(B, qL, H, S, maxlen);
    if (workspace_bytes < need)
        return fail(LLMOPS_EWORKSPACE, "attention_rope needs %zu workspace bytes, got %zu", need, workspace_bytes);
    hipStream_t st = as_stream(stream);
    if (cache_dtype == LLMOPS_CACHE_F32)
        return attention_impl<float>(q, k, v, B, qL, H, S, inv_freq, half, reinterpret_cast<float*>(kv_cache), maxlen, slots,
                                     position_id, pos_dev, layer_id, workspace, workspace_bytes, st, rec_stats, rec_outs);
    return attention_impl<__half>(q, k, v, B, qL, H, S, inv_freq, half, reinterpret_cast<__half*>(kv_cache), maxlen, slots,
                                  position_id, pos_dev, layer_id, workspace, workspace_bytes, st, rec_stats, rec_outs);
}

extern "C" int llmops_attention_rope(float* q, float* k, const float* v, int64_t B, int64_t qL, int64_t H, int64_t S,
                                     const float* inv_freq, int64_t half, void* kv_cache, int cache_dtype,
                                     int64_t planes, int64_t maxlen, const int32_t* slots, int position_id,
                                     int layer_id, void* workspace, size_t workspace_bytes, llmops_stream_t stream) {
    return attention_entry(q, k, v, B, qL, H, S, inv_freq, half, kv_cache, cache_dtype, planes, maxlen, slots, position_id,
                           nullptr, layer_id, workspace, workspace_bytes, stream);
}

extern "C" int llmops_attention_rope_decode(float* q, float* k, const float* v, int64_t B, int64_t H, int64_t S,
                                            const float* inv_freq, int64_t half, void* kv_cache, int cache_dtype,
                                            int64_t planes, int64_t maxlen, const int32_t* slot,
                                            const int32_t* position_id, int layer_id, void* workspace,
                                            size_t workspace_bytes, llmops_stream_t stream) {
    LLMOPS_REQUIRE(position_id != nullptr && (half % 4) == 0);
    return attention_entry(q, k, v, B, 1, H, S, inv_freq, half, kv_cache, cache_dtype, planes, maxlen, slot, 0, position_id,
                           layer_id, workspace, workspace_bytes, stream);
}

extern "C" int64_t llmops_attention_records_chunks(int64_t maxlen, int cache_dtype) {
    return records_chunk_rows(maxlen, cache_dtype == LLMOPS_CACHE_F16) ? kAttnRecChunks : 0;
}

extern "C" int64_t llmops_attention_records_chunk_rows(int64_t maxlen, int cache_dtype) {
    return records_chunk_rows(maxlen, cache_dtype == LLMOPS_CACHE_F16);
}

extern "C" int llmops_attention_rope_decode_records(float* q, float* k, const float* v, int64_t B, int64_t H, int64_t S,
                                                    const float* inv_freq, int64_t half, void* kv_cache, int cache_dtype,
                                                    int64_t planes, int64_t maxlen, const int32_t* slot, int position_id,
                                                    const int32_t* position_id_dev, int layer_id, float* rec_stats,
                                                    float* rec_outs, void* workspace, size_t workspace_bytes,
                                                    llmops_stream_t stream) {
    LLMOPS_REQUIRE(rec_stats != nullptr && rec_outs != nullptr && aligned(rec_stats, 16) && aligned(rec_outs, 16));
    return attention_entry(q, k, v, B, 1, H, S, inv_freq, half, kv_cache, cache_dtype, planes, maxlen, slot, position_id,
                           position_id_dev, layer_id, workspace, workspace_bytes, stream, rec_stats, rec_outs);
}

extern "C" void llmops_test_attn_set_decode_plan(int rows_per_wave) {
    if (llmops::test_hooks_enabled("llmops_test_attn_set_decode_plan")) llmops::g_decode_pw = rows_per_wave;
}

extern "C" int llmops_softmax(float* x, int64_t rows, int64_t K, llmops_stream_t stream) {
    LLMOPS_REQUIRE(x != nullptr && rows > 0 && K > 0 && rows < ((int64_t)1 << 31));
    softmax_kernel<<<(unsigned)rows, 256, 0, as_stream(stream)>>>(x, K);
    LLMOPS_LAUNCH_CHECK();
    return LLMOPS_OK;
}
