// Element-wise and row-wise neighbours of the FC/attention path that one decode step needs
// (/root/reference/ops/op_misc.hpp, ops/op_embedding.hpp).  All fp32, all in place like the
// reference; each is a single bandwidth-trivial launch.
#include "common.h"

namespace llmops {

// rmsnorm (ops/op_misc.hpp:142-181): one workgroup of 1024 threads per row; the row is read once
// with 16-byte loads and kept in registers (hidden <= 4*1024*VPT), `out` may alias `x`
template <int VPT>
__global__ __launch_bounds__(1024) void rmsnorm_kernel(const float* __restrict__ x, float* out, int64_t hidden,
                                                        const float* __restrict__ w, float eps) {
    __shared__ float red[16];
    const float* row = x + (int64_t)blockIdx.x * hidden;
    float* orow = out + (int64_t)blockIdx.x * hidden;
    float4 v[VPT];
    const float rs = rmsnorm_row_scale<VPT>(row, hidden, eps, v, red);
#pragma unroll
    for (int i = 0; i < VPT; i++) {
        const int64_t e = ((int64_t)i * 1024 + threadIdx.x) * 4;
        if (e < hidden) {
            const float4 ww = *reinterpret_cast<const float4*>(w + e);
            *reinterpret_cast<float4*>(orow + e) =
                make_float4(v[i].x * rs * ww.x, v[i].y * rs * ww.y, v[i].z * rs * ww.z, v[i].w * rs * ww.w);
        }
    }
}

// general fallback (any hidden size, any alignment)
__global__ __launch_bounds__(256) void rmsnorm_generic_kernel(const float* __restrict__ x, float* out, int64_t hidden,
                                                               const float* __restrict__ w, float eps) {
    __shared__ float red[4];
    const float* row = x + (int64_t)blockIdx.x * hidden;
    float* orow = out + (int64_t)blockIdx.x * hidden;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float ss = 0.0f;
    for (int64_t i = threadIdx.x; i < hidden; i += 256) ss = fmaf(row[i], row[i], ss);
    ss = wave_sum(ss);
    if (lane == 0) red[wave] = ss;
    __syncthreads();
    const float rms = (((red[0] + red[1]) + red[2]) + red[3]) / (float)hidden;
    const float rs = 1.0f / sqrtf(rms + eps);
    __syncthreads();
    for (int64_t i = threadIdx.x; i < hidden; i += 256) orow[i] = row[i] * rs * w[i];
}

// out[r, i] = silu(gu[r, i]) * gu[r, F + i]   (itrans "silu" followed by imul, ops/op_misc.hpp:83-138,
// on a row that holds the gate and the up projection side by side)
__global__ void silu_mul_kernel(const float* __restrict__ gu, float* __restrict__ out, int64_t rows, int64_t F) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= rows * F) return;
    const int64_t r = i / F, c = i % F;
    const float g = gu[r * 2 * F + c], u = gu[r * 2 * F + F + c];
    out[i] = silu_times(g, u);
}

// the same for a row whose strips of 32 columns alternate gate, up, gate, up ... (the layout a gate|up FC over
// interleaved strips leaves behind): out[r, i] = silu(gu[r, (i/32)*64 + i%32]) * gu[r, (i/32)*64 + 32 + i%32]
__global__ void silu_mul_interleaved_kernel(const float* __restrict__ gu, float* __restrict__ out, int64_t rows, int64_t F) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= rows * F) return;
    const int64_t r = i / F, c = i % F;
    const int64_t base = r * 2 * F + (c >> 5) * 64 + (c & 31);
    out[i] = silu_times(gu[base], gu[base + 32]);
}

// sum of squares of every strip of 32 columns of y [rows, N] (columns beyond N count as 0): out [rows, Ng].
// One half-wave per (row, strip).  What the decode FC's epilogue hands to the next rmsnorm, for many rows.
__global__ __launch_bounds__(256) void strip_sumsq_kernel(const float* __restrict__ y, int64_t rows, int64_t N, int64_t Ng,
                                                           float* __restrict__ out) {
    const int64_t item = ((int64_t)blockIdx.x * 256 + threadIdx.x) >> 5;
    const int c = threadIdx.x & 31;
    const bool live = item < rows * Ng;
    const int64_t r = live ? item / Ng : 0, nb = live ? item % Ng : 0;
    const int64_t n = nb * 32 + c;
    const float v = (live && n < N) ? y[r * N + n] : 0.0f;
    float sq = v * v;
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) sq += __shfl_xor(sq, o, 64);
    if (live && c == 0) out[r * Ng + nb] = sq;
}

template <bool MUL>
__global__ void ibinary_kernel(float* __restrict__ a, const float* __restrict__ b, int64_t total, int64_t inner,
                               int b_is_row) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const float bv = b[b_is_row ? i % inner : i];
    a[i] = MUL ? a[i] * bv : a[i] + bv;
}

// itrans "silu" (ops/op_misc.hpp:127-138): x * 1/(1+exp(-x)), exact reciprocal
__global__ void silu_kernel(float* __restrict__ a, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float v = a[i];
    a[i] = v * (1.0f / (1.0f + expf(-v)));
}

// embedding_q8c_quant_w (ops/op_embedding.hpp:51-78): per-row amax/127 scale, RNE int8 codes
__global__ __launch_bounds__(256) void emb_quant_kernel(const float* __restrict__ w, int64_t E, int8_t* __restrict__ q,
                                                         float* __restrict__ scales) {
    __shared__ float red[4];
    const float* row = w + (int64_t)blockIdx.x * E;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float amax = 0.0f;
    for (int64_t i = threadIdx.x; i < E; i += 256) amax = fmaxf(amax, fabsf(row[i]));
    amax = wave_max(amax);
    if (lane == 0) red[wave] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    const float d = amax / 127.0f;
    const float id = (d != 0.0f) ? (1.0f / d) : 0.0f;
    if (threadIdx.x == 0) scales[blockIdx.x] = d;
    const int64_t vec = E & ~(int64_t)7;  // the reference's scalar tail rounds half away (ops/utils.hpp:217-219)
    for (int64_t i = threadIdx.x; i < E; i += 256) {
        const float t = row[i] * id;
        float r = (i < vec) ? rintf(t) : roundf(t);
        r = fminf(127.0f, fmaxf(-128.0f, r));
        q[(int64_t)blockIdx.x * E + i] = (t != t) ? (int8_t)-128 : (int8_t)(int)r;
    }
}

// embedding_q8c (ops/op_embedding.hpp:81-137): out[i,:] = scales[id] * q[id,:]
__global__ void emb_q8c_kernel(float* __restrict__ out, const int64_t* __restrict__ ids, const int8_t* __restrict__ q,
                               const float* __restrict__ scales, int64_t E) {
    const int64_t id = ids[blockIdx.x];
    const float s = scales[id];
    for (int64_t e = threadIdx.x; e < E; e += blockDim.x) out[(int64_t)blockIdx.x * E + e] = s * (float)q[id * E + e];
}

// The same with E a multiple of 4 and 4-byte aligned rows: four codes per thread, blockIdx.y walks the row, so a
// single token's row is one round of independent loads instead of a loop in one workgroup.
__global__ __launch_bounds__(256) void emb_q8c_vec_kernel(float* __restrict__ out, const int64_t* __restrict__ ids,
                                                          const int8_t* __restrict__ q, const float* __restrict__ scales,
                                                          int64_t E) {
    const int64_t e = ((int64_t)blockIdx.y * 256 + threadIdx.x) * 4;
    if (e >= E) return;
    const int64_t id = ids[blockIdx.x];
    const float s = scales[id];
    const uint32_t c = *reinterpret_cast<const uint32_t*>(q + id * E + e);
    float4 v;
    v.x = s * (float)(int8_t)(c & 0xFFu);
    v.y = s * (float)(int8_t)((c >> 8) & 0xFFu);
    v.z = s * (float)(int8_t)((c >> 16) & 0xFFu);
    v.w = s * (float)(int8_t)(c >> 24);
    *reinterpret_cast<float4*>(out + (int64_t)blockIdx.x * E + e) = v;
}

// embedding (ops/op_embedding.hpp:24-49): out[i,:] = w[ids[i],:]
__global__ void emb_kernel(float* __restrict__ out, const int64_t* __restrict__ ids, const float* __restrict__ w, int64_t E) {
    const int64_t id = ids[blockIdx.x];
    for (int64_t e = threadIdx.x; e < E; e += blockDim.x) out[(int64_t)blockIdx.x * E + e] = w[id * E + e];
}

}  // namespace llmops

using namespace llmops;

namespace llmops {
int launch_strip_sumsq(const float* y, int64_t rows, int64_t N, float* out, hipStream_t st);
}

static int rmsnorm_launch(const float* x, float* out, int64_t rows, int64_t hidden, const float* w, float eps,
                          llmops_stream_t stream) {
    LLMOPS_REQUIRE(x != nullptr && out != nullptr && w != nullptr && rows > 0 && hidden > 0 && rows < ((int64_t)1 << 31));
    hipStream_t st = as_stream(stream);
    const bool vec = (hidden % 4) == 0 && aligned(x, 16) && aligned(out, 16) && aligned(w, 16);
    if (vec && hidden <= 4096)
        rmsnorm_kernel<1><<<(unsigned)rows, 1024, 0, st>>>(x, out, hidden, w, eps);
    else if (vec && hidden <= 8192)
        rmsnorm_kernel<2><<<(unsigned)rows, 1024, 0, st>>>(x, out, hidden, w, eps);
    else if (vec && hidden <= 16384)
        rmsnorm_kernel<4><<<(unsigned)rows, 1024, 0, st>>>(x, out, hidden, w, eps);
    else
        rmsnorm_generic_kernel<<<(unsigned)rows, 256, 0, st>>>(x, out, hidden, w, eps);
    LLMOPS_LAUNCH_CHECK();
    return LLMOPS_OK;
}

extern "C" int llmops_rmsnorm(float* x, int64_t rows, int64_t hidden, const float* w, float eps, llmops_stream_t stream) {
    return rmsnorm_launch(x, x, rows, hidden, w, eps, stream);
}

extern "C" int llmops_rmsnorm_out(const float* x, float* out, int64_t rows, int64_t hidden, const float* w, float eps,
                                  llmops_stream_t stream) {
    return rmsnorm_launch(x, out, rows, hidden, w, eps, stream);
}

extern "C" int llmops_silu_mul(const float* gate_up, float* out, int64_t rows, int64_t F, llmops_stream_t stream) {
    LLMOPS_REQUIRE(gate_up != nullptr && out != nullptr && rows > 0 && F > 0);
    const int64_t total = rows * F;
    LLMOPS_REQUIRE((total + 255) / 256 < ((int64_t)1 << 31));
    silu_mul_kernel<<<(unsigned)((total + 255) / 256), 256, 0, as_stream(stream)>>>(gate_up, out, rows, F);
    LLMOPS_LAUNCH_CHECK();
    return LLMOPS_OK;
}

extern "C" int llmops_silu_mul_interleaved(const float* gate_up, float* out, int64_t rows, int64_t F, llmops_stream_t stream) {
    LLMOPS_REQUIRE(gate_up != nullptr && out != nullptr && rows > 0 && F > 0 && (F % 32) == 0);
    const int64_t total = rows * F;
    LLMOPS_REQUIRE((total + 255) / 256 < ((int64_t)1 << 31));
    silu_mul_interleaved_kernel<<<(unsigned)((total + 255) / 256), 256, 0, as_stream(stream)>>>(gate_up, out, rows, F);
    LLMOPS_LAUNCH_CHECK();
    return LLMOPS_OK;
}

extern "C" int llmops_strip_sumsq(const float* y, int64_t rows, int64_t N, float* out, llmops_stream_t stream) {
    LLMOPS_REQUIRE(y != nullptr && out != nullptr && rows > 0 && N > 0);
    return launch_strip_sumsq(y, rows, N, out, as_stream(stream));
}

namespace llmops {
int launch_strip_sumsq(const float* y, int64_t rows, int64_t N, float* out, hipStream_t st) {
    const int64_t Ng = (N + 31) / 32, threads = rows * Ng * 32;
    if ((threads + 255) / 256 >= ((int64_t)1 << 31)) return fail(LLMOPS_EINVAL, "strip_sumsq: too many strips for one launch");
    strip_sumsq_kernel<<<(unsigned)((threads + 255) / 256), 256, 0, st>>>(y, rows, N, Ng, out);
    LLMOPS_LAUNCH_CHECK();
    return LLMOPS_OK;
}
int launch_add(float* a, const float* b, int64_t total, hipStream_t st) {
    ibinary_kernel<false><<<(unsigned)((total + 255) / 256), 256, 0, st>>>(a, b, total, total, 0);
    LLMOPS_LAUNCH_CHECK();
    return LLMOPS_OK;
}
}  // namespace llmops

static int ibinary(bool mul, float* a, const float* b, int64_t rows, int64_t inner, int b_is_row, llmops_stream_t stream) {
    LLMOPS_REQUIRE(a != nullptr && b != nullptr && rows > 0 && inner > 0);
    const int64_t total = rows * inner;
    LLMOPS_REQUIRE((total + 255) / 256 < ((int64_t)1 << 31));
    const unsigned grid = (unsigned)((total + 255) / 256);
    if (mul)
        ibinary_kernel<true><<<grid, 256, 0, as_stream(stream)>>>(a, b, total, inner, b_is_row);
    else
        ibinary_kernel<false><<<grid, 256, 0, as_stream(stream)>>>(a, b, total, inner, b_is_row);
    LLMOPS_LAUNCH_CHECK();
    return LLMOPS_OK;
}

extern "C" int llmops_iadd(float* a, const float* b, int64_t rows, int64_t inner, int b_is_row, llmops_stream_t stream) {
    return ibinary(false, a, b, rows, inner, b_is_row, stream);
}
extern "C" int llmops_imul(float* a, const float* b, int64_t rows, int64_t inner, int b_is_row, llmops_stream_t stream) {
    return ibinary(true, a, b, rows, inner, b_is_row, stream);
}

extern "C" int llmops_itrans_silu(float* a, int64_t n, llmops_stream_t stream) {
    LLMOPS_REQUIRE(a != nullptr && n > 0 && (n + 255) / 256 < ((int64_t)1 << 31));
    silu_kernel<<<(unsigned)((n + 255) / 256), 256, 0, as_stream(stream)>>>(a, n);
    LLMOPS_LAUNCH_CHECK();
    return LLMOPS_OK;
}

extern "C" int llmops_embedding_q8c_quant_w(const float* w, int64_t V, int64_t E, int8_t* q, float* scales,
                                            llmops_stream_t stream) {
    LLMOPS_REQUIRE(w != nullptr && q != nullptr && scales != nullptr && V > 0 && E > 0 && V < ((int64_t)1 << 31));
    emb_quant_kernel<<<(unsigned)V, 256, 0, as_stream(stream)>>>(w, E, q, scales);
    LLMOPS_LAUNCH_CHECK();
    return LLMOPS_OK;
}

extern "C" int llmops_embedding_q8c(float* out, const int64_t* ids, int64_t n, const int8_t* q, const float* scales,
                                    int64_t V, int64_t E, llmops_stream_t stream) {
    (void)V;
    LLMOPS_REQUIRE(out != nullptr && ids != nullptr && q != nullptr && scales != nullptr && n > 0 && E > 0);
    LLMOPS_REQUIRE(n < ((int64_t)1 << 31));
    if ((E % 4) == 0 && aligned(q, 4) && aligned(out, 16) && (E + 1023) / 1024 < 65536)
        emb_q8c_vec_kernel<<<dim3((unsigned)n, (unsigned)((E + 1023) / 1024)), 256, 0, as_stream(stream)>>>(out, ids, q, scales, E);
    else
        emb_q8c_kernel<<<(unsigned)n, 256, 0, as_stream(stream)>>>(out, ids, q, scales, E);
    LLMOPS_LAUNCH_CHECK();
    return LLMOPS_OK;
}

extern "C" int llmops_embedding(float* out, const int64_t* ids, int64_t n, const float* w, int64_t V, int64_t E,
                                llmops_stream_t stream) {
    (void)V;
    LLMOPS_REQUIRE(out != nullptr && ids != nullptr && w != nullptr && n > 0 && E > 0 && n < ((int64_t)1 << 31));
    emb_kernel<<<(unsigned)n, 256, 0, as_stream(stream)>>>(out, ids, w, E);
    LLMOPS_LAUNCH_CHECK();
    return LLMOPS_OK;
}
