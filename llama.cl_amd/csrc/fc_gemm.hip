// Q4_1 x Q8 fully-connected product for many activation rows (prefill): int8 MFMA.
//
// A wavefront owns two adjacent strips (64 output columns) and RT tiles of 16 activation rows.
// Operand layout of v_mfma_i32_16x16x{64,32}_i8: lane = 16*g + jj; the A lane holds row jj,
// the B lane holds column jj, both for the same set of k-values chosen by g.  The packed
// format gives, per 16-byte load, 4 adjacent columns x 8 k-values of one k8-row.  So lane
// (g, jj) loads the k8-rows that belong to g for columns 4*(jj&7)..+3 of strip (jj>>3); dword c
// of that load is the lane's B operand for MFMA number c, whose 16 tile columns are
// { strip (jj>>3), column 4*(jj&7)+c }.  Unpacking is two ANDs and a shift per dword; nothing is
// shuffled between lanes and the weights never pass through LDS.
//   G=128: one MFMA 16x16x64 covers 8 k8-rows (g owns rows 2g,2g+1 = 16 consecutive k);
//          two of them make one k-group.
//   G=32 : one MFMA 16x16x32 covers the group's 4 k8-rows (g owns row g = 8 consecutive k).
// After every k-group the int32 tile is folded into fp32 accumulators:
//   f += (d[n]*dx[row]) * float(acc) ; f += m[n]*gsum[row]        (fc_Q4A,
//   /root/reference/ops/op_fc.hpp:381-412; min term is m * raw group sum).
// The group-128 kernels with LDS tiles compute the first term as fma(fma(X, d, -B*d), dx, f): their
// int32 sums start at the bit pattern of the float B = 1.5 * 2^23, so the sum's register, read as a
// float X, IS B + sum (|sum| <= 128*15*127 < 2^22), and X*d - B*d = sum*d is exact before the fma's
// one rounding because B*d (2 significant bits times the 11 of an fp16) is itself a float.  Two
// vector instructions per output element and k-group instead of three (convert, multiply, fma).
// Result tile layout of the 16x16 MFMAs: lane holds column jj, rows 4*g+v in register v.
#include "common.h"
#include "gemv_device.h"

namespace llmops {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kFoldBiasBits = 0x4B400000;  // the float 1.5 * 2^23 ...
constexpr float kFoldBias = 12582912.0f;   // ... whose low mantissa bits count in units of 1

__device__ __forceinline__ uint32_t lo4(uint32_t w) { return w & 0x0F0F0F0Fu; }
__device__ __forceinline__ uint32_t hi4(uint32_t w) { return (w >> 4) & 0x0F0F0F0Fu; }

template <int G>
struct GemmTraits;
template <>
struct GemmTraits<128> {
    static constexpr int kSteps = 2;  // MFMAs per k-group
};
template <>
struct GemmTraits<32> {
    static constexpr int kSteps = 1;
};

// acc[t][c] += A(row tile t) x B(column set c) over one k-group
template <int G, int RT>
__device__ __forceinline__ void mma_group(const uint8_t* blk, const int8_t* const xrow[RT], int64_t kofs, int g, int q,
                                          v4i acc[RT][4]) {
    if (G == 128) {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const uint4 wa = *reinterpret_cast<const uint4*>(blk + h * 1024 + (2 * g) * kRowBytes + q * 16);
            const uint4 wb = *reinterpret_cast<const uint4*>(blk + h * 1024 + (2 * g + 1) * kRowBytes + q * 16);
            const uint32_t* pa = reinterpret_cast<const uint32_t*>(&wa);
            const uint32_t* pb = reinterpret_cast<const uint32_t*>(&wb);
            v4i b[4];
#pragma unroll
            for (int c = 0; c < 4; c++) {
                b[c][0] = (int)lo4(pa[c]);
                b[c][1] = (int)hi4(pa[c]);
                b[c][2] = (int)lo4(pb[c]);
                b[c][3] = (int)hi4(pb[c]);
            }
#pragma unroll
            for (int t = 0; t < RT; t++) {
                const v4i a = *reinterpret_cast<const v4i*>(xrow[t] + kofs + h * 64 + g * 16);
#pragma unroll
                for (int c = 0; c < 4; c++) acc[t][c] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b[c], acc[t][c], 0, 0, 0);
            }
        }
    } else {
        const uint4 wa = *reinterpret_cast<const uint4*>(blk + g * kRowBytes + q * 16);
        const uint32_t* pa = reinterpret_cast<const uint32_t*>(&wa);
        long b[4];
#pragma unroll
        for (int c = 0; c < 4; c++) b[c] = (long)(((uint64_t)hi4(pa[c]) << 32) | (uint64_t)lo4(pa[c]));
#pragma unroll
        for (int t = 0; t < RT; t++) {
            const long a = *reinterpret_cast<const long*>(xrow[t] + kofs + g * 8);
#pragma unroll
            for (int c = 0; c < 4; c++) acc[t][c] = __builtin_amdgcn_mfma_i32_16x16x32_i8(a, b[c], acc[t][c], 0, 0, 0);
        }
    }
}

// grid: x = ceil(pairs/4) (4 waves = 4 strip pairs per workgroup), y = row blocks of RT*16, z = k splits
template <int G, int RT>
__global__ __launch_bounds__(256) void fc_gemm_kernel(const uint8_t* __restrict__ weiq, const int8_t* __restrict__ xq,
                                                       const float* __restrict__ xd, const float* __restrict__ gs,
                                                       float* __restrict__ out, int Ng, int Kg, int64_t ldo, int64_t N,
                                                       int rows, int kb_per_split, int64_t split_stride) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane >> 4, jj = lane & 15, q = jj & 7, sp = jj >> 3;
    const int pair = blockIdx.x * 4 + wave;
    if (pair * 2 >= Ng) return;
    const int strip = pair * 2 + sp;
    const bool strip_ok = strip < Ng;
    const int strip_c = strip_ok ? strip : Ng - 1;
    const int row0 = blockIdx.y * (RT * 16);
    const int kb0 = blockIdx.z * kb_per_split, kb1 = min(Kg, kb0 + kb_per_split);
    const int64_t Kp = (int64_t)Kg * G;
    const uint8_t* sbase = weiq + (int64_t)strip_c * Kg * block_bytes(G);

    const int8_t* xrow[RT];
    int vrow[RT][4];  // clamped global row of result register v
#pragma unroll
    for (int t = 0; t < RT; t++) {
        xrow[t] = xq + (int64_t)min(rows - 1, row0 + t * 16 + jj) * Kp;
#pragma unroll
        for (int v = 0; v < 4; v++) vrow[t][v] = min(rows - 1, row0 + t * 16 + g * 4 + v);
    }

    float f[RT][4][4];
#pragma unroll
    for (int t = 0; t < RT; t++)
#pragma unroll
        for (int c = 0; c < 4; c++)
#pragma unroll
            for (int v = 0; v < 4; v++) f[t][c][v] = 0.0f;

    for (int kb = kb0; kb < kb1; kb++) {
        const uint8_t* blk = sbase + (int64_t)kb * block_bytes(G);
        v4i acc[RT][4];
#pragma unroll
        for (int t = 0; t < RT; t++)
#pragma unroll
            for (int c = 0; c < 4; c++) acc[t][c] = v4i{0, 0, 0, 0};
        mma_group<G, RT>(blk, xrow, (int64_t)kb * G, g, q, acc);

        const uint2 dh = *reinterpret_cast<const uint2*>(blk + (G / 8) * kRowBytes + q * 8);
        const uint2 mh = *reinterpret_cast<const uint2*>(blk + (G / 8) * kRowBytes + 64 + q * 8);
        float d[4], m[4];
        d[0] = f16_bits_to_f32((uint16_t)(dh.x & 0xFFFFu));
        d[1] = f16_bits_to_f32((uint16_t)(dh.x >> 16));
        d[2] = f16_bits_to_f32((uint16_t)(dh.y & 0xFFFFu));
        d[3] = f16_bits_to_f32((uint16_t)(dh.y >> 16));
        m[0] = f16_bits_to_f32((uint16_t)(mh.x & 0xFFFFu));
        m[1] = f16_bits_to_f32((uint16_t)(mh.x >> 16));
        m[2] = f16_bits_to_f32((uint16_t)(mh.y & 0xFFFFu));
        m[3] = f16_bits_to_f32((uint16_t)(mh.y >> 16));
#pragma unroll
        for (int t = 0; t < RT; t++)
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const float dx = xd[(int64_t)vrow[t][v] * Kg + kb];
                const float gsum = gs[(int64_t)vrow[t][v] * Kg + kb];
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    f[t][c][v] = fmaf(d[c] * dx, (float)acc[t][c][v], f[t][c][v]);
                    f[t][c][v] = fmaf(m[c], gsum, f[t][c][v]);
                }
            }
    }

    if (!strip_ok) return;
    float* o = out + (int64_t)blockIdx.z * split_stride;
    const int64_t n0 = (int64_t)strip * kGroupN + q * 4;
#pragma unroll
    for (int t = 0; t < RT; t++)
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const int row = row0 + t * 16 + g * 4 + v;
            if (row >= rows) continue;
#pragma unroll
            for (int c = 0; c < 4; c++)
                if (n0 + c < N) o[(int64_t)row * ldo + n0 + c] = f[t][c][v];
        }
}

// ---- split-K without a second launch -------------------------------------------------------------------
// Every split stores its tile of partial sums with device-scope (write-through) stores, waits for them and
// takes a ticket on the tile's counter; the split that draws the last ticket adds all splits' tiles in
// index order (so the sum does not depend on who arrives when), adds the residual and writes the result.
// Nobody waits for anybody.  The partial sums' row stride is a multiple of 32 floats; strips beyond Ng and
// rows beyond `rows` fall outside the buffer descriptor (loads return 0, stores are dropped).
// Called by every thread of the workgroup.  row0 / tile_rows: first row and row count of the rows this
// thread's wave group owns; wave_row: the wave's first row inside them; a thread holds rows
// wave_row + 16t + 4g + v, columns 32*strip + 4q .. + 3 in f[t][c][v].
// The last arrival works one row tile at a time with all of its loads (up to SU splits x 4 rows) in flight
// together: the reduction then costs about RT round trips to memory whatever the split count.  A split past
// the last is asked for through an empty descriptor: it returns 0 without touching memory.
template <int RT, int SU>
__device__ __forceinline__ void splitk_finish(const v4f (&f)[RT][4], float* __restrict__ out, int64_t split_stride, int64_t ldo,
                                              int row0, int tile_rows, int wave_row, int strip, int Ng, int q, int g, int rows,
                                              float* __restrict__ y_final, int64_t Ny, const float* __restrict__ residual,
                                              unsigned* counter, int tid) {
    constexpr int kAgent = 16;  // sc1: coherent at device scope, as a relaxed atomic store / load would be
    const int S = (int)gridDim.z;
    const uint32_t tile_bytes = tile_rows > 0 ? (uint32_t)tile_rows * (uint32_t)ldo * 4u : 0u;
    const uint32_t col_off = (uint32_t)(strip * kGroupN + q * 4) * 4u;
    const bool strip_ok = strip < Ng;
    {
        const buffer_rsrc rs = make_rsrc(out + (int64_t)blockIdx.z * split_stride + (int64_t)row0 * ldo, strip_ok ? tile_bytes : 0u);
#pragma unroll
        for (int t = 0; t < RT; t++)
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int r = wave_row + t * 16 + g * 4 + v;
                const u32x4 val = {__float_as_uint(f[t][0][v]), __float_as_uint(f[t][1][v]), __float_as_uint(f[t][2][v]),
                                   __float_as_uint(f[t][3][v])};
                __builtin_amdgcn_raw_buffer_store_b128(val, rs, (uint32_t)r * (uint32_t)ldo * 4u + col_off, 0, kAgent);
            }
    }
    __shared__ unsigned ticket_sh;
    __builtin_amdgcn_s_waitcnt(0);  // this wave's stores have been acknowledged
    __syncthreads();
    if (tid == 0) ticket_sh = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (ticket_sh != (unsigned)(S - 1)) return;
    if (tid == 0) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // next launch
    if (!strip_ok) return;
    const int64_t n0 = (int64_t)strip * kGroupN + q * 4;
#pragma unroll
    for (int t = 0; t < RT; t++) {
        float4 a[4];
#pragma unroll
        for (int v = 0; v < 4; v++) a[v] = make_float4(0.f, 0.f, 0.f, 0.f);
        for (int s0 = 0; s0 < S; s0 += SU) {
            u32x4 pv[SU][4];
#pragma unroll
            for (int u = 0; u < SU; u++) {
                const int sidx = min(s0 + u, S - 1);
                const buffer_rsrc rs =
                    make_rsrc(out + (int64_t)sidx * split_stride + (int64_t)row0 * ldo, s0 + u < S ? tile_bytes : 0u);
#pragma unroll
                for (int v = 0; v < 4; v++)
                    pv[u][v] = __builtin_amdgcn_raw_buffer_load_b128(
                        rs, (uint32_t)(wave_row + t * 16 + g * 4 + v) * (uint32_t)ldo * 4u + col_off, 0, kAgent);
            }
#pragma unroll
            for (int u = 0; u < SU; u++)
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    a[v].x += __uint_as_float(pv[u][v][0]), a[v].y += __uint_as_float(pv[u][v][1]);
                    a[v].z += __uint_as_float(pv[u][v][2]), a[v].w += __uint_as_float(pv[u][v][3]);
                }
        }
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const int row = row0 + wave_row + t * 16 + g * 4 + v;
            if (row >= rows) continue;
            float* dst = y_final + (int64_t)row * Ny + n0;
            const float* res = residual ? residual + (int64_t)row * Ny + n0 : nullptr;
            if (n0 + 3 < Ny && (Ny & 3) == 0) {
                float4 val = a[v];
                if (res) {
                    const float4 r4 = *reinterpret_cast<const float4*>(res);
                    val.x += r4.x, val.y += r4.y, val.z += r4.z, val.w += r4.w;
                }
                *reinterpret_cast<float4*>(dst) = val;
            } else {
                const float av[4] = {a[v].x, a[v].y, a[v].z, a[v].w};
#pragma unroll
                for (int c = 0; c < 4; c++)
                    if (n0 + c < Ny) dst[c] = res ? av[c] + res[c] : av[c];
            }
        }
    }
}

// ---- LDS-tiled kernel for group 128 ---------------------------------------------------------------
// Workgroup = 4 wavefronts (2 x 2), tile = BM rows x 128 columns (4 strips), one k-group per
// iteration.  Per iteration the workgroup stages into LDS, through registers and double buffered:
//   A : BM rows x 128 activation codes (row stride 144 B so that the 16 rows a ds_read_b128 wave
//       access touches fall into different banks)
//   B : the 4 packed blocks as they are in memory (nibbles + fp16 d + fp16 m, 2176 B each)
//   XS: (dx, gsum) of the BM rows for this k-group
// The global loads of iteration kb+1 are issued before the MFMAs of iteration kb and written to the
// other LDS buffer after them; one barrier per iteration.  Each wave owns 64 rows x 64 columns
// (RT = BM/32 row tiles x 4 column sets); operand mapping as in mma_group above, but from LDS.
constexpr int kAStride = 144;
constexpr int kBlk128 = 2176;

__device__ __forceinline__ v2f buf_ld_pair(buffer_rsrc r, uint32_t voff, uint32_t soff) {
    typedef unsigned int u32x2_g __attribute__((ext_vector_type(2)));
    const u32x2_g t = __builtin_amdgcn_raw_buffer_load_b64(r, voff, soff, 0);
    return v2f{__uint_as_float(t.x), __uint_as_float(t.y)};
}

// ---- the min term of a tile on the fp16 matrix cores -------------------------------------------------
// sum over k-groups of m[column][kg] * gsum[row][kg] is a product with K = number of k-groups.  It is
// taken out of the k-group loop and computed once per tile, 32 k-groups per MFMA, with fp32 accumulation:
// gsum = hi + lo (hi = gsum rounded toward zero to fp16, lo = the rest: 22 significant bits in all), m as
// it is stored (fp16), two MFMAs per 16x16 tile.  (The fp32 MFMA that did this inside the loop stalls the
// vector ALU for its whole duration; the fp16 one runs beside vector work.)  That is good for a row's eight
// k-groups in one lane if the largest |gsum| among them lies in [1/8, 60000]: below that lo falls into fp16's
// subnormals and the row could lose bits relative to its own size, above it hi overflows.  Zeros are exact.
// When a lane of the wave does not qualify, the wave takes the round with fp32 MFMAs instead (four k-groups
// each, exact products): the slow path, there for correctness on any input.
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
union Halves8 {
    v8h h;
    uint32_t u[4];
};

// What a lane fetches for one round of 32 k-groups (k32 .. k32+31, those below kb1): for its eight k-groups
// kgs .. kgs+7 the group sums of its row in each of RT row tiles (32 contiguous bytes of the [row][kg] matrix, which
// start on a 4-byte boundary only) and the mins of its four columns.  kgs is k32 + 8g unless that would read past
// the end of a row: then it is Kg - 8, and the slots below k32 + 8g do not count (min_term_add).
struct __attribute__((packed, aligned(4))) Float4U {
    float v[4];
};
template <int RT>
struct MinTermRound {
    Float4U ga[RT][2];
    uint2 mb[8];
};
// roff[t] = Kg * the lane's row of row tile t (clamped to the matrix); strip: its strip (clamped); q: its column
// quad.  Rows and strip count from wherever gs and weiq point (the matrix, or the workgroup's tile of it): offsets
// from there must fit 32 bits.
template <int RT>
__device__ __forceinline__ void min_term_fetch(MinTermRound<RT>& r, const float* __restrict__ gs, const int (&roff)[RT],
                                               const uint8_t* __restrict__ weiq, int Kg, int kgs, int strip, int q) {
    // (a uniform base and a 32-bit byte offset per lane: one address register per load, not two)
    const uint8_t* gb = reinterpret_cast<const uint8_t*>(gs);
#pragma unroll
    for (int t = 0; t < RT; t++) {
        const uint32_t off = (uint32_t)(roff[t] + kgs) * 4u;
        r.ga[t][0] = *reinterpret_cast<const Float4U*>(gb + off);
        r.ga[t][1] = *reinterpret_cast<const Float4U*>(gb + off + 16u);
    }
    const uint32_t moff = (uint32_t)((strip * Kg + kgs) * kBlk128 + 2112 + q * 8);
#pragma unroll
    for (int i = 0; i < 8; i++) r.mb[i] = *reinterpret_cast<const uint2*>(weiq + (moff + (uint32_t)(i * kBlk128)));
}
// f[t][c] += the round's part of the min term; operand layout of the 16x16x32 MFMA: A lane (row = lane & 15,
// k = 8 * (lane >> 4) + i), B lane (column = lane & 15, same k), D as the int8 MFMAs' (row 4g+v, column = lane & 15).
// Slot i of the lane is k-group kgs + i and counts if it lies in [lo, kb1).  FIRST: f = instead of f += (the
// accumulators then do not exist yet while the operands are fetched and examined).
template <int RT, bool FIRST>
__device__ __forceinline__ void min_term_add(v4f (&f)[RT][4], const MinTermRound<RT>& r, int kgs, int lo, int kb1) {
    const v4f zero = {0.f, 0.f, 0.f, 0.f};
    // (the slot tests are repeated where the values are used -- behind an empty asm statement, or the compiler
    // keeps the 8 * RT masked values of the first pass in registers, which do not fit beside the accumulators,
    // the operands and what the k-group loop keeps across this prologue)
#define LLMOPS_GSUM(T, I) ((kgs + (I) >= lo && kgs + (I) < kb1) ? r.ga[T][(I) >> 2].v[(I) & 3] : 0.0f)
    // (tested per lane, i.e. per row and eight k-groups, which is stricter than per row and needs no exchange)
    bool rows_fit = true;
#pragma unroll
    for (int t = 0; t < RT; t++) {
        float big = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; i++) big = fmaxf(big, fabsf(LLMOPS_GSUM(t, i)));
        rows_fit = rows_fit && (big == 0.0f || (big >= 0.125f && big <= 60000.0f));
    }
    asm volatile("" : "+v"(lo));
    if (__all(rows_fit)) {
        Halves8 m[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint2 e = r.mb[2 * j], o = r.mb[2 * j + 1];
            m[0].u[j] = __builtin_amdgcn_perm(o.x, e.x, 0x05040100u);
            m[1].u[j] = __builtin_amdgcn_perm(o.x, e.x, 0x07060302u);
            m[2].u[j] = __builtin_amdgcn_perm(o.y, e.y, 0x05040100u);
            m[3].u[j] = __builtin_amdgcn_perm(o.y, e.y, 0x07060302u);
        }
#pragma unroll
        for (int t = 0; t < RT; t++) {
            Halves8 ah, al;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const float e = LLMOPS_GSUM(t, 2 * j), o = LLMOPS_GSUM(t, 2 * j + 1);
                const v2h h = __builtin_bit_cast(v2h, __builtin_amdgcn_cvt_pkrtz(e, o));
                ah.u[j] = __builtin_bit_cast(uint32_t, h);
                al.u[j] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(e - (float)h[0], o - (float)h[1]));
            }
#pragma unroll
            for (int c = 0; c < 4; c++)
                f[t][c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(al.h, m[c].h, FIRST ? zero : f[t][c], 0, 0, 0);
#pragma unroll
            for (int c = 0; c < 4; c++) f[t][c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ah.h, m[c].h, f[t][c], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);  // one row tile's halves at a time: registers
        }
    } else {
        // slot i of the four lanes (row or column, g = 0..3) is one 16x16x4 product: k = g
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const float mc[4] = {f16_bits_to_f32((uint16_t)(r.mb[i].x & 0xFFFFu)), f16_bits_to_f32((uint16_t)(r.mb[i].x >> 16)),
                                 f16_bits_to_f32((uint16_t)(r.mb[i].y & 0xFFFFu)), f16_bits_to_f32((uint16_t)(r.mb[i].y >> 16))};
#pragma unroll
            for (int t = 0; t < RT; t++) {
                const float a = LLMOPS_GSUM(t, i);
#pragma unroll
                for (int c = 0; c < 4; c++)
                    f[t][c] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, mc[c], (FIRST && i == 0) ? zero : f[t][c], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);  // one slot's operands at a time: registers, not speed, matter here
        }
    }
#undef LLMOPS_GSUM
}

template <int RT>
struct GemmSmem {
    static constexpr int BM = RT * 32;
    uint8_t a[2][BM * kAStride];
    uint8_t b[2][4 * kBlk128];
    float2 xs[2][BM];
};

template <int RT, bool PARTIALS>
__global__ __launch_bounds__(256, (RT == 4 ? 2 : (RT == 2 ? 3 : 4))) void fc_gemm_lds_kernel(const uint8_t* __restrict__ weiq, const int8_t* __restrict__ xq,
                                                           const float* __restrict__ xd, const float* __restrict__ gs,
                                                           const float2* __restrict__ xsT, float* __restrict__ out,
                                                           int32_t* __restrict__ out_i, int Ng, int Kg, int64_t ldo,
                                                           int64_t N, int rows, int kb_per_split, int64_t split_stride,
                                                           const float* __restrict__ residual, float* __restrict__ y_final,
                                                           int64_t Ny, unsigned* __restrict__ counters) {
    constexpr int BM = RT * 32;
    constexpr int A_CHUNKS = BM * 8;                     // 16-byte chunks of the A tile
    constexpr int A_PER_THREAD = A_CHUNKS / 256;         // RT
    constexpr int B_CHUNKS = 4 * (kBlk128 / 16);         // 544
    constexpr int B_PER_THREAD = (B_CHUNKS + 255) / 256; // 3
    extern __shared__ __align__(16) uint8_t smem_raw[];
    GemmSmem<RT>& sm = *reinterpret_cast<GemmSmem<RT>*>(smem_raw);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wr = wave >> 1, wc = wave & 1;  // wave's row half / column half
    const int g = lane >> 4, jj = lane & 15, q = jj & 7, sp = jj >> 3;
    // Which tile: workgroups go to the 8 XCDs round robin, each XCD has its own L2, and an XCD runs
    // about 32 CUs x (workgroups per CU) workgroups at a time.  The tiles are therefore numbered so that
    // each XCD gets one contiguous run of them and a run walks the tile grid in bands of 8 row blocks,
    // rows fastest: the workgroups resident on one XCD then cover about 8 row blocks x 8..16 column
    // blocks and every activation and weight tile is fetched into that L2 once instead of once per
    // workgroup.  (With column blocks fastest across the whole chip the weights, re-read by every row
    // block, came from beyond the L2 each time.)
    const int nbx = (Ng + 3) / 4, nby = (rows + BM - 1) / BM;
    int bx, by;
    {
        const int total = nbx * nby, per_xcd = (total + 7) / 8;
        const int i = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
        if ((int)(blockIdx.x >> 3) >= per_xcd || i >= total) return;  // uniform for the workgroup
        constexpr int kBand = 8;
        const int band = i / (kBand * nbx), in_band = i % (kBand * nbx);
        const int first = band * kBand, rows_in_band = min(kBand, nby - first);
        by = first + in_band % rows_in_band;
        bx = in_band / rows_in_band;
    }
    const int strip0 = bx * 4;
    const int row0 = by * BM;
    const int kb0 = blockIdx.z * kb_per_split, kb1 = min(Kg, kb0 + kb_per_split);
    const int64_t Kp = (int64_t)Kg * 128;

    // ---- global -> register staging of one k-group (macros: the arrays must stay in registers) ----
    v4u ra[A_PER_THREAD], rb[B_PER_THREAD];  // native vector types: these must live in registers
    v2f rxs = {0.f, 0.f};
    // Source addresses: buffer descriptors whose base is the same for the whole workgroup, a scalar offset that advances
    // with kb, and a 32-bit offset per thread that does not depend on kb: no 64-bit address arithmetic in the loop,
    // which is bound by instruction issue (128 rows, 4096 -> 11008: 26.65 -> 26.2 us).
    const buffer_rsrc a_rs = make_rsrc(xq + (int64_t)row0 * Kp, (uint32_t)min(BM, rows - row0) * (uint32_t)Kp);
    const buffer_rsrc b_rs = make_rsrc(weiq + (int64_t)strip0 * Kg * kBlk128, (uint32_t)min(4, Ng - strip0) * (uint32_t)Kg * (uint32_t)kBlk128);
    const buffer_rsrc x_rs = make_rsrc(xsT != nullptr ? xsT : reinterpret_cast<const float2*>(xq), xsT != nullptr ? (uint32_t)Kg * (uint32_t)rows * 8u : 0u);
    uint32_t aoff[A_PER_THREAD];
    int adst[A_PER_THREAD];
#pragma unroll
    for (int i = 0; i < A_PER_THREAD; i++) {
        const int c = tid + i * 256, r = c >> 3, part = c & 7;
        aoff[i] = (uint32_t)(min(rows - 1, row0 + r) - row0) * (uint32_t)Kp + (uint32_t)(part * 16);
        adst[i] = r * kAStride + part * 16;
    }
    uint32_t boff[B_PER_THREAD];
#pragma unroll
    for (int i = 0; i < B_PER_THREAD; i++) {
        const int c = min(B_CHUNKS - 1, tid + i * 256);
        const int st = c / (kBlk128 / 16), off = c % (kBlk128 / 16);
        boff[i] = (uint32_t)(min(Ng - 1, strip0 + st) - strip0) * (uint32_t)Kg * (uint32_t)kBlk128 + (uint32_t)(off * 16);
    }
    const int64_t xrow = min(rows - 1, row0 + (tid < BM ? tid : 0));
#define LLMOPS_FETCH(KB)                                                                                              \
    do {                                                                                                              \
        _Pragma("unroll") for (int i = 0; i < A_PER_THREAD; i++) {                                                    \
            const u32x4 t_ = __builtin_amdgcn_raw_buffer_load_b128(a_rs, aoff[i], (uint32_t)(KB) * 128u, 0);          \
            ra[i] = v4u{t_.x, t_.y, t_.z, t_.w};                                                                      \
        }                                                                                                             \
        _Pragma("unroll") for (int i = 0; i < B_PER_THREAD; i++) { /* clamped offset */                               \
            const u32x4 t_ = __builtin_amdgcn_raw_buffer_load_b128(b_rs, boff[i], (uint32_t)(KB) * (uint32_t)kBlk128, 0); \
            rb[i] = v4u{t_.x, t_.y, t_.z, t_.w};                                                                      \
        }                                                                                                             \
        if (!PARTIALS)                                                                                                \
            rxs = xsT ? buf_ld_pair(x_rs, (uint32_t)xrow * 8u, (uint32_t)(KB) * (uint32_t)rows * 8u)                  \
                      : v2f{xd[xrow * Kg + (KB)], gs[xrow * Kg + (KB)]};                                            \
    } while (0)
#define LLMOPS_STASH(BUF)                                                                                  \
    do {                                                                                                   \
        _Pragma("unroll") for (int i = 0; i < A_PER_THREAD; i++)                                           \
            *reinterpret_cast<v4u*>(&sm.a[BUF][adst[i]]) = ra[i];                                          \
        _Pragma("unroll") for (int i = 0; i < B_PER_THREAD; i++)                                           \
            if (tid + i * 256 < B_CHUNKS) *reinterpret_cast<v4u*>(&sm.b[BUF][(tid + i * 256) * 16]) = rb[i]; \
        if (tid < BM) *reinterpret_cast<v2f*>(&sm.xs[BUF][tid]) = rxs;                                                            \
    } while (0)

    v4f f[RT][4];
#pragma unroll
    for (int t = 0; t < RT; t++)
#pragma unroll
        for (int c = 0; c < 4; c++) f[t][c] = v4f{0.f, 0.f, 0.f, 0.f};
    // Min term sum_kb m[n,kb]*gsum[row,kb]: a rank-Kg product, done four k-groups at a time by
    // v_mfma_f32_16x16x4_f32 straight into the fp32 accumulators (same tile layout as the int8
    // MFMAs).  Lane (jj, g) keeps gsum of row jj and m of its columns for the group with index g
    // of the current four.
    float gk[RT], mk[4];
#pragma unroll
    for (int t = 0; t < RT; t++) gk[t] = 0.0f;
#pragma unroll
    for (int c = 0; c < 4; c++) mk[c] = 0.0f;

    if (kb0 < kb1) {
        LLMOPS_FETCH(kb0);
        LLMOPS_STASH(0);
    }
    __syncthreads();

    const int strip_l = wc * 2 + sp;  // strip (0..3) of the tile this lane's B operands come from
    for (int kb = kb0; kb < kb1; kb++) {
        const int buf = (kb - kb0) & 1;
        if (kb + 1 < kb1) LLMOPS_FETCH(kb + 1);

        const uint8_t* bblk = &sm.b[buf][strip_l * kBlk128];
        const uint8_t* abase = &sm.a[buf][(wr * (BM / 2) + jj) * kAStride + g * 16];
        v4i acc[RT][4];
        // the sums start at the bit pattern of 1.5 * 2^23, so that the fold needs no convert instruction
        // (see fc_gemm_pp_kernel)
        constexpr int kInit = PARTIALS ? 0 : kFoldBiasBits;
#pragma unroll
        for (int t = 0; t < RT; t++)
#pragma unroll
            for (int c = 0; c < 4; c++) acc[t][c] = v4i{kInit, kInit, kInit, kInit};
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const uint4 wa = *reinterpret_cast<const uint4*>(bblk + h * 1024 + (2 * g) * kRowBytes + q * 16);
            const uint4 wb = *reinterpret_cast<const uint4*>(bblk + h * 1024 + (2 * g + 1) * kRowBytes + q * 16);
            const uint32_t* pa = reinterpret_cast<const uint32_t*>(&wa);
            const uint32_t* pb = reinterpret_cast<const uint32_t*>(&wb);
            v4i b[4];
#pragma unroll
            for (int c = 0; c < 4; c++) {
                b[c][0] = (int)lo4(pa[c]);
                b[c][1] = (int)hi4(pa[c]);
                b[c][2] = (int)lo4(pb[c]);
                b[c][3] = (int)hi4(pb[c]);
            }
#pragma unroll
            for (int t = 0; t < RT; t++) {
                const v4i a = *reinterpret_cast<const v4i*>(abase + t * 16 * kAStride + h * 64);
#pragma unroll
                for (int c = 0; c < 4; c++) acc[t][c] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b[c], acc[t][c], 0, 0, 0);
            }
        }

        if (PARTIALS) {
            const int strip = strip0 + strip_l;
            if (strip < Ng) {
#pragma unroll
                for (int t = 0; t < RT; t++)
#pragma unroll
                    for (int v = 0; v < 4; v++) {
                        const int row = row0 + wr * (BM / 2) + t * 16 + g * 4 + v;
                        if (row < rows) {
#pragma unroll
                            for (int c = 0; c < 4; c++)
                                out_i[((int64_t)row * ((int64_t)Ng * kGroupN) + strip * kGroupN + q * 4 + c) * Kg + kb] =
                                    acc[t][c][v];
                        }
                    }
            }
        } else {
            const uint2 dh = *reinterpret_cast<const uint2*>(bblk + 2048 + q * 8);
            const uint2 mh = *reinterpret_cast<const uint2*>(bblk + 2048 + 64 + q * 8);
            float d[4], m[4];
            d[0] = f16_bits_to_f32((uint16_t)(dh.x & 0xFFFFu));
            d[1] = f16_bits_to_f32((uint16_t)(dh.x >> 16));
            d[2] = f16_bits_to_f32((uint16_t)(dh.y & 0xFFFFu));
            d[3] = f16_bits_to_f32((uint16_t)(dh.y >> 16));
            m[0] = f16_bits_to_f32((uint16_t)(mh.x & 0xFFFFu));
            m[1] = f16_bits_to_f32((uint16_t)(mh.x >> 16));
            m[2] = f16_bits_to_f32((uint16_t)(mh.y & 0xFFFFu));
            m[3] = f16_bits_to_f32((uint16_t)(mh.y >> 16));
            const float nbd[4] = {-kFoldBias * d[0], -kFoldBias * d[1], -kFoldBias * d[2], -kFoldBias * d[3]};
            const int slot4 = (kb - kb0) & 3;
            const bool mine4 = slot4 == g;
#pragma unroll
            for (int c = 0; c < 4; c++) mk[c] = mine4 ? m[c] : mk[c];
#pragma unroll
            for (int t = 0; t < RT; t++) {
                const float gsr = sm.xs[buf][wr * (BM / 2) + t * 16 + jj].y;
                gk[t] = mine4 ? gsr : gk[t];
                // dx of the 4 rows this lane holds results for: rows wr*BM/2 + t*16 + 4g + v
                const float4* xp = reinterpret_cast<const float4*>(&sm.xs[buf][wr * (BM / 2) + t * 16 + g * 4]);
                const float4 x01 = xp[0], x23 = xp[1];
                const float dxv[4] = {x01.x, x01.z, x23.x, x23.z};
#pragma unroll
                for (int v = 0; v < 4; v++)
#pragma unroll
                    for (int c = 0; c < 4; c++)
                        f[t][c][v] = fmaf(fmaf(__int_as_float(acc[t][c][v]), d[c], nbd[c]), dxv[v], f[t][c][v]);
            }
            if (slot4 == 3 || kb + 1 == kb1) {
#pragma unroll
                for (int t = 0; t < RT; t++) {
#pragma unroll
                    for (int c = 0; c < 4; c++) f[t][c] = __builtin_amdgcn_mfma_f32_16x16x4f32(gk[t], mk[c], f[t][c], 0, 0, 0);
                    gk[t] = 0.0f;
                }
#pragma unroll
                for (int c = 0; c < 4; c++) mk[c] = 0.0f;
            }
        }

        if (kb + 1 < kb1) LLMOPS_STASH(buf ^ 1);
        __syncthreads();
    }
#undef LLMOPS_FETCH
#undef LLMOPS_STASH

    if (PARTIALS) return;
    const int strip = strip0 + strip_l;
    if (counters != nullptr) {
        splitk_finish<RT, (RT == 4 ? 12 : (RT == 2 ? 6 : 4))>(f, out, split_stride, ldo, row0, min(BM, rows - row0), wr * (BM / 2), strip,
                                                             Ng, q, g, rows, y_final, Ny, residual, &counters[by * nbx + bx], tid);
        return;
    }
    if (strip >= Ng) return;
    float* o = out + (int64_t)blockIdx.z * split_stride;
    const int64_t n0 = (int64_t)strip * kGroupN + q * 4;
#pragma unroll
    for (int t = 0; t < RT; t++)
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const int row = row0 + wr * (BM / 2) + t * 16 + g * 4 + v;
            if (row >= rows) continue;
            float* dst = o + (int64_t)row * ldo + n0;
            // residual != nullptr only without split-K: then o is the result itself, row stride ldo
            const float* res = residual ? residual + (int64_t)row * ldo + n0 : nullptr;
            if (n0 + 3 < N && (ldo & 3) == 0) {
                float4 val = make_float4(f[t][0][v], f[t][1][v], f[t][2][v], f[t][3][v]);
                if (res) {
                    const float4 r4 = *reinterpret_cast<const float4*>(res);
                    val.x += r4.x, val.y += r4.y, val.z += r4.z, val.w += r4.w;
                }
                *reinterpret_cast<float4*>(dst) = val;
            } else {
#pragma unroll
                for (int c = 0; c < 4; c++)
                    if (n0 + c < N) dst[c] = res ? f[t][c][v] + res[c] : f[t][c][v];
            }
        }
}

// ---- two groups of wavefronts in alternating phases (group 128, many rows) -------------------------
// Per k-group a wavefront has a matrix-core phase (operand reads, 32 int8 MFMAs) and a vector-ALU
// phase (the fp32 fold: convert, scale product, fma per output element).  Two independent wavefronts
// on one SIMD drift into the same phase and then simply take turns on the same pipe, so nothing
// overlaps.  Here a workgroup has 8 wavefronts = two groups of 4, one of each per SIMD, and the phases
// are separated by workgroup barriers with the second group started one phase late: while one group's
// MFMAs run, the other group's fold has the vector ALU, by construction.  The vector ALU is the
// scarcer unit (3 instructions per output element and k-group against 2 MFMAs per 256 elements), so
// everything else is kept off it:
//   tile: 256 rows x 128 columns; group p owns rows 128p..128p+127 (wave = 64 x 64, as in the kernel
//   above); the weights of the tile are staged once and used by both groups.
//   weights: fetched by group 0 (the one ahead in time) into registers one k-group ahead, unpacked
//   ONCE per workgroup to int8 and stored to LDS in MFMA operand order ([strip][k half][column
//   set c][g][q] -> 16 bytes), fp16 scales converted to fp32 on the way; a wave's B operands are
//   then plain 16-byte LDS reads, no unpacking per wave.
//   activations and their scales: asynchronous global->LDS copies (no registers, no LDS store
//   instructions) for the next k-group, issued one at a time between the MFMAs of the matrix-core
//   phase and waited for before the iteration's last barrier; each group copies its own rows.
//   (All copies at the top of the phase measured ~500 cycles before the first MFMA: the four waves'
//   copies queue up in the CU's address unit.)  Tile rows are 128 bytes with the
//   16-byte chunk c of row r at chunk position c ^ key(r), key(r) = (r + ((r >> 3) & 1)) & 7: the 16
//   rows that one ds_read_b128 touches then fall on 16 different 16-byte bank groups of the 256-byte
//   bank line (and any aligned 8 of them on 8 different ones).  The copies land lane by lane, so the
//   spreading is done by choosing what each lane fetches.  The unpacked weights of a strip take
//   4096 + 128 bytes for the same reason (a read touches two strips).
//   Group 1 still folds k-group kb-1 while group 0 overwrites that k-group's weight buffer, which is
//   why the weight scales are taken into registers in the matrix-core phase.
//   The A operands are read by hand-placed ds_read_b128 (four row tiles ahead of the MFMAs that use
//   them) with hand-placed waits: the compiler would issue each read right before its use and leave
//   the matrix cores waiting for LDS eight times per k-group.
//   The fold is register arithmetic and the MFMAs have no side effects, so the compiler is free to
//   move either across a barrier into the other phase (it did: the fold ended up next to the same
//   group's MFMAs).  Empty asm statements that name the accumulators as operands pin them.
//   The min term is not in the loop: the accumulators start at it (min_term_add above), formed from
//   the [row][kg] group sums and the blocks' mins before the first k-group -- by group 0 while group 1
//   unpacks the first k-group's weights, by group 1 in the phase it has to wait anyway.  In the loop
//   it was 16 fp32 MFMAs per four k-groups and wave, each of which holds up the vector ALU of its SIMD
//   for its 32 cycles (2048 rows: 11008 x 4096 187 -> 181 us, 4096 x 11008 164 -> 159 us).
// Measured per k-group with the min term still in the loop (2048 x 11008 x 4096, cycles of the shader clock): matrix-core side ~1500
// (operand reads 450, 32 MFMAs with the copies between them 1000), fold side ~1350-1900 (the fold
// itself 1350: the vector ALU is shared with the other group's MFMA issue; unpacking the weights on
// group 0 adds the wait for their fetch), barriers ~400; 4000 per k-group against ~4700 for the
// four-wave kernel above.
constexpr int kBuStrip = 2 * 4 * 4 * 8 * 16 + 128;
struct GemmPPSmem {
    static constexpr int BM = 256;
    uint8_t a[2][BM * 128];
    uint8_t bu[2][4 * kBuStrip];            // unpacked weights: [strip][h][c][g][q][16], strips padded
    float d[2][4 * 32];                     // weight scale per strip column
    float dx[2][BM];
};

__device__ __forceinline__ uint32_t lds_off(const void* p) {
    return (uint32_t)(uintptr_t)((const __attribute__((address_space(3))) void*)p);
}
// lane i's 16 (4) bytes at base + off (base the same for the whole wave, off a byte offset per lane)
// land at lds_base + 16*i (4*i); counts in vmcnt like any load
__device__ __forceinline__ void copy16_to_lds(const void* base, uint32_t off, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(off), "s"(base), "s"(lds_base) : "memory", "m0");
}
__device__ __forceinline__ void copy4_to_lds(const void* base, uint32_t off, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1" : : "v"(off), "s"(base), "s"(lds_base) : "memory", "m0");
}
// 16-byte LDS read whose result may only be used after lds_ready<N>() on it, N = number of LDS
// operations issued after this one that may still be pending (LDS operations complete in order).
// Between the two calls the variable must not be touched.
// Between the two calls the variable must not be touched -- which the compiler cannot know, so this
// pair is only for code that is known not to spill registers (the build of the kernel below that
// writes int32 tiles does spill, and passes PLAIN = true to get an ordinary load instead).
template <int OFF, bool PLAIN>
__device__ __forceinline__ void lds_read16_issue(v4i& r, uint32_t addr) {
    if (PLAIN) {
        r = *reinterpret_cast<const __attribute__((address_space(3))) v4i*>((uintptr_t)(addr + OFF));
    } else {
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(r) : "v"(addr), "n"(OFF) : "memory");
    }
}
template <int N, bool PLAIN>
__device__ __forceinline__ void lds_ready(v4i& r) {
    if (!PLAIN) asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(r) : "n"(N) : "memory");
}

template <bool PARTIALS>
__global__ __launch_bounds__(512, 2) void fc_gemm_pp_kernel(const uint8_t* __restrict__ weiq, const int8_t* __restrict__ xq,
                                                             const float* __restrict__ xd, const float* __restrict__ gs,
                                                             const float2* __restrict__ xsT, float* __restrict__ out,
                                                             int32_t* __restrict__ out_i, int Ng, int Kg, int64_t ldo,
                                                             int64_t N, int rows, int kb_per_split, int64_t split_stride,
                                                             const float* __restrict__ residual) {
    constexpr int RT = 4, BM = 256, GM = 128;
    extern __shared__ __align__(16) uint8_t smem_raw[];
    GemmPPSmem& sm = *reinterpret_cast<GemmPPSmem*>(smem_raw);

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int grp = wave >> 2, w4 = wave & 3;
    const int wr = w4 >> 1, wc = w4 & 1;
    const int g = lane >> 4, jj = lane & 15, q = jj & 7, sp = jj >> 3;
    // tile numbering: one contiguous run of tiles per XCD, bands of 8 row blocks, rows fastest
    const int nbx = (Ng + 3) / 4, nby = (rows + BM - 1) / BM;
    int bx, by;
    {
        const int total = nbx * nby, per_xcd = (total + 7) / 8;
        const int i = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
        if ((int)(blockIdx.x >> 3) >= per_xcd || i >= total) return;  // uniform for the workgroup
        constexpr int kBand = 8;
        const int band = i / (kBand * nbx), in_band = i % (kBand * nbx);
        const int first = band * kBand, rows_in_band = min(kBand, nby - first);
        by = first + in_band % rows_in_band;
        bx = in_band / rows_in_band;
    }
    const int strip0 = bx * 4;
    const int row0 = by * BM + grp * GM;  // first row of this group
    const int kb0 = blockIdx.z * kb_per_split, kb1 = min(Kg, kb0 + kb_per_split);
    const int64_t Kp = (int64_t)Kg * 128;

    // ---- what this lane copies per k-group ----
    // activations: wave w4 of a group copies its row blocks 4*w4 .. 4*w4+3 (8 rows x 128 bytes each)
    // (all sources are a wave-uniform base pointer, which moves with the k-group, plus a 32-bit byte
    // offset per lane; the host only launches this kernel when the tensors are below 2 GiB)
    uint32_t aoff[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int r = (w4 * 4 + i) * 8 + (lane >> 3);  // row within the group (a multiple of 16 rows per group)
        const int key = (r + ((r >> 3) & 1)) & 7;
        aoff[i] = (uint32_t)(min(rows - 1, row0 + r) * (int)Kp + (((lane & 7) ^ key) * 16));
    }
    // activation scales: waves 0,1 of a group copy dx of rows 64*w4 + lane
    const int xr = (w4 & 1) * 64 + lane;
    const int64_t xrow = min(rows - 1, row0 + xr);
    const uint8_t* xbase = nullptr;
    uint32_t xoff = 0;
    int64_t xstep = 0;  // bytes per k-group
    if (!PARTIALS) {
        if (xsT) {
            xbase = reinterpret_cast<const uint8_t*>(xsT);
            xoff = (uint32_t)(xrow * 8);
            xstep = (int64_t)rows * 8;
        } else {
            xbase = reinterpret_cast<const uint8_t*>(xd);
            xoff = (uint32_t)(xrow * Kg * 4);
            xstep = 4;
        }
    }
    const uint32_t lds_a = lds_off(&sm.a[0][0]);
    const uint32_t lds_x = lds_off(&sm.dx[0][0]);
#define LLMOPS_COPY_A(KB, BUF, I)                                                                                  \
    copy16_to_lds(xq + (int64_t)(KB) * 128, aoff[I], lds_a + (BUF) * (BM * 128) + (grp * GM + (w4 * 4 + (I)) * 8) * 128)
#define LLMOPS_COPY_X(KB, BUF)                                                                                     \
    do {                                                                                                           \
        if (!PARTIALS && w4 < 2) copy4_to_lds(xbase + (int64_t)(KB) * xstep, xoff, lds_x + (BUF) * (BM * 4) + (grp * GM + w4 * 64) * 4); \
    } while (0)
#define LLMOPS_COPY(KB, BUF)                                                                                       \
    do {                                                                                                           \
        _Pragma("unroll") for (int i = 0; i < 4; i++) LLMOPS_COPY_A(KB, BUF, i);                                   \
        LLMOPS_COPY_X(KB, BUF);                                                                                    \
    } while (0)

    // weights (group 0; group 1 for the first k-group, while group 0 has the min term to compute): thread t
    // of the group takes the 16-byte chunks t and t + 256 of the tile's 512 (chunk = strip (2 bits) | k8-row
    // (4 bits) | column quad (3 bits)); its first 16 threads also the 16 chunks of fp16 scales d (strip
    // (2 bits) | column octet (2 bits))
    const int gtid = tid & 255;
    uint32_t boff[2];
    int bdst[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int ch = gtid + i * 256, st = ch >> 7, r = (ch >> 3) & 15, q4 = ch & 7;
        boff[i] = (uint32_t)(min(Ng - 1, strip0 + st) * Kg * kBlk128 + r * 128 + q4 * 16);
        // [strip][h = r>>3][c][g = (r&7)>>1][q4][8 * (r&1)]; c adds 512 bytes
        bdst[i] = st * kBuStrip + ((((r >> 3) * 4) * 4 + ((r & 7) >> 1)) * 8 + q4) * 16 + (r & 1) * 8;
    }
    const int sst = (gtid >> 2) & 3, spart = gtid & 3;
    const uint32_t soff = (uint32_t)(min(Ng - 1, strip0 + sst) * Kg * kBlk128 + 2048 + spart * 16);
    v4u rb[2], rs = {0u, 0u, 0u, 0u};
#define LLMOPS_FETCH_B(KB, WHO)                                                                            \
    do {                                                                                                   \
        if (grp == (WHO)) {                                                                                \
            const uint8_t* wkb = weiq + (int64_t)(KB) * kBlk128;                                           \
            rb[0] = *reinterpret_cast<const v4u*>(wkb + boff[0]);                                          \
            rb[1] = *reinterpret_cast<const v4u*>(wkb + boff[1]);                                          \
            if (gtid < 16) rs = *reinterpret_cast<const v4u*>(wkb + soff);                                 \
        }                                                                                                  \
    } while (0)
#define LLMOPS_STASH_B(BUF, WHO)                                                                           \
    do {                                                                                                   \
        if (grp == (WHO)) {                                                                                \
            _Pragma("unroll") for (int i = 0; i < 2; i++)                                                  \
                _Pragma("unroll") for (int c = 0; c < 4; c++) {                                            \
                    uint2 u;                                                                               \
                    u.x = lo4(rb[i][c]);                                                                   \
                    u.y = hi4(rb[i][c]);                                                                   \
                    *reinterpret_cast<uint2*>(&sm.bu[BUF][bdst[i] + c * 512]) = u;                         \
                }                                                                                          \
            if (gtid < 16) {                                                                               \
                float* dstf = sm.d[BUF] + sst * 32 + spart * 8;                                            \
                float4 lo, hi;                                                                             \
                lo.x = f16_bits_to_f32((uint16_t)(rs[0] & 0xFFFFu));                                       \
                lo.y = f16_bits_to_f32((uint16_t)(rs[0] >> 16));                                           \
                lo.z = f16_bits_to_f32((uint16_t)(rs[1] & 0xFFFFu));                                       \
                lo.w = f16_bits_to_f32((uint16_t)(rs[1] >> 16));                                           \
                hi.x = f16_bits_to_f32((uint16_t)(rs[2] & 0xFFFFu));                                       \
                hi.y = f16_bits_to_f32((uint16_t)(rs[2] >> 16));                                           \
                hi.z = f16_bits_to_f32((uint16_t)(rs[3] & 0xFFFFu));                                       \
                hi.w = f16_bits_to_f32((uint16_t)(rs[3] >> 16));                                           \
                *reinterpret_cast<float4*>(dstf) = lo;                                                     \
                *reinterpret_cast<float4*>(dstf + 4) = hi;                                                 \
            }                                                                                              \
        }                                                                                                  \
    } while (0)

    v4f f[RT][4];
    const int strip_l = wc * 2 + sp;          // strip (0..3) of the tile this lane's B operands come from
    const int lrow = grp * GM + wr * 64;      // first tile row of this wave

    // The accumulators start at the tile's min term (min_term_add).  Its operands are asked for ahead of the first
    // k-group's; group 0 forms it while group 1 unpacks the first k-group's weights, group 1 in the phase it
    // has to wait anyway (it runs one phase behind group 0).  A second and third round of 32 k-groups are
    // fetched while the round before is being added.
    MinTermRound<RT> mt;
    int mroff[RT];
#pragma unroll
    for (int t = 0; t < RT; t++) mroff[t] = min(rows - 1, row0 + wr * 64 + t * 16 + jj) * Kg;
    const int mstrip = min(Ng - 1, strip0 + strip_l);
    if (kb0 < kb1) {
        LLMOPS_COPY(kb0, 0);
        LLMOPS_FETCH_B(kb0, 1);
    }
    __builtin_amdgcn_sched_barrier(0);  // the first k-group's operands are asked for first
    if (!PARTIALS && kb0 < kb1) min_term_fetch<RT>(mt, gs, mroff, weiq, Kg, min(kb0 + 8 * g, Kg - 8), mstrip, q);
#define LLMOPS_MIN_TERM()                                                                                  \
    do {                                                                                                   \
        if (!PARTIALS && kb0 < kb1) {                                                                      \
            min_term_add<RT, true>(f, mt, min(kb0 + 8 * g, Kg - 8), kb0 + 8 * g, kb1);                     \
            for (int k32 = kb0 + 32; k32 < kb1; k32 += 32) {                                               \
                min_term_fetch<RT>(mt, gs, mroff, weiq, Kg, min(k32 + 8 * g, Kg - 8), mstrip, q);          \
                min_term_add<RT, false>(f, mt, min(k32 + 8 * g, Kg - 8), k32 + 8 * g, kb1);                \
            }                                                                                              \
        } else {                                                                                           \
            _Pragma("unroll") for (int t = 0; t < RT; t++)                                                 \
                _Pragma("unroll") for (int c = 0; c < 4; c++) f[t][c] = v4f{0.f, 0.f, 0.f, 0.f};           \
        }                                                                                                  \
    } while (0)
    // (s_waitcnt through the builtin, so that the compiler knows that no load of this prologue is pending in
    // the k-group loop: left to its own bookkeeping it assumes that a further round may have been asked for and
    // waits for "it" -- in fact for the k-group's asynchronous copies -- where the loop reuses the registers)
    constexpr int kVmcnt0 = 0x0F70;  // vmcnt(0), the other counters left alone
    if (grp == 1) {
        if (kb0 < kb1) LLMOPS_STASH_B(0, 1);
        __builtin_amdgcn_s_waitcnt(kVmcnt0);
        __syncthreads();  // group 0 arrives here with its min term done ...
    }
    LLMOPS_MIN_TERM();
    __builtin_amdgcn_s_waitcnt(kVmcnt0);
    __syncthreads();  // ... by this one; for group 1 it is the barrier that puts it one phase behind group 0
#undef LLMOPS_MIN_TERM
    // A operand of row tile t, k half h: row lrow + 16t + jj, chunk 4h + g, swizzled by the row's low bits
    const int akey = (jj + (jj >> 3)) & 7;
    const uint32_t a_rd0 = lds_a + (lrow + jj) * 128 + (((0 + g) ^ akey) * 16);
    const uint32_t a_rd1 = lds_a + (lrow + jj) * 128 + (((4 + g) ^ akey) * 16);
    const int b_rd = strip_l * kBuStrip + (g * 8 + q) * 16;  // + (4h + c) * 512
    for (int kb = kb0; kb < kb1; kb++) {
        const int buf = (kb - kb0) & 1;
        const bool more = kb + 1 < kb1;

        // ---- matrix-core phase ----
        // (the copies for the next k-group are issued between the MFMAs, one per four: four waves
        // issuing all of theirs at once right after the barrier keep the address unit busy for
        // several hundred cycles, during which none of them would reach its first MFMA)
        const uint32_t ar0 = a_rd0 + buf * (BM * 128), ar1 = a_rd1 + buf * (BM * 128);
        v4i a00, a01, a02, a03, a10, a11, a12, a13;
        lds_read16_issue<0 * 2048, PARTIALS>(a00, ar0);
        lds_read16_issue<1 * 2048, PARTIALS>(a01, ar0);
        lds_read16_issue<2 * 2048, PARTIALS>(a02, ar0);
        lds_read16_issue<3 * 2048, PARTIALS>(a03, ar0);
        v4i b[2][4];
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int c = 0; c < 4; c++) b[h][c] = *reinterpret_cast<const v4i*>(&sm.bu[buf][b_rd + (h * 4 + c) * 512]);
        const float4 d4 = *reinterpret_cast<const float4*>(&sm.d[buf][strip_l * 32 + q * 4]);
        v4i acc[RT][4];
        // The int32 sums start at the bit pattern of 1.5 * 2^23: read as a float, bits + sum IS the number
        // 1.5 * 2^23 + sum (|sum| <= 128 * 15 * 127 < 2^22), so the fold needs no convert instruction.
        const v4i zero4 = PARTIALS ? v4i{0, 0, 0, 0} : v4i{kFoldBiasBits, kFoldBiasBits, kFoldBiasBits, kFoldBiasBits};
#define LLMOPS_MMA4(T, H, A)                                                                              \
    _Pragma("unroll") for (int c = 0; c < 4; c++)                                                         \
        acc[T][c] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A, b[H][c], (H) == 0 ? zero4 : acc[T][c], 0, 0, 0)
        lds_ready<3, PARTIALS>(a00);
        LLMOPS_MMA4(0, 0, a00);
        lds_read16_issue<0 * 2048, PARTIALS>(a10, ar1);
        if (more) LLMOPS_COPY_A(kb + 1, buf ^ 1, 0);
        lds_ready<3, PARTIALS>(a01);
        LLMOPS_MMA4(1, 0, a01);
        lds_read16_issue<1 * 2048, PARTIALS>(a11, ar1);
        if (more) LLMOPS_COPY_A(kb + 1, buf ^ 1, 1);
        lds_ready<3, PARTIALS>(a02);
        LLMOPS_MMA4(2, 0, a02);
        lds_read16_issue<2 * 2048, PARTIALS>(a12, ar1);
        if (more) LLMOPS_COPY_A(kb + 1, buf ^ 1, 2);
        lds_ready<3, PARTIALS>(a03);
        LLMOPS_MMA4(3, 0, a03);
        lds_read16_issue<3 * 2048, PARTIALS>(a13, ar1);
        if (more) LLMOPS_COPY_A(kb + 1, buf ^ 1, 3);
        lds_ready<3, PARTIALS>(a10);
        LLMOPS_MMA4(0, 1, a10);
        if (more) LLMOPS_COPY_X(kb + 1, buf ^ 1);
        lds_ready<2, PARTIALS>(a11);
        LLMOPS_MMA4(1, 1, a11);
        if (more) LLMOPS_FETCH_B(kb + 1, 0);
        lds_ready<1, PARTIALS>(a12);
        LLMOPS_MMA4(2, 1, a12);
        lds_ready<0, PARTIALS>(a13);
        LLMOPS_MMA4(3, 1, a13);
#undef LLMOPS_MMA4
        const float d[4] = {d4.x, d4.y, d4.z, d4.w};
        const float nbd[4] = {-kFoldBias * d4.x, -kFoldBias * d4.y, -kFoldBias * d4.z, -kFoldBias * d4.w};
        asm volatile("" : "+v"(acc[0][0]), "+v"(acc[0][1]), "+v"(acc[0][2]), "+v"(acc[0][3]), "+v"(acc[1][0]),
                          "+v"(acc[1][1]), "+v"(acc[1][2]), "+v"(acc[1][3]), "+v"(acc[2][0]), "+v"(acc[2][1]),
                          "+v"(acc[2][2]), "+v"(acc[2][3]), "+v"(acc[3][0]), "+v"(acc[3][1]), "+v"(acc[3][2]),
                          "+v"(acc[3][3]));  // likewise: the MFMAs stay in the matrix-core phase
        __syncthreads();

        // ---- vector phase: fold the int32 tiles into the fp32 accumulators ----
        if (PARTIALS) {
            const int strip = strip0 + strip_l;
            if (strip < Ng) {
#pragma unroll
                for (int t = 0; t < RT; t++)
#pragma unroll
                    for (int v = 0; v < 4; v++) {
                        const int row = row0 + wr * 64 + t * 16 + g * 4 + v;
                        if (row < rows) {
#pragma unroll
                            for (int c = 0; c < 4; c++)
                                out_i[((int64_t)row * ((int64_t)Ng * kGroupN) + strip * kGroupN + q * 4 + c) * Kg + kb] =
                                    acc[t][c][v];
                        }
                    }
            }
        } else {
#pragma unroll
            for (int t = 0; t < RT; t++) {
                // dx of the 4 rows this lane holds results for: rows lrow + t*16 + 4g + v
                const float4 x4 = *reinterpret_cast<const float4*>(&sm.dx[buf][lrow + t * 16 + g * 4]);
                const float dxv[4] = {x4.x, x4.y, x4.z, x4.w};
                // sum * d in one fma: (bias + sum) * d - bias * d, exact before its single rounding because
                // bias * d (2 significant bits times the 11 of an fp16) is a float; then one fma with dx
#pragma unroll
                for (int v = 0; v < 4; v++)
#pragma unroll
                    for (int c = 0; c < 4; c++)
                        f[t][c][v] = fmaf(fmaf(__int_as_float(acc[t][c][v]), d[c], nbd[c]), dxv[v], f[t][c][v]);
            }
        }
        // the fold is register arithmetic, which the compiler may move across the barrier into the other
        // phase; naming the accumulators as operands of an (empty) asm statement keeps it on this side
        asm volatile("" : "+v"(f[0][0]), "+v"(f[0][1]), "+v"(f[0][2]), "+v"(f[0][3]), "+v"(f[1][0]), "+v"(f[1][1]),
                          "+v"(f[1][2]), "+v"(f[1][3]), "+v"(f[2][0]), "+v"(f[2][1]), "+v"(f[2][2]), "+v"(f[2][3]),
                          "+v"(f[3][0]), "+v"(f[3][1]), "+v"(f[3][2]), "+v"(f[3][3]));
        if (kb + 1 < kb1) LLMOPS_STASH_B(buf ^ 1, 0);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's copies for the next k-group have landed
        __syncthreads();
    }
    if (grp == 0) __syncthreads();  // pairs with group 1's last barrier
#undef LLMOPS_COPY
#undef LLMOPS_COPY_A
#undef LLMOPS_COPY_X
#undef LLMOPS_FETCH_B
#undef LLMOPS_STASH_B

    if (PARTIALS) return;
    const int strip = strip0 + strip_l;
    if (strip >= Ng) return;
    float* o = out + (int64_t)blockIdx.z * split_stride;
    const int64_t n0 = (int64_t)strip * kGroupN + q * 4;
#pragma unroll
    for (int t = 0; t < RT; t++)
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const int row = row0 + wr * 64 + t * 16 + g * 4 + v;
            if (row >= rows) continue;
            float* dst = o + (int64_t)row * ldo + n0;
            // residual != nullptr only without split-K: then o is the result itself, row stride ldo
            const float* res = residual ? residual + (int64_t)row * ldo + n0 : nullptr;
            if (n0 + 3 < N && (ldo & 3) == 0) {
                float4 val = make_float4(f[t][0][v], f[t][1][v], f[t][2][v], f[t][3][v]);
                if (res) {
                    const float4 r4 = *reinterpret_cast<const float4*>(res);
                    val.x += r4.x, val.y += r4.y, val.z += r4.z, val.w += r4.w;
                }
                *reinterpret_cast<float4*>(dst) = val;
            } else {
#pragma unroll
                for (int c = 0; c < 4; c++)
                    if (n0 + c < N) dst[c] = res ? f[t][c][v] + res[c] : f[t][c][v];
            }
        }
}

// y[row][n] = sum over splits (index order) of part[s][row][n] (+ residual[row][n]); four columns per
// thread (the partial sums' row stride ldp is a multiple of 32 floats, so their 16-byte loads are aligned)
__global__ void gemm_reduce_kernel(const float* __restrict__ part, float* __restrict__ y, int64_t rows, int64_t N,
                                   int64_t ldp, int64_t split_stride, int S, const float* __restrict__ residual) {
    const int64_t nq = (N + 3) / 4;
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= rows * nq) return;
    const int64_t r = i / nq, n = (i % nq) * 4;
    float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
    float* dst = y + r * N + n;
    const float* res = residual ? residual + r * N + n : nullptr;
    const bool whole = n + 3 < N && (N & 3) == 0;
    float4 r4 = make_float4(0.f, 0.f, 0.f, 0.f);
    if (whole && res) r4 = *reinterpret_cast<const float4*>(res);
    // four splits' loads in flight at a time (a split past the last re-reads the last and is not added)
    for (int s0 = 0; s0 < S; s0 += 4) {
        float4 v[4];
#pragma unroll
        for (int u = 0; u < 4; u++)
            v[u] = *reinterpret_cast<const float4*>(part + (int64_t)min(s0 + u, S - 1) * split_stride + r * ldp + n);
#pragma unroll
        for (int u = 0; u < 4; u++)
            if (s0 + u < S) a.x += v[u].x, a.y += v[u].y, a.z += v[u].z, a.w += v[u].w;
    }
    if (whole) {
        if (res) a.x += r4.x, a.y += r4.y, a.z += r4.z, a.w += r4.w;
        *reinterpret_cast<float4*>(dst) = a;
    } else {
        const float av[4] = {a.x, a.y, a.z, a.w};
        for (int c = 0; c < 4; c++)
            if (n + c < N) dst[c] = res ? av[c] + res[c] : av[c];
    }
}

// Integer core only, through the same mma_group: acc[row][n][kb]
template <int G>
__global__ __launch_bounds__(256) void fc_gemm_partials_kernel(const uint8_t* __restrict__ weiq,
                                                                const int8_t* __restrict__ xq, int32_t* __restrict__ out,
                                                                int Ng, int Kg, int rows) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane >> 4, jj = lane & 15, q = jj & 7, sp = jj >> 3;
    const int pair = blockIdx.x * 4 + wave;
    if (pair * 2 >= Ng) return;
    const int strip = pair * 2 + sp;
    const bool strip_ok = strip < Ng;
    const int strip_c = strip_ok ? strip : Ng - 1;
    const int row0 = blockIdx.y * 16;
    const int kb = blockIdx.z;
    const int64_t Kp = (int64_t)Kg * G;
    const int64_t Np = (int64_t)Ng * kGroupN;
    const uint8_t* blk = weiq + ((int64_t)strip_c * Kg + kb) * block_bytes(G);
    const int8_t* xrow[1] = {xq + (int64_t)min(rows - 1, row0 + jj) * Kp};
    v4i acc[1][4];
#pragma unroll
    for (int c = 0; c < 4; c++) acc[0][c] = v4i{0, 0, 0, 0};
    mma_group<G, 1>(blk, xrow, (int64_t)kb * G, g, q, acc);
    if (!strip_ok) return;
#pragma unroll
    for (int v = 0; v < 4; v++) {
        const int row = row0 + g * 4 + v;
        if (row >= rows) continue;
#pragma unroll
        for (int c = 0; c < 4; c++) out[((int64_t)row * Np + strip * kGroupN + q * 4 + c) * Kg + kb] = acc[0][c][v];
    }
}

struct GemmPlan {
    int RT, S, kb_per_split;
    bool lds;
};

static int g_gemm_pp_min_rows = 256;
static int g_gemm_rt = 0;  // 0 = choose per shape; -1 = also keep 9..32 rows on the tiled kernel
static int g_gemm_fused_reduce = 1;  // split-K partial sums added by the product kernel itself (0: by a second launch)
static int g_gemm_force_split = 0;   // > 0: the split-K factor to use whatever the estimate says (tests)
bool gemm_rows_kernel_enabled() { return g_gemm_rt >= 0; }

// Split-K factor for `tiles` output tiles on a machine with `slots` resident workgroups.
static void gemm_split(int64_t tiles, int64_t slots, int64_t Kg, GemmPlan& p) {
    int S = (int)((slots + tiles - 1) / tiles);
    if (S > Kg) S = (int)Kg;
    if (S < 1) S = 1;
    p.kb_per_split = (int)((Kg + S - 1) / S);
    p.S = (int)((Kg + p.kb_per_split - 1) / p.kb_per_split);
}

static GemmPlan plan_gemm(int64_t rows, int64_t Ng, int64_t Kg, int G) {
    GemmPlan p;
    p.lds = (G == 128);
    if (!p.lds) {
        p.RT = rows > 32 ? 4 : (rows > 16 ? 2 : 1);  // RT*16 rows per wave
        gemm_split((((Ng + 1) / 2 + 3) / 4) * ((rows + p.RT * 16 - 1) / (p.RT * 16)), 512, Kg, p);
        return p;
    }
    // Candidates: the 256-row kernel with two wave groups (one workgroup per CU) and the four-wave
    // kernel with 128, 64 or 32 rows per workgroup (two, three, four workgroups per CU: bigger tiles
    // reuse the unpacked weights over more rows but need more registers).  Measured rate per row at
    // full occupancy (M = 2048): 1.17 : 1.0 : 0.98 : 0.77.  What decides between them at smaller M is
    // how evenly the tiles fill the machine, so the plan takes the candidate and split-K factor with
    // the least estimated time: rounds of resident workgroups x (rows per CU per round / efficiency)
    // x share of K per split.  Split factors tried: the largest that still runs in one round and the
    // smallest that fills the machine (a second round of half-length workgroups costs what one round
    // of full-length ones does, plus the reduction of the partial sums).
    // (the 256-row kernel's lanes address the tensors with 32-bit byte offsets)
    const bool small = rows * Kg * 128 < ((int64_t)1 << 31) && Ng * Kg * 2176 < ((int64_t)1 << 31);
    static const int kRT[4] = {8, 4, 2, 1};
    static const int kRows[4] = {256, 128, 64, 32};
    static const int kWgPerCu[4] = {1, 2, 3, 4};
    static const double kEff[4] = {1.17, 1.0, 0.98, 0.77};
    double best = 0.0;
    for (int i = 0; i < 4; i++) {
        if (g_gemm_rt > 0 && kRT[i] != g_gemm_rt) continue;
        if (kRT[i] == 8 && (!small || Kg < 8 || (g_gemm_rt != 8 && rows < g_gemm_pp_min_rows))) continue;
        const int64_t bm = kRows[i], slots = 256 * kWgPerCu[i];
        const int64_t tiles = ((Ng + 3) / 4) * ((rows + bm - 1) / bm);
        const int64_t s_floor = slots / tiles, s_ceil = (slots + tiles - 1) / tiles;
        // (a third candidate where the machine would take more: the most splits the product kernel still adds itself)
        const int64_t s_cap = 12 * (int64_t)g_gemm_fused_reduce;
        // Below the 256-row kernel's range a workgroup's run of k-groups is short and what a workgroup costs before
        // and after it decides: every split factor the kernel can finish itself is tried, a workgroup counts as
        // its run plus 3 k-groups, and a split as 2.0 * bm / Kg (measured: sweeps of every tiling x 1..12 splits at
        // 24..256 rows on 4096^2, 11008|12288|22016 x 4096 and 4096 x 11008; the choices made this way are 1.4 %
        // slower on average than the best measured one, against 5 % -- up to 27 % at 24..64 rows -- before).
        const bool few_rows = rows < g_gemm_pp_min_rows && g_gemm_fused_reduce && kRT[i] != 8;
        const int n_try = few_rows ? 12 : 3;
        for (int it = 0; it < n_try; it++) {
            const int64_t s_try = few_rows ? it + 1
                                           : (it == 0 ? s_floor : (it == 1 ? s_ceil : ((s_cap > 0 && s_cap < s_floor && kRT[i] != 8) ? s_cap : s_floor)));
            GemmPlan q = p;
            q.RT = kRT[i];
            int64_t S = s_try < 1 ? 1 : (s_try > Kg ? Kg : s_try);
            if (g_gemm_force_split > 0) S = g_gemm_force_split > Kg ? Kg : g_gemm_force_split;
            q.kb_per_split = (int)((Kg + S - 1) / S);
            q.S = (int)((Kg + q.kb_per_split - 1) / q.kb_per_split);
            const int64_t rounds = (tiles * q.S + slots - 1) / slots;
            double cost = (double)rounds * (double)(bm * kWgPerCu[i]) / kEff[i] * (double)(q.kb_per_split + (few_rows ? 3 : 0)) / (double)Kg;
            // Split-K is not free.  In the unit of this estimate (rows x share of K; about 0.014 us x Kg) the last
            // split of a tile to arrive adds S tiles of bm rows at ~150 GB/s (0.24 * S * bm / Kg); a second launch
            // over the partial sums costs 8-11 us whatever the shape (800 / Kg: the price at which the measured
            // choices came out best; 4096x11008 at 40-64 rows 24-25.5 -> 21-21.8 us against 570 / Kg).
            if (q.S > 1) {
                const bool in_kernel = g_gemm_fused_reduce && q.S <= 12 * g_gemm_fused_reduce && kRT[i] != 8;
                cost += in_kernel ? (few_rows ? 2.0 : 0.24) * (double)q.S * (double)bm / (double)Kg : 800.0 / (double)Kg;
            }
            if (best == 0.0 || cost < best) {
                best = cost;
                p = q;
            }
        }
    }
    if (best == 0.0) {  // a forced candidate that cannot run here: fall back to the 128-row kernel
        p.RT = 4;
        gemm_split(((Ng + 3) / 4) * ((rows + 127) / 128), 512, Kg, p);
    }
    return p;
}

size_t gemm_workspace_bytes(int64_t rows, int64_t Ng, int64_t Kg, int G) {
    const GemmPlan p = plan_gemm(rows, Ng, Kg, G);
    return p.S > 1 ? (size_t)p.S * rows * Ng * kGroupN * sizeof(float) : 0;
}

template <int G, int RT>
static void launch_gemm_t(const uint8_t* w, const int8_t* xq, const float* xd, const float* gs, float* out, int64_t Ng,
                          int64_t Kg, int64_t ldo, int64_t N, int64_t rows, const GemmPlan& p, int64_t split_stride,
                          hipStream_t st) {
    dim3 grid((unsigned)(((Ng + 1) / 2 + 3) / 4), (unsigned)((rows + RT * 16 - 1) / (RT * 16)), (unsigned)p.S);
    fc_gemm_kernel<G, RT><<<grid, 256, 0, st>>>(w, xq, xd, gs, out, (int)Ng, (int)Kg, ldo, N, (int)rows, p.kb_per_split,
                                                split_stride);
}

template <int RT>
static int launch_gemm_lds_t(const uint8_t* w, const int8_t* xq, const float* xd, const float* gs, const float2* xsT,
                             float* out, int64_t Ng, int64_t Kg, int64_t ldo, int64_t N, int64_t rows, const GemmPlan& p,
                             int64_t split_stride, const float* residual, float* y_final, int64_t Ny, unsigned* counters,
                             hipStream_t st) {
    static bool configured = false;  // opt in to more than 64 KiB of dynamic LDS once per kernel
    if (!configured) {
        LLMOPS_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&fc_gemm_lds_kernel<RT, false>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)sizeof(GemmSmem<RT>)));
        configured = true;
    }
    // (the kernel's staging loads take 32-bit offsets into the scale pairs [Kg][rows] and into a tile's rows)
    if (rows * Kg * 8 >= ((int64_t)1 << 32) || Kg * 128 * 128 >= ((int64_t)1 << 32))
        return fail(LLMOPS_EINVAL, "fc_Q4A: rows * Kg must be below 2^29 for the tiled kernel");
    const int64_t tiles = ((Ng + 3) / 4) * ((rows + RT * 32 - 1) / (RT * 32));
    dim3 grid((unsigned)(8 * ((tiles + 7) / 8)), 1, (unsigned)p.S);  // one run of tiles per XCD
    fc_gemm_lds_kernel<RT, false><<<grid, 256, sizeof(GemmSmem<RT>), st>>>(w, xq, xd, gs, xsT, out, nullptr, (int)Ng, (int)Kg,
                                                                          ldo, N, (int)rows, p.kb_per_split, split_stride,
                                                                          residual, y_final, Ny, counters);
    return LLMOPS_OK;
}

static int launch_gemm_pp(const uint8_t* w, const int8_t* xq, const float* xd, const float* gs, const float2* xsT, float* out,
                          int64_t Ng, int64_t Kg, int64_t ldo, int64_t N, int64_t rows, const GemmPlan& p,
                          int64_t split_stride, const float* residual, hipStream_t st) {
    static bool configured = false;
    if (!configured) {
        LLMOPS_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&fc_gemm_pp_kernel<false>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)sizeof(GemmPPSmem)));
        configured = true;
    }
    const int64_t tiles = ((Ng + 3) / 4) * ((rows + 255) / 256);
    dim3 grid((unsigned)(8 * ((tiles + 7) / 8)), 1, (unsigned)p.S);
    fc_gemm_pp_kernel<false><<<grid, 512, sizeof(GemmPPSmem), st>>>(w, xq, xd, gs, xsT, out, nullptr, (int)Ng, (int)Kg, ldo, N,
                                                                   (int)rows, p.kb_per_split, split_stride, residual);
    return LLMOPS_OK;
}

int launch_add(float* a, const float* b, int64_t total, hipStream_t st);  // misc.hip

// y = product (+ residual, fp32 [rows, N], may be y itself)
int launch_gemm(const uint8_t* w, const int8_t* xq, const float* xd, const float* gs, const float2* xsT, float* y,
                float* part, unsigned* counters, int64_t rows, int64_t Ng, int64_t Kg, int G, int64_t N, const float* residual,
                hipStream_t st) {
    const GemmPlan p = plan_gemm(rows, Ng, Kg, G);
    // With up to 12 splits the four-wave kernel adds the partial sums itself (the last split of a tile to arrive
    // does), given one zeroed arrival counter per tile; otherwise a second launch adds them.  Measured (us, second
    // launch / in kernel): 11008x4096 at 128 rows 29.3 / 25.7, at 256 rows 43.9 / 38.8; 4096x11008 at 384 rows
    // 61.0 / 53.9, at 96 rows (11 splits) 28.6 / 24.6 - but at 128 rows (16 splits of a 128-row tile) 31.9 / 38.8:
    // the one workgroup that adds 16 tiles takes longer than a launch that spreads them over the chip.  The
    // 256-row kernel keeps the second launch: with one workgroup per CU nothing covers the last arrival's tail
    // (4096x11008, 256 rows: 42.2 / 49.1; 512 rows: 66.1 / 70.4).
    const int64_t lds_tiles = ((Ng + 3) / 4) * ((rows + p.RT * 32 - 1) / (p.RT * 32));
    const bool fused_reduce = g_gemm_fused_reduce && p.S > 1 && p.lds && p.RT != 8 && counters != nullptr &&
                              p.S <= 12 * g_gemm_fused_reduce && lds_tiles <= kTicketBytes / 4 && (int64_t)p.RT * 32 * Ng * kGroupN * 4 < ((int64_t)1 << 31);
    // the residual is added where the result is written: in the kernel's stores without split-K, in
    // the reduction of the partial sums with it
    const float* kres = (p.S > 1 && !fused_reduce) ? nullptr : residual;
    unsigned* kcnt = fused_reduce ? counters : nullptr;
    const int64_t Np = Ng * kGroupN;
    float* out = p.S > 1 ? part : y;
    const int64_t ldo = p.S > 1 ? Np : N;
    const int64_t Nw = p.S > 1 ? Np : N;
    const int64_t ss = rows * Np;
    if (p.lds) {
        int rc;
        if (p.RT == 8) rc = launch_gemm_pp(w, xq, xd, gs, xsT, out, Ng, Kg, ldo, Nw, rows, p, ss, kres, st);
        else if (p.RT == 4) rc = launch_gemm_lds_t<4>(w, xq, xd, gs, xsT, out, Ng, Kg, ldo, Nw, rows, p, ss, kres, y, N, kcnt, st);
        else if (p.RT == 2) rc = launch_gemm_lds_t<2>(w, xq, xd, gs, xsT, out, Ng, Kg, ldo, Nw, rows, p, ss, kres, y, N, kcnt, st);
        else rc = launch_gemm_lds_t<1>(w, xq, xd, gs, xsT, out, Ng, Kg, ldo, Nw, rows, p, ss, kres, y, N, kcnt, st);
        if (rc) return rc;
    } else {
        if (p.RT == 4) launch_gemm_t<32, 4>(w, xq, xd, gs, out, Ng, Kg, ldo, Nw, rows, p, ss, st);
        else if (p.RT == 2) launch_gemm_t<32, 2>(w, xq, xd, gs, out, Ng, Kg, ldo, Nw, rows, p, ss, st);
        else launch_gemm_t<32, 1>(w, xq, xd, gs, out, Ng, Kg, ldo, Nw, rows, p, ss, st);
    }
    LLMOPS_LAUNCH_CHECK();
    if (p.S > 1 && !fused_reduce) {
        const int64_t total = rows * ((N + 3) / 4);
        gemm_reduce_kernel<<<(unsigned)((total + 255) / 256), 256, 0, st>>>(part, y, rows, N, Np, ss, p.S, residual);
        LLMOPS_LAUNCH_CHECK();
    } else if (residual != nullptr && !p.lds) {
        return launch_add(y, residual, rows * N, st);  // the group-32 kernel has no residual in its stores
    }
    return LLMOPS_OK;
}

int launch_gemm_partials(const uint8_t* w, const int8_t* xq, int32_t* acc, int64_t rows, int64_t Ng, int64_t Kg, int G,
                         bool two_groups, hipStream_t st) {
    if (G == 128 && two_groups) {
        if (!(rows * Kg * 128 < ((int64_t)1 << 31) && Ng * Kg * 2176 < ((int64_t)1 << 31)))
            return fail(LLMOPS_EINVAL, "the 256-row kernel addresses its operands with 32-bit offsets");
        static bool configured = false;
        if (!configured) {
            LLMOPS_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&fc_gemm_pp_kernel<true>),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)sizeof(GemmPPSmem)));
            configured = true;
        }
        const int64_t tiles = ((Ng + 3) / 4) * ((rows + 255) / 256);
        dim3 grid((unsigned)(8 * ((tiles + 7) / 8)), 1, 1);
        fc_gemm_pp_kernel<true><<<grid, 512, sizeof(GemmPPSmem), st>>>(w, xq, nullptr, nullptr, nullptr, nullptr, acc, (int)Ng,
                                                                      (int)Kg, 0, 0, (int)rows, (int)Kg, 0, nullptr);
    } else if (G == 128) {  // the production LDS-tiled loop, writing its int32 tiles instead of folding them
        static bool configured = false;
        if (!configured) {
            LLMOPS_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&fc_gemm_lds_kernel<2, true>),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)sizeof(GemmSmem<2>)));
            configured = true;
        }
        const int64_t tiles = ((Ng + 3) / 4) * ((rows + 63) / 64);
        dim3 grid((unsigned)(8 * ((tiles + 7) / 8)), 1, 1);
        fc_gemm_lds_kernel<2, true><<<grid, 256, sizeof(GemmSmem<2>), st>>>(w, xq, nullptr, nullptr, nullptr, nullptr, acc,
                                                                          (int)Ng, (int)Kg, 0, 0, (int)rows, (int)Kg, 0, nullptr, nullptr, 0, nullptr);
    } else {
        dim3 grid((unsigned)(((Ng + 1) / 2 + 3) / 4), (unsigned)((rows + 15) / 16), (unsigned)Kg);
        fc_gemm_partials_kernel<32><<<grid, 256, 0, st>>>(w, xq, acc, (int)Ng, (int)Kg, (int)rows);
    }
    LLMOPS_LAUNCH_CHECK();
    return LLMOPS_OK;
}

}  // namespace llmops

extern "C" void llmops_test_gemm_set_tuning(int rows_per_wave_tile) {
    if (llmops::test_hooks_enabled(__func__)) llmops::g_gemm_rt = rows_per_wave_tile;
}
extern "C" void llmops_test_gemm_set_split(int splits) {
    if (llmops::test_hooks_enabled(__func__)) llmops::g_gemm_force_split = splits < 0 ? 0 : splits;
}
extern "C" int llmops_test_gemm_plan(int64_t rows, int64_t Ng, int64_t Kg, int group_k, int* row_tile_factor, int* splits) {
    LLMOPS_TEST_HOOK();
    if (rows < 1 || Ng < 1 || Kg < 1 || (group_k != 32 && group_k != 128) || !row_tile_factor || !splits) return LLMOPS_EINVAL;
    const llmops::GemmPlan p = llmops::plan_gemm(rows, Ng, Kg, group_k);
    *row_tile_factor = p.RT;
    *splits = p.S;
    return LLMOPS_OK;
}
extern "C" void llmops_test_gemm_set_reduce(int in_kernel) {
    if (llmops::test_hooks_enabled(__func__)) llmops::g_gemm_fused_reduce = in_kernel < 0 ? 0 : in_kernel;
}
