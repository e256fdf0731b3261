/* TEST INFRASTRUCTURE ONLY -- not part of the shipped library.
 *
 * Plain-C restatement (scalar loops, OpenMP over the same units the reference parallelises over)
 * of the reference's Q4_1 fully-connected path and of the KV-cache attention op that wraps it.
 * Only tests, the smoke check and the CPU-baseline leg of the benchmark may load this file's
 * shared object; the product path never does.
 *
 * Every function cites the reference lines it follows (paths relative to /root/reference).
 * Unlike the reference, the k-group size G (32 or 128) is a run-time argument here; the
 * reference fixes it at compile time (ops/op_fc.hpp:109).
 *
 * Pinning status (what each function is checked against in tests/):
 *   fp16 conversion         numpy float16 (IEEE RNE) on all 65536 halves + random floats
 *   orc_quant_w / dequant   reference build (oracle/_ref) byte-for-byte, committed golden
 *                           vectors produced by it, closed-form exactly-representable data,
 *                           half-away tie and constant-group cases
 *   orc_quant_x             reference build bit-for-bit, golden vectors, RNE tie cases
 *   orc_fc_partials         int64 brute-force einsum over unpacked nibbles (pure integers)
 *   orc_fc                  reference build bit-for-bit (same fma order), closed-form x@W.T
 *   orc_mm_qk               fp64 einsum (the check the reference's own perf script makes,
 *                           ops/perf_ops.py:168-175), strided and padded-plane cases
 *   orc_rope / orc_attention / orc_softmax / orc_rmsnorm / orc_silu / orc_embedding_q8c
 *                           reference build within 1e-5 (float op order differs), fp64 textbook
 *                           formulas, literal softmax vectors of ops/test_ops.py:171-172
 *
 * Compile with -ffp-contract=off: fused multiply-adds appear only where fmaf() is written.
 */
#include <float.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <omp.h>

#define GROUP_N 32

static inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

/* ---- fp16 <-> fp32, IEEE round-to-nearest-even (ops/utils.hpp:81-90: vcvtps2ph / vcvtph2ps
 *      under the default MXCSR rounding mode) ------------------------------------------------ */
uint16_t orc_fp32_to_fp16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t mag = x & 0x7fffffffu;
    if (mag >= 0x7f800000u) /* inf / nan (quiet the nan, keep top payload bits) */
        return (uint16_t)(sign | 0x7c00u | (mag > 0x7f800000u ? (0x0200u | ((mag >> 13) & 0x3ffu)) : 0));
    if (mag >= 0x477ff000u) /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7c00u);
    if (mag < 0x33000001u) /* <= 2^-25 rounds to zero (2^-25 itself ties to even = 0) */
        return (uint16_t)sign;
    int32_t e = (int32_t)(mag >> 23) - 127;
    uint32_t man = (mag & 0x7fffffu) | 0x800000u; /* 24-bit significand */
    int shift;                                    /* bits dropped from the 24-bit significand */
    uint32_t base;
    if (e >= -14) { /* normal half */
        shift = 13;
        base = (uint32_t)(e + 15) << 10;
        man &= 0x7fffffu; /* implicit bit goes into the exponent field */
    } else {            /* subnormal half: value = man * 2^(e-23), unit = 2^-24 */
        shift = 13 + (-14 - e);
        base = 0;
    }
    uint32_t q = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (q & 1u)))
        q++; /* carry may ripple into the exponent field, which is the right result */
    return (uint16_t)(sign | (base + q));
}

float orc_fp16_to_fp32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t x;
    if (e == 0) {
        if (man == 0) {
            x = sign;
        } else { /* subnormal: normalise */
            int s = 0;
            while (!(man & 0x400u)) {
                man <<= 1;
                s++;
            }
            man &= 0x3ffu;
            x = sign | ((uint32_t)(127 - 15 - s + 1) << 23) | (man << 13);
        }
    } else if (e == 31) {
        x = sign | 0x7f800000u | (man << 13) | (man ? 0x400000u : 0u); /* vcvtph2ps quiets sNaN */
    } else {
        x = sign | ((e + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &x, 4);
    return f;
}

/* ---- block geometry (ops/op_fc.hpp:14-24): G/8 rows of 128 nibble bytes, then 32 fp16 d,
 *      then 32 fp16 m ------------------------------------------------------------------------ */
int64_t orc_block_bytes(int G) { return (int64_t)(G / 8) * 128 + 64 + 64; }

static inline uint8_t* blk_nib(uint8_t* blk) { return blk; }
static inline uint16_t* blk_d(uint8_t* blk, int G) { return (uint16_t*)(blk + (G / 8) * 128); }
static inline uint16_t* blk_m(uint8_t* blk, int G) { return (uint16_t*)(blk + (G / 8) * 128 + 64); }

/* element (k,n) of a block: byte (k>>3)*128 + n*4 + (k&3); high nibble iff (k/4)&1
 * (ops/op_fc.hpp:39-48) */
static inline void nib_set(uint8_t* nib, int k, int n, int v) {
    uint8_t* b = &nib[(k >> 3) * 128 + n * 4 + (k & 3)];
    if ((k >> 2) & 1)
        *b = (uint8_t)((*b & 0x0F) | (v << 4));
    else
        *b = (uint8_t)((*b & 0xF0) | (v & 0x0F));
}
static inline int nib_get(const uint8_t* nib, int k, int n) {
    uint8_t b = nib[(k >> 3) * 128 + n * 4 + (k & 3)];
    return ((k >> 2) & 1) ? (b >> 4) & 0xF : (b & 0xF);
}

/* ---- offline_FC_quant_Q4A (ops/op_fc.hpp:151-219; get_min_max :112-122).
 *      wei fp32 [N,K] row-major -> out [ceil(N/32), ceil(K/G), blk(G)].
 *      The reference leaves the nibbles of padded rows (n >= N) unwritten in an uninitialised
 *      buffer; here the buffer is zero-filled first, so those nibbles read 0.
 *      The reference's min/max scan always reads G floats even past K (:184); this restatement
 *      requires K % G == 0 for the real rows like every shape the reference is used with, and
 *      clips the scan to K otherwise. -------------------------------------------------------- */
void orc_quant_w(const float* wei, int64_t N, int64_t K, int G, uint8_t* out) {
    const int64_t Ng = cdiv(N, GROUP_N), Kg = cdiv(K, G), bb = orc_block_bytes(G);
    memset(out, 0, (size_t)(Ng * Kg * bb));
#pragma omp parallel for schedule(static)
    for (int64_t nb = 0; nb < Ng; nb++) {
        for (int64_t kb = 0; kb < Kg; kb++) {
            uint8_t* blk = out + (nb * Kg + kb) * bb;
            const int64_t k0 = kb * G;
            for (int ni = 0; ni < GROUP_N; ni++) {
                const int64_t n = nb * GROUP_N + ni;
                if (n >= N) {
                    blk_d(blk, G)[ni] = 0;
                    blk_m(blk, G)[ni] = 0;
                    continue;
                }
                const float* row = wei + n * K + k0;
                const int len = (int)((K - k0) < G ? (K - k0) : G);
                float vmin = row[0], vmax = row[0];
                for (int i = 1; i < len; i++) {
                    float a = row[i];
                    if (vmax < a) vmax = a;
                    if (vmin > a) vmin = a;
                }
                const float d = (vmax - vmin) / 15.0f;
                const float m = vmin;
                const float id = (d != 0) ? (1.0f / d) : 0.0f;
                blk_d(blk, G)[ni] = orc_fp32_to_fp16(d);
                blk_m(blk, G)[ni] = orc_fp32_to_fp16(m);
                for (int ki = 0; ki < G; ki++) {
                    int q = 0;
                    if (k0 + ki < K) {
                        float r = roundf((row[ki] - m) * id); /* half away from zero (:209) */
                        r = fminf(15.0f, fmaxf(r, 0.0f));
                        q = (int)(int8_t)r;
                    }
                    nib_set(blk_nib(blk), ki, ni, q);
                }
            }
        }
    }
}

/* ---- offline_FC_dequant_Q4A (ops/op_fc.hpp:124-149; q4_1_block::get :49-61): d*q + m with the
 *      fp16-rounded d,m; out fp32 [Ng*32, Kg*G].  The source writes `d * q + m`; whether the
 *      reference's compiler contracts it is not observable on the data the tests use, so this
 *      restatement uses the uncontracted form. ---------------------------------------------- */
void orc_dequant_w(const uint8_t* weiq, int64_t Ng, int64_t Kg, int G, float* out) {
    const int64_t bb = orc_block_bytes(G), ld = Kg * G;
#pragma omp parallel for schedule(static)
    for (int64_t nb = 0; nb < Ng; nb++)
        for (int64_t kb = 0; kb < Kg; kb++) {
            uint8_t* blk = (uint8_t*)weiq + (nb * Kg + kb) * bb;
            for (int ni = 0; ni < GROUP_N; ni++) {
                const float d = orc_fp16_to_fp32(blk_d(blk, G)[ni]);
                const float m = orc_fp16_to_fp32(blk_m(blk, G)[ni]);
                for (int ki = 0; ki < G; ki++)
                    out[(nb * GROUP_N + ni) * ld + kb * G + ki] = d * (float)nib_get(blk, ki, ni) + m;
            }
        }
}

/* unpack the 4-bit codes only: out uint8 [Ng*32, Kg*G] (test helper; layout of :39-48) */
void orc_unpack_codes(const uint8_t* weiq, int64_t Ng, int64_t Kg, int G, uint8_t* out) {
    const int64_t bb = orc_block_bytes(G), ld = Kg * G;
    for (int64_t nb = 0; nb < Ng; nb++)
        for (int64_t kb = 0; kb < Kg; kb++) {
            const uint8_t* blk = weiq + (nb * Kg + kb) * bb;
            for (int ni = 0; ni < GROUP_N; ni++)
                for (int ki = 0; ki < G; ki++)
                    out[(nb * GROUP_N + ni) * ld + kb * G + ki] = (uint8_t)nib_get(blk, ki, ni);
        }
}

/* ---- FC_dynamic_quantize_x (ops/op_fc.hpp:221-272), get_amax (ops/utils.hpp:177-197),
 *      quant_row_q8_0 (ops/utils.hpp:200-220).
 *      x fp32 [rows,K] -> xq int8 [rows,Kg*G], xd fp32 [rows,Kg], gsum fp32 [rows,Kg].
 *      Codes: mul by id, round half to EVEN (vroundps imm 0), saturate to int8 (packs).
 *      The reference's scalar tail for len%8 != 0 rounds half away instead (:217-219); it is
 *      reproduced for the last (len%8) elements of a short tail group. ---------------------- */
static inline int8_t sat_i8(float r) {
    if (!(r == r)) return (int8_t)-128; /* cvtps2dq(nan)=INT_MIN -> packs -> -128 */
    if (r > 127.0f) return 127;
    if (r < -128.0f) return -128;
    return (int8_t)(int)r;
}

void orc_quant_x(const float* x, int64_t rows, int64_t K, int G, int8_t* xq, float* xd, float* gsum) {
    const int64_t Kg = cdiv(K, G);
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++) {
        const float* raw = x + r * K;
        int8_t* q = xq + r * Kg * G;
        for (int64_t kb = 0; kb < Kg; kb++, raw += G, q += G) {
            const int64_t left = K - kb * G;
            const int len = (int)(left < G ? left : G);
            float amax = 0.0f;
            for (int i = 0; i < len; i++) {
                float a = fabsf(raw[i]);
                if (amax < a) amax = a;
            }
            const float d = amax / 127;
            const float id = (d != 0) ? (1.0f / d) : 0.0f;
            xd[r * Kg + kb] = d * 1.0f;
            const int vec = len & ~7;
            for (int i = 0; i < vec; i++) q[i] = sat_i8(nearbyintf(raw[i] * id)); /* RNE */
            for (int i = vec; i < len; i++) q[i] = (int8_t)roundf(raw[i] * id);   /* tail */
            for (int i = len; i < G; i++) q[i] = 0;
            float s = 0.0f;
            for (int i = 0; i < len; i++) s += raw[i]; /* sequential fp32 (:262-268) */
            gsum[r * Kg + kb] = s;
        }
    }
}

/* ---- integer core of fc_Q4A (ops/op_fc.hpp:337-363; vnni ops/utils.hpp:222-233):
 *      acc[r, n, kb] = sum_{ki<G} code(kb*G+ki, n) * xq[r, kb*G+ki]      (int32, exact)
 *      acc int32 [rows, Ng*32, Kg] -------------------------------------------------------- */
void orc_fc_partials(const int8_t* xq, int64_t rows, const uint8_t* weiq, int64_t Ng, int64_t Kg, int G, int32_t* acc) {
    const int64_t bb = orc_block_bytes(G), Np = Ng * GROUP_N;
#pragma omp parallel for schedule(static)
    for (int64_t nb = 0; nb < Ng; nb++)
        for (int64_t r = 0; r < rows; r++)
            for (int64_t kb = 0; kb < Kg; kb++) {
                const uint8_t* blk = weiq + (nb * Kg + kb) * bb;
                const int8_t* q = xq + (r * Kg + kb) * G;
                int32_t a[GROUP_N] = {0};
                for (int k8 = 0; k8 < G / 8; k8++) {
                    const uint8_t* rowb = blk + k8 * 128;
                    for (int ni = 0; ni < GROUP_N; ni++) {
                        int32_t s = 0;
                        for (int j = 0; j < 4; j++) {
                            uint8_t b = rowb[ni * 4 + j];
                            s += (int32_t)(b & 0xF) * q[k8 * 8 + j] + (int32_t)(b >> 4) * q[k8 * 8 + 4 + j];
                        }
                        a[ni] += s;
                    }
                }
                for (int ni = 0; ni < GROUP_N; ni++) acc[(r * Np + nb * GROUP_N + ni) * Kg + kb] = a[ni];
            }
}

/* ---- fc_Q4A (ops/op_fc.hpp:286-426).  x fp32 [rows,K] -> y fp32 [rows,N] (dense, stride N).
 *      Per output: for kb ascending  acc = fma(fp32(d16)*dx, float(acci), acc);
 *                                    acc = fma(fp32(m16), gsum, acc)          (:381-412).
 *      The reference stores 32 floats per strip regardless of N (:416-419); this restatement
 *      stores only n < N. -------------------------------------------------------------------- */
void orc_fc(const float* x, int64_t rows, int64_t K, const uint8_t* weiq, int64_t Ng, int64_t Kg, int G, int64_t N, float* y) {
    const int64_t bb = orc_block_bytes(G);
    int8_t* xq = (int8_t*)malloc((size_t)(rows * Kg * G));
    float* xd = (float*)malloc(sizeof(float) * (size_t)(rows * Kg));
    float* gs = (float*)malloc(sizeof(float) * (size_t)(rows * Kg));
    orc_quant_x(x, rows, K, G, xq, xd, gs);
#pragma omp parallel for schedule(static)
    for (int64_t nb = 0; nb < Ng; nb++)
        for (int64_t r = 0; r < rows; r++) {
            float accf[GROUP_N];
            for (int ni = 0; ni < GROUP_N; ni++) accf[ni] = 0.0f;
            for (int64_t kb = 0; kb < Kg; kb++) {
                const uint8_t* blk = weiq + (nb * Kg + kb) * bb;
                const int8_t* q = xq + (r * Kg + kb) * G;
                int32_t a[GROUP_N] = {0};
                for (int k8 = 0; k8 < G / 8; k8++) {
                    const uint8_t* rowb = blk + k8 * 128;
                    for (int ni = 0; ni < GROUP_N; ni++) {
                        int32_t s = 0;
                        for (int j = 0; j < 4; j++) {
                            uint8_t b = rowb[ni * 4 + j];
                            s += (int32_t)(b & 0xF) * q[k8 * 8 + j] + (int32_t)(b >> 4) * q[k8 * 8 + 4 + j];
                        }
                        a[ni] += s;
                    }
                }
                const float dx = xd[r * Kg + kb], g = gs[r * Kg + kb];
                const uint16_t* wd = blk_d((uint8_t*)blk, G);
                const uint16_t* wm = blk_m((uint8_t*)blk, G);
                for (int ni = 0; ni < GROUP_N; ni++) {
                    const float dd = orc_fp16_to_fp32(wd[ni]) * dx;
                    accf[ni] = fmaf(dd, (float)a[ni], accf[ni]);
                    accf[ni] = fmaf(orc_fp16_to_fp32(wm[ni]), g, accf[ni]);
                }
            }
            for (int ni = 0; ni < GROUP_N; ni++) {
                const int64_t n = nb * GROUP_N + ni;
                if (n < N) y[r * N + n] = accf[ni];
            }
        }
    free(xq);
    free(xd);
    free(gs);
}

/* ---- rope_embed (ops/op_attn.hpp:44-94, table :15-34): x fp32 [B,H,L,S] in place.
 *      theta = inv_freq[i] * (float)pos (fp32 product), cosf/sinf, rotate-half pairs (i, i+half).
 *      The reference caches the table keyed by length only (:15-17); this restatement
 *      recomputes it, i.e. it behaves like a fresh process. ---------------------------------- */
void orc_rope(float* x, int64_t B, int64_t H, int64_t L, int64_t S, const float* inv_freq, int64_t half, int position_id) {
#pragma omp parallel for schedule(static)
    for (int64_t bh = 0; bh < B * H; bh++)
        for (int64_t l = 0; l < L; l++) {
            float* px = x + (bh * L + l) * S;
            const int64_t pos = l + position_id;
            for (int64_t i = 0; i < half; i++) {
                const float xita = inv_freq[i] * pos;
                const float c = cosf(xita), s = sinf(xita);
                const float x0 = px[i], x1 = px[i + half];
                px[i] = c * x0 - s * x1;
                px[i + half] = s * x0 + c * x1;
            }
        }
}

/* ---- _softmax (ops/utils.hpp:484-490): max, exp(x-max), sum, scale by 1/sum.  The reference's
 *      exp is a 5-term polynomial that returns exactly 0 below ln(FLT_MIN) (ops/utils.hpp:
 *      293-371); expf differs from it by ~1e-7 relative and also underflows to 0 for the
 *      -FLT_MAX mask value. ------------------------------------------------------------------ */
static void softmax_row(float* a, int64_t n) {
    float mx = -FLT_MAX;
    for (int64_t i = 0; i < n; i++)
        if (a[i] > mx) mx = a[i];
    float sum = 0.0f;
    for (int64_t i = 0; i < n; i++) {
        a[i] = expf(a[i] - mx);
        sum += a[i];
    }
    const float sc = 1.0f / sum;
    for (int64_t i = 0; i < n; i++) a[i] *= sc;
}

/* softmax op (ops/op_misc.hpp:183-194): in place over the last dim */
void orc_softmax(float* x, int64_t rows, int64_t K) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++) softmax_row(x + r * K, K);
}

/* mm_qk / mm_qk42 / mm_qk81 / mm_qk24 (ops/op_attn.hpp:149-193, 195-298, 300-422, 424-515): the four
 *      benchmark ops compute one product, attn_w[b,h,pq,pk] = dot(q[b,h,pq,:], k[b,h,pk,:]) * (1/sqrt(S)),
 *      with q addressed through strides (elements) and the cache plane holding kv_max rows per head. */
void orc_mm_qk(const float* q, int64_t qs_b, int64_t qs_h, int64_t qs_q, const float* kcache, int64_t kv_max,
               float* attn_w, int64_t B, int64_t H, int64_t qL, int64_t kvLen, int64_t S) {
    const float d_scale = 1.0f / sqrtf((float)S);
#pragma omp parallel for schedule(static)
    for (int64_t bh = 0; bh < B * H; bh++) {
        const int64_t b = bh / H, h = bh % H;
        for (int64_t pq = 0; pq < qL; pq++) {
            const float* qr = q + b * qs_b + h * qs_h + pq * qs_q;
            for (int64_t pk = 0; pk < kvLen; pk++) {
                const float* kr = kcache + (bh * kv_max + pk) * S;
                float sum = 0.0f;
                for (int64_t s = 0; s < S; s++) sum += qr[s] * kr[s];
                attn_w[(bh * qL + pq) * kvLen + pk] = sum * d_scale;
            }
        }
    }
}

/* ---- attention_rope2 / attention_rope (ops/op_attn.hpp:721-1029 / :518-718; same contract).
 *      q,k,v fp32 [B,qL,H*S]; kv_cache fp32 [planes,B,H,maxlen,S]; slots int32 [qL].
 *      (1) rope q,k in place (k stays rotated, :760-761)   (2) cache[2l+{0,1},b,h,slots[p],:] = k,v
 *      (3) kvLen = min(pos+qL, maxlen)                      (4) w = (q.k)/sqrt(S) for pk < kvLen
 *      (5) for p' in (pq,qL): w[pq, slots[p']] = -FLT_MAX   (6) softmax  (7) q <- w.V         */
void orc_attention(float* q, float* k, float* v, int64_t B, int64_t qL, int64_t H, int64_t S, const float* inv_freq,
                   int64_t half, float* kv_cache, int64_t planes, int64_t maxlen, const int32_t* slots, int position_id,
                   int layer_id) {
    (void)planes;
    float* kc = kv_cache + (int64_t)(2 * layer_id + 0) * B * H * maxlen * S;
    float* vc = kv_cache + (int64_t)(2 * layer_id + 1) * B * H * maxlen * S;
    /* q,k are [B,qL,H,S] in memory: rope per (b,l,h) */
#pragma omp parallel for schedule(static)
    for (int64_t bh = 0; bh < B * H; bh++) {
        const int64_t b = bh / H, h = bh % H;
        for (int64_t l = 0; l < qL; l++) {
            const int64_t pos = l + position_id;
            float* pq = q + ((b * qL + l) * H + h) * S;
            float* pk = k + ((b * qL + l) * H + h) * S;
            for (int64_t i = 0; i < half; i++) {
                const float xita = inv_freq[i] * pos;
                const float c = cosf(xita), s = sinf(xita);
                float x0 = pq[i], x1 = pq[i + half];
                pq[i] = c * x0 - s * x1;
                pq[i + half] = s * x0 + c * x1;
                x0 = pk[i];
                x1 = pk[i + half];
                pk[i] = c * x0 - s * x1;
                pk[i + half] = s * x0 + c * x1;
            }
            memcpy(kc + ((b * H + h) * maxlen + slots[l]) * S, pk, sizeof(float) * S);
            memcpy(vc + ((b * H + h) * maxlen + slots[l]) * S, v + ((b * qL + l) * H + h) * S, sizeof(float) * S);
        }
    }
    int64_t kvLen = position_id + qL;
    if (kvLen > maxlen) kvLen = maxlen;
    const float d_scale = 1.0f / sqrtf((float)S);
#pragma omp parallel
    {
        float* w = (float*)malloc(sizeof(float) * (size_t)kvLen);
        float* o = (float*)malloc(sizeof(float) * (size_t)S);
#pragma omp for schedule(static)
        for (int64_t bh = 0; bh < B * H; bh++) {
            const int64_t b = bh / H, h = bh % H;
            const float* kb = kc + (b * H + h) * maxlen * S;
            const float* vb = vc + (b * H + h) * maxlen * S;
            for (int64_t l = 0; l < qL; l++) {
                float* pq = q + ((b * qL + l) * H + h) * S;
                for (int64_t p = 0; p < kvLen; p++) {
                    float s = 0.0f;
                    for (int64_t i = 0; i < S; i++) s = fmaf(pq[i], kb[p * S + i], s);
                    w[p] = s * d_scale;
                }
                for (int64_t p2 = l + 1; p2 < qL; p2++) w[slots[p2]] = -FLT_MAX;
                softmax_row(w, kvLen);
                for (int64_t i = 0; i < S; i++) o[i] = 0.0f;
                for (int64_t p = 0; p < kvLen; p++)
                    for (int64_t i = 0; i < S; i++) o[i] = fmaf(w[p], vb[p * S + i], o[i]);
                memcpy(pq, o, sizeof(float) * S);
            }
        }
        free(w);
        free(o);
    }
}

/* ---- rmsnorm (ops/op_misc.hpp:142-181): x * (1/sqrt(mean(x^2)+eps)) * w, in place ---------- */
void orc_rmsnorm(float* x, int64_t rows, int64_t Hd, const float* w, float eps) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++) {
        float* p = x + r * Hd;
        float ss = 0.0f;
        for (int64_t i = 0; i < Hd; i++) ss = fmaf(p[i], p[i], ss);
        const float rs = 1.0f / sqrtf(ss / Hd + eps);
        for (int64_t i = 0; i < Hd; i++) p[i] = p[i] * rs * w[i];
    }
}

/* iadd / imul (ops/op_misc.hpp:55-107): a op= b, b either [rows,inner] or [inner] broadcast */
void orc_iadd(float* a, const float* b, int64_t rows, int64_t inner, int b_rank1) {
    for (int64_t r = 0; r < rows; r++)
        for (int64_t i = 0; i < inner; i++) a[r * inner + i] += b[(b_rank1 ? 0 : r * inner) + i];
}
void orc_imul(float* a, const float* b, int64_t rows, int64_t inner, int b_rank1) {
    for (int64_t r = 0; r < rows; r++)
        for (int64_t i = 0; i < inner; i++) a[r * inner + i] *= b[(b_rank1 ? 0 : r * inner) + i];
}

/* itrans "silu" (ops/op_misc.hpp:127-138): x * 1/(1+exp(-x)).  The reference uses the 12-bit
 * rcpps approximation (ops/utils.hpp:373-378), so it is itself ~3e-4 off the exact value. */
void orc_silu(float* a, int64_t n) {
    for (int64_t i = 0; i < n; i++) a[i] = a[i] * (1.0f / (1.0f + expf(-a[i])));
}

/* embedding_q8c_quant_w (ops/op_embedding.hpp:51-78): per-row amax/127 scale + RNE int8 codes */
void orc_embedding_q8c_quant_w(const float* w, int64_t V, int64_t E, int8_t* q, float* scales) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < V; r++) {
        const float* raw = w + r * E;
        float amax = 0.0f;
        for (int64_t i = 0; i < E; i++) {
            float a = fabsf(raw[i]);
            if (amax < a) amax = a;
        }
        const float d = amax / 127;
        const float id = (d != 0) ? (1.0f / d) : 0.0f;
        scales[r] = d;
        const int64_t vec = E & ~(int64_t)7;
        for (int64_t i = 0; i < vec; i++) q[r * E + i] = sat_i8(nearbyintf(raw[i] * id));
        for (int64_t i = vec; i < E; i++) q[r * E + i] = (int8_t)roundf(raw[i] * id);
    }
}

/* embedding_q8c (ops/op_embedding.hpp:81-137): out[i,:] = scales[id] * q[id,:] */
void orc_embedding_q8c(float* out, const int64_t* ids, int64_t n, const int8_t* q, const float* scales, int64_t E) {
    for (int64_t i = 0; i < n; i++)
        for (int64_t e = 0; e < E; e++) out[i * E + e] = scales[ids[i]] * (float)q[ids[i] * E + e];
}

int orc_max_threads(void) { return omp_get_max_threads(); }
void orc_set_threads(int n) { omp_set_num_threads(n > 0 ? n : omp_get_num_procs()); }
