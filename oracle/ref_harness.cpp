// TEST INFRASTRUCTURE ONLY.  C-callable shim around the *unmodified* reference kernels.
//
// This translation unit contains no algorithm of its own: it wraps raw host pointers in the
// reference's `tensor` views, calls the reference's functions and copies results out.  It is
// compiled by oracle/Makefile against the headers where they lie (-I/root/reference/ops) and the
// result goes to oracle/_ref/ only.  The reference headers define non-inline free functions, so
// they may be included from exactly one TU -- this one (same include order as ops/main.cpp:1-11).
//
// Reference entry points wrapped (file:line in /root/reference):
//   offline_FC_quant_Q4A     ops/op_fc.hpp:151     offline_FC_dequant_Q4A  ops/op_fc.hpp:124
//   FC_dynamic_quantize_x    ops/op_fc.hpp:221     fc_Q4A                  ops/op_fc.hpp:286
//   rope_embed               ops/op_attn.hpp:44    attention_rope          ops/op_attn.hpp:518
//   attention_rope2          ops/op_attn.hpp:721   softmax                 ops/op_misc.hpp:183
//   rmsnorm/iadd/imul/itrans ops/op_misc.hpp:55-181
//   embedding_q8c_quant_w / embedding_q8c          ops/op_embedding.hpp:51,108
#include <algorithm>
#include <cassert>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <iostream>
#include <limits>
#include <string>
#include <vector>

#include "tensor.hpp"
#include "utils.hpp"
#include "op_fc.hpp"
#include "op_attn.hpp"
#include "op_embedding.hpp"
#include "op_misc.hpp"

namespace {

thread_local std::string g_last_error;

template <typename T>
tensor view(const T* p, std::vector<int64_t> shape) {
    tensor t;
    t.reset(const_cast<T*>(p), shape);
    return t;
}

template <typename F>
int guarded(F&& f) {
    try {
        f();
        return 0;
    } catch (const std::exception& e) {
        g_last_error = e.what();
        return 1;
    }
}

}  // namespace

extern "C" {

const char* ref_last_error() { return g_last_error.c_str(); }

int ref_group_k() { return q4_block::group_k; }
int ref_block_bytes() { return static_cast<int>(sizeof(q4_block)); }
int ref_has_avxvnni() {
#if __AVXVNNI__
    return 1;
#else
    return 0;
#endif
}
int ref_max_threads() { return omp_get_max_threads(); }
void ref_set_threads(int n) { omp_set_num_threads(n > 0 ? n : omp_get_num_procs()); }

// wei fp32 [N,K] -> out int8 [ceil(N/32), ceil(K/G), sizeof(q4_block)]
int ref_offline_FC_quant_Q4A(const float* wei, int64_t N, int64_t K, int8_t* out) {
    return guarded([&] {
        tensor r = offline_FC_quant_Q4A(view(wei, {N, K}));
        memcpy(out, r.data<int8_t>(), r.byte_size());
    });
}

// weiq int8 [Ng,Kg,blk] -> out fp32 [Ng*32, Kg*G]
int ref_offline_FC_dequant_Q4A(const int8_t* weiq, int64_t Ng, int64_t Kg, float* out) {
    return guarded([&] {
        tensor r = offline_FC_dequant_Q4A(view(weiq, {Ng, Kg, (int64_t)sizeof(q4_block)}));
        memcpy(out, r.data<float>(), r.byte_size());
    });
}

// x fp32 [B,M,K] -> xq int8 [B,M,Kg*G], xd fp32 [B,M,Kg], gsum fp32 [B,M,Kg]
int ref_FC_dynamic_quantize_x(const float* x, int64_t B, int64_t M, int64_t K, int8_t* xq, float* xd, float* gsum) {
    return guarded([&] {
        int64_t G = q4_block::group_k;
        int64_t Kg = (K + G - 1) / G;
        tensor tx = view(x, {B, M, K});
        tensor txq = view(xq, {B, M, Kg * G});
        tensor txd = view(xd, {B, M, Kg});
        tensor tgs = view(gsum, {B, M, Kg});
        FC_dynamic_quantize_x(tx, txq, txd, &tgs, Kg, G, 1.0f);
    });
}

// x fp32 [B,M,K], weiq int8 [Ng,Kg,blk] -> y fp32 [B,M,N]
int ref_fc_Q4A(const float* x, int64_t B, int64_t M, int64_t K, const int8_t* weiq, int64_t Ng, int64_t Kg, int N, float* y) {
    return guarded([&] {
        tensor r = fc_Q4A(view(x, {B, M, K}), view(weiq, {Ng, Kg, (int64_t)sizeof(q4_block)}), N);
        memcpy(y, r.data<float>(), r.byte_size());
    });
}

// in place on x fp32 [B,H,L,S]
int ref_rope_embed(float* x, int64_t B, int64_t H, int64_t L, int64_t S, const float* inv_freq, int64_t half, int position_id) {
    return guarded([&] {
        tensor tx = view(x, {B, H, L, S});
        rope_embed(tx, view(inv_freq, {half}), position_id);
    });
}

// version 1 -> attention_rope, 2 -> attention_rope2.  q,k,v fp32 [B,qL,H*S] (q overwritten with
// the output, k rotated in place); kv_cache fp32 [planes,B,H,maxlen,S]; slots int32 [qL].
int ref_attention_rope(int version, float* q, float* k, float* v, int64_t B, int64_t qL, int64_t H, int64_t S,
                       const float* inv_freq, int64_t half, float* kv_cache, int64_t planes, int64_t maxlen,
                       const int32_t* slots, int position_id, int layer_id) {
    return guarded([&] {
        tensor tq = view(q, {B, qL, H * S});
        tensor tk = view(k, {B, qL, H * S});
        tensor tv = view(v, {B, qL, H * S});
        tensor tc = view(kv_cache, {planes, B, H, maxlen, S});
        tensor ts = view(slots, {qL});
        tensor tf = view(inv_freq, {half});
        if (version == 1)
            attention_rope(tq, tk, tv, tf, tc, ts, position_id, layer_id);
        else
            attention_rope2(tq, tk, tv, tf, tc, ts, position_id, layer_id);
    });
}

// variant 0: mm_qk, 1: mm_qk42, 2: mm_qk81, 3: mm_qk24 (ops/op_attn.hpp:149-515).  q is [B,qL,H*S] for
// 0/2/3 and [B,H,qL,S] for 1; kcache [B,H,kv_max,S]; attn_w [B,H,qL,kvLen].  Variants 0/2/3 take kvLen from
// the cache's shape, so they are given kv_max == kvLen.
int ref_mm_qk(int variant, float* q, float* kcache, float* attn_w, int64_t B, int64_t H, int64_t qL, int64_t kv_max,
              int64_t kvLen, int64_t S) {
    return guarded([&] {
        tensor tk = view(kcache, {B, H, kv_max, S});
        tensor out;
        if (variant == 1) {
            tensor tq = view(q, {B, H, qL, S});
            tensor tw = view(attn_w, {B, H, qL, kvLen});
            mm_qk42(tq, tk, tw);
            return;
        }
        tensor tq = view(q, {B, qL, H * S});
        if (variant == 0)
            out = mm_qk(tq, tk);
        else if (variant == 2)
            out = mm_qk81(tq, tk);
        else
            out = mm_qk24(tq, tk);
        std::memcpy(attn_w, out.data<float>(), sizeof(float) * B * H * qL * kvLen);
    });
}

// in place, rows of length K
int ref_softmax(float* x, int64_t rows, int64_t K) {
    return guarded([&] { softmax(view(x, {rows, K})); });
}

int ref_rmsnorm(float* x, int64_t B, int64_t L, int64_t Hd, const float* w, float eps) {
    return guarded([&] { rmsnorm(view(x, {B, L, Hd}), view(w, {Hd}), eps); });
}

// a += b ; b is [rows,inner] (b_rank1 == 0) or [inner] broadcast (b_rank1 != 0)
int ref_iadd(float* a, const float* b, int64_t rows, int64_t inner, int b_rank1) {
    return guarded([&] {
        tensor tb = b_rank1 ? view(b, {inner}) : view(b, {rows, inner});
        iadd(view(a, {rows, inner}), tb);
    });
}

int ref_imul(float* a, const float* b, int64_t rows, int64_t inner, int b_rank1) {
    return guarded([&] {
        tensor tb = b_rank1 ? view(b, {inner}) : view(b, {rows, inner});
        imul(view(a, {rows, inner}), tb);
    });
}

int ref_itrans_silu(float* a, int64_t rows, int64_t inner) {
    return guarded([&] { itrans(view(a, {rows, inner}), "silu"); });
}

// w fp32 [V,E] -> q int8 [V,E], scales fp32 [V]
int ref_embedding_q8c_quant_w(const float* w, int64_t V, int64_t E, int8_t* q, float* scales) {
    return guarded([&] {
        tensor tw = view(w, {V, E});
        auto r = embedding_q8c_quant_w(tw);
        memcpy(q, r[0].data<int8_t>(), r[0].byte_size());
        memcpy(scales, r[1].data<float>(), r[1].byte_size());
    });
}

// ids int64 [n] ; out fp32 [n,E]
int ref_embedding_q8c(float* out, const int64_t* ids, int64_t n, const int8_t* q, const float* scales, int64_t V, int64_t E) {
    return guarded([&] { embedding_q8c(view(out, {n, E}), view(ids, {n}), view(q, {V, E}), view(scales, {V})); });
}

}  // extern "C"
