// C ABI of the Q4_1 x Q8 fully-connected op: argument checks, workspace layout and dispatch
// between the dot4 streaming kernel (few rows) and the int8 MFMA kernel (many rows).
#include "common.h"

#include <mutex>

namespace llmops {

constexpr int kMaxGemvRows = 8;

int launch_quant_x(const float* x, int64_t rows, int64_t K, int group_k, int8_t* xq, float* xd, float* gsum, float2* xsT,
                   bool exact_sum, hipStream_t stream);
int launch_quant_x_fused(const float* x, int64_t rows, int64_t K, int group_k, const float* norm_w, float eps, bool glu_in,
                         int8_t* xq, float* xd, float* gsum, float2* xsT, hipStream_t stream);
int launch_strip_sumsq(const float* y, int64_t rows, int64_t N, float* out, hipStream_t st);
size_t gemv_workspace_bytes(int64_t rows, int64_t Ng, int64_t Kg, int G);
int launch_gemv(const uint8_t* w, const int8_t* xq, const float* xd, const float* gs, float* y, float* part,
                unsigned* counters, int64_t rows, int64_t Ng, int64_t Kg, int G, int64_t N, hipStream_t st);
int launch_gemv_fused(const uint8_t* w, const float* x, float* y, float* part, unsigned* counters, int64_t rows, int64_t Ng,
                      int64_t Kg, int G, int64_t N, const float* residual, const float* norm_w, float eps, int glu,
                      const float* sumsq_in, int sumsq_parts, float* sumsq_out, hipStream_t st, const DumpBufs* dump = nullptr,
                      const float* rec_stats = nullptr, const float* rec_outs = nullptr, int rec_chunks = 0);
int launch_add(float* a, const float* b, int64_t total, hipStream_t st);
int launch_gemv_partials(const uint8_t* w, const int8_t* xq, int32_t* acc, int64_t rows, int64_t Ng, int64_t Kg, int G,
                         hipStream_t st);
size_t gemm_workspace_bytes(int64_t rows, int64_t Ng, int64_t Kg, int G);
int launch_gemm(const uint8_t* w, const int8_t* xq, const float* xd, const float* gs, const float2* xsT, float* y,
                float* part, unsigned* counters, int64_t rows, int64_t Ng, int64_t Kg, int G, int64_t N, const float* residual,
                hipStream_t st);
int launch_gemm_partials(const uint8_t* w, const int8_t* xq, int32_t* acc, int64_t rows, int64_t Ng, int64_t Kg, int G,
                         bool two_groups, hipStream_t st);
int launch_fc_rows(const uint8_t* w, const int8_t* xq, const float2* xsT, float* y, int64_t rows, int64_t Ng, int64_t Kg,
                   int64_t N, const float* residual, unsigned long long* slots, size_t slot_bytes, hipStream_t st);
int launch_fc_rows_partials(const uint8_t* w, const int8_t* xq, int32_t* acc, int64_t rows, int64_t Ng, int64_t Kg,
                            hipStream_t st);
bool gemm_rows_kernel_enabled();

static inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

struct FcWorkspace {
    size_t off_xq, off_xd, off_gs, off_xst, off_part, total;
};

static FcWorkspace fc_layout(int64_t rows, int64_t Ng, int64_t Kg, int G) {
    FcWorkspace w;
    size_t o = LLMOPS_FC_COUNTER_BYTES;
    w.off_xq = o;
    o = align_up(o + (size_t)rows * Kg * G, 256);
    w.off_xd = o;
    o = align_up(o + (size_t)rows * Kg * sizeof(float), 256);
    w.off_gs = o;
    o = align_up(o + (size_t)rows * Kg * sizeof(float), 256);
    w.off_xst = o;
    // (+256: the weight-streaming MFMA kernel fetches the pairs of whole 16-row tiles, up to 31 pairs past the last row)
    o = align_up(o + (size_t)rows * Kg * 2 * sizeof(float) + 256, 256);
    w.off_part = o;
    o = align_up(o + (rows <= kMaxGemvRows ? gemv_workspace_bytes(rows, Ng, Kg, G) : gemm_workspace_bytes(rows, Ng, Kg, G)), 256);
    w.total = o;
    return w;
}

}  // namespace llmops

using namespace llmops;

extern "C" size_t llmops_fc_Q4A_workspace_bytes(int64_t rows, int64_t K, int64_t Ng, int64_t Kg, int group_k) {
    (void)K;
    if (!valid_group(group_k) || rows <= 0 || Ng <= 0 || Kg <= 0) return 0;
    return fc_layout(rows, Ng, Kg, group_k).total;
}

// from how many rows the weight-streaming MFMA kernel takes over from the streaming kernel that quantizes
// on the fly: tensors of up to 256 strips / of more
static int g_rows_from_small = 4, g_rows_from_large = 3;

// argument checks of fc_Q4A that do not involve the workspace
static int fc_check_args(const float* x, int64_t rows, int64_t K, const int8_t* weiq, int64_t Ng, int64_t Kg, int group_k,
                         int64_t N, const float* y) {
    LLMOPS_REQUIRE(valid_group(group_k));
    LLMOPS_REQUIRE(x != nullptr && weiq != nullptr && y != nullptr);
    LLMOPS_REQUIRE(rows > 0 && K > 0 && Ng > 0 && Kg > 0);
    LLMOPS_REQUIRE(K > (Kg - 1) * group_k && K <= Kg * group_k);  // a short last k-group is zero padded (ops/op_fc.hpp:259-261)
    LLMOPS_REQUIRE(N > (Ng - 1) * kGroupN && N <= Ng * kGroupN);
    LLMOPS_REQUIRE(Ng <= kTicketBytes / 4);
    LLMOPS_REQUIRE(Ng * 64 < ((int64_t)1 << 31));
    LLMOPS_REQUIRE(aligned(weiq, 16) && aligned(x, K != Kg * group_k ? 4 : 8));
    return LLMOPS_OK;
}

// the product for activations that a quantization launch has left in the workspace (more rows than the streaming
// kernel that quantizes on the fly takes)
static int fc_product_many_rows(const uint8_t* w, uint8_t* ws, const FcWorkspace& lay, int64_t rows, int64_t Ng, int64_t Kg,
                                int group_k, int64_t N, const float* residual, float* y, hipStream_t st) {
    const int8_t* xq = reinterpret_cast<const int8_t*>(ws + lay.off_xq);
    const float* xd = reinterpret_cast<const float*>(ws + lay.off_xd);
    const float* gs = reinterpret_cast<const float*>(ws + lay.off_gs);
    const float2* xst = reinterpret_cast<const float2*>(ws + lay.off_xst);
    const bool rows_kernel = group_k == 128 && Ng >= 64 && gemm_rows_kernel_enabled();
    // up to 16 rows are still bound by the weight stream: one strip per workgroup, MFMA inner product
    // (measured against the tiled kernel: 15 vs 18 us at 16 rows, 11008x4096).  17..32 rows (two row tiles
    // per wave) only win for tensors of fewer than 256 strips, where the tiled kernel has too few tiles
    // (us, tiled / streaming: 4096x4096 at 17 rows 20.2 / 9.9, at 32 rows 24.3 / 11.9; 4096x11008 at 24 rows
    // 22.0 / 15.7; 11008x4096 at 24 rows 19.3 / 18.8; 12288x4096 17.9 / 19.0; 22016x4096 23.0 / 27.4)
    if (rows_kernel && (rows <= 16 || (rows <= 32 && Ng < 256)))
        return launch_fc_rows(w, xq, xst, y, rows, Ng, Kg, N, residual, reinterpret_cast<unsigned long long*>(ws + kTicketBytes),
                              LLMOPS_FC_COUNTER_BYTES - kTicketBytes, st);
    return launch_gemm(w, xq, xd, gs, xst, y, reinterpret_cast<float*>(ws + lay.off_part), reinterpret_cast<unsigned*>(ws), rows, Ng,
                       Kg, group_k, N, residual, st);
}

static int fc_impl(const float* x, int64_t rows, int64_t K, const int8_t* weiq, int64_t Ng, int64_t Kg, int group_k,
                   int64_t N, const float* residual, float* y, void* workspace, size_t workspace_bytes,
                   llmops_stream_t stream) {
    const int bad = fc_check_args(x, rows, K, weiq, Ng, Kg, group_k, N, y);
    if (bad) return bad;
    LLMOPS_REQUIRE(workspace != nullptr && aligned(workspace, 256));
    const bool k_tail = K != Kg * group_k;
    const FcWorkspace lay = fc_layout(rows, Ng, Kg, group_k);
    if (workspace_bytes < lay.total)
        return fail(LLMOPS_EWORKSPACE, "fc_Q4A needs %zu workspace bytes, got %zu", lay.total, workspace_bytes);
    uint8_t* ws = reinterpret_cast<uint8_t*>(workspace);
    unsigned* counters = reinterpret_cast<unsigned*>(ws);
    int8_t* xq = reinterpret_cast<int8_t*>(ws + lay.off_xq);
    float* xd = reinterpret_cast<float*>(ws + lay.off_xd);
    float* gs = reinterpret_cast<float*>(ws + lay.off_gs);
    float* part = reinterpret_cast<float*>(ws + lay.off_part);
    hipStream_t st = as_stream(stream);
    const uint8_t* w = reinterpret_cast<const uint8_t*>(weiq);
    // few rows: one launch, the streaming kernel quantizes the activations it needs on the fly.  Its work per
    // weight byte grows with the row count (every row is quantized and dotted separately), while the time of
    // the weight-streaming MFMA kernel below hardly depends on it, separate quantization launch included
    // (us, streaming / MFMA):
    //   4096x4096 (128 strips):    2 rows  6.0 /  8.0, 3 rows  7.5 /  8.2, 4 rows  8.3 /  8.2, 8 rows 10.2 /  8.4
    //   4096x11008 (128 strips):   2 rows  9.3 / 11.6, 3 rows 11.5 / 11.8, 4 rows 13.0 / 12.0, 8 rows 20.3 / 12.5
    //   8192x4096 (256 strips):    2 rows  6.7 /  8.9, 3 rows  8.1 /  8.6, 4 rows  8.8 /  8.6, 8 rows 14.5 /  8.9
    //   12288x4096 (384 strips):   2 rows  9.3 / 12.0, 3 rows 13.4 / 11.6, 4 rows 15.6 / 11.7, 8 rows 22.4 / 12.2
    //   22016x4096 (688 strips):   2 rows 12.8 / 16.1, 3 rows 20.1 / 16.0, 4 rows 22.2 / 15.3, 8 rows 31.0 / 16.1
    if (k_tail) {
        // K is not a whole number of k-groups (no shape the reference is used with): the general quantization kernel
        // pads the last group's codes with zeros, as FC_dynamic_quantize_x does, and the product runs on the codes
        float2* xst_t = reinterpret_cast<float2*>(ws + lay.off_xst);
        int rc_t = launch_quant_x(x, rows, K, group_k, xq, xd, gs, xst_t, false, st);
        if (rc_t) return rc_t;
        if (rows > kMaxGemvRows) return launch_gemm(w, xq, xd, gs, xst_t, y, part, counters, rows, Ng, Kg, group_k, N, residual, st);
        if (residual == y) return fail(LLMOPS_EINVAL, "fc_Q4A with a short last k-group and up to 8 rows: residual must not be y");
        rc_t = launch_gemv(w, xq, xd, gs, y, part, counters, rows, Ng, Kg, group_k, N, st);
        if (rc_t == 0 && residual != nullptr) rc_t = launch_add(y, residual, rows * N, st);
        return rc_t;
    }
    const bool rows_kernel = group_k == 128 && Ng >= 64 && gemm_rows_kernel_enabled();
    const bool gemv = rows <= kMaxGemvRows && !(rows_kernel && rows >= (Ng > 256 ? g_rows_from_large : g_rows_from_small));
    if (gemv)
        return launch_gemv_fused(w, x, y, part, counters, rows, Ng, Kg, group_k, N, residual, nullptr, 0.0f, 0, nullptr, 0,
                                 nullptr, st);
    float2* xst = reinterpret_cast<float2*>(ws + lay.off_xst);
    int rc = launch_quant_x(x, rows, K, group_k, xq, xd, gs, xst, false, st);
    if (rc) return rc;
    return fc_product_many_rows(w, ws, lay, rows, Ng, Kg, group_k, N, residual, y, st);
}

extern "C" int llmops_fc_Q4A(const float* x, int64_t rows, int64_t K, const int8_t* weiq, int64_t Ng, int64_t Kg,
                             int group_k, int64_t N, float* y, void* workspace, size_t workspace_bytes,
                             llmops_stream_t stream) {
    return fc_impl(x, rows, K, weiq, Ng, Kg, group_k, N, nullptr, y, workspace, workspace_bytes, stream);
}

extern "C" int llmops_fc_Q4A_residual(const float* x, int64_t rows, int64_t K, const int8_t* weiq, int64_t Ng,
                                      int64_t Kg, int group_k, int64_t N, const float* residual, float* y,
                                      void* workspace, size_t workspace_bytes, llmops_stream_t stream) {
    LLMOPS_REQUIRE(residual != nullptr);
    return fc_impl(x, rows, K, weiq, Ng, Kg, group_k, N, residual, y, workspace, workspace_bytes, stream);
}

static int fc_decode_impl(const float* x, int64_t rows, int64_t K, const int8_t* weiq, int64_t Ng, int64_t Kg, int group_k,
                          int64_t N_out, const float* norm_w, float eps, const float* residual, int glu,
                          const float* sumsq_in, int64_t sumsq_parts, float* sumsq_out, float* y, int64_t out_parts,
                          void* workspace, size_t workspace_bytes, llmops_stream_t stream) {
    LLMOPS_REQUIRE(valid_group(group_k));
    LLMOPS_REQUIRE(x != nullptr && weiq != nullptr && y != nullptr && workspace != nullptr);
    LLMOPS_REQUIRE(rows > 0);
    LLMOPS_REQUIRE(K > 0 && Ng > 0 && Kg > 0 && K == Kg * group_k);
    LLMOPS_REQUIRE(Ng <= kTicketBytes / 4 && Ng * 64 < ((int64_t)1 << 31));
    LLMOPS_REQUIRE(aligned(weiq, 16) && aligned(workspace, 256) && aligned(x, 8));
    LLMOPS_REQUIRE(glu >= 0 && glu <= 2);
    if (glu == 1) {
        LLMOPS_REQUIRE((Ng % 2) == 0 && residual == nullptr);
        LLMOPS_REQUIRE(N_out > (Ng / 2 - 1) * kGroupN && N_out <= Ng / 2 * kGroupN);
    } else {
        LLMOPS_REQUIRE(N_out > (Ng - 1) * kGroupN && N_out <= Ng * kGroupN);
    }
    if (norm_w != nullptr) LLMOPS_REQUIRE((K % 4) == 0 && aligned(x, 16) && aligned(norm_w, 8));
    if (sumsq_in != nullptr) LLMOPS_REQUIRE(norm_w != nullptr && sumsq_parts > 0 && sumsq_parts <= 65536);
    if (sumsq_out != nullptr) LLMOPS_REQUIRE(glu != 1);
    if (glu == 2) LLMOPS_REQUIRE(norm_w == nullptr && sumsq_in == nullptr);
    LLMOPS_REQUIRE(out_parts >= 1);
    if (out_parts > 1)
        LLMOPS_REQUIRE(glu != 1 && residual == nullptr && sumsq_out == nullptr && (Ng % out_parts) == 0 &&
                       N_out == Ng * kGroupN);
    const FcWorkspace lay = fc_layout(rows, Ng, Kg, group_k);
    if (workspace_bytes < lay.total)
        return fail(LLMOPS_EWORKSPACE, "fc_Q4A needs %zu workspace bytes, got %zu", lay.total, workspace_bytes);
    uint8_t* ws = reinterpret_cast<uint8_t*>(workspace);
    if (rows > kMaxGemvRows) {
        // More rows than the streaming kernel takes: the producer is folded into the quantization launch instead
        // (its fp32 result never goes through memory), the residual into the product's stores, and the sums of
        // squares take a launch of their own.  The statistic of the rmsnorm is computed from the row (sumsq_in is
        // not needed: the launch has the whole row in registers).
        if (glu == 1) return fail(LLMOPS_EINVAL, "fc_Q4A_decode with more than 8 rows: gate and up stacked (glu 2), not interleaved");
        hipStream_t st = as_stream(stream);
        int8_t* xq = reinterpret_cast<int8_t*>(ws + lay.off_xq);
        float* xd = reinterpret_cast<float*>(ws + lay.off_xd);
        float* gs = reinterpret_cast<float*>(ws + lay.off_gs);
        float2* xst = reinterpret_cast<float2*>(ws + lay.off_xst);
        int rc = (norm_w != nullptr || glu == 2)
                     ? launch_quant_x_fused(x, rows, K, group_k, norm_w, eps, glu == 2, xq, xd, gs, xst, st)
                     : launch_quant_x(x, rows, K, group_k, xq, xd, gs, xst, false, st);
        if (rc) return rc;
        if (out_parts > 1) {
            // y is [out_parts][rows][N_out / out_parts]: one product per slice of strips on the same quantized rows
            // (q, k and v of a fused q|k|v tensor come out as three dense matrices instead of one to be cut up)
            const int64_t ngp = Ng / out_parts, np = N_out / out_parts;
            for (int64_t p = 0; p < out_parts && rc == 0; p++)
                rc = fc_product_many_rows(reinterpret_cast<const uint8_t*>(weiq) + p * ngp * Kg * block_bytes(group_k), ws, lay,
                                          rows, ngp, Kg, group_k, np, nullptr, y + p * rows * np, st);
            return rc;
        }
        rc = fc_product_many_rows(reinterpret_cast<const uint8_t*>(weiq), ws, lay, rows, Ng, Kg, group_k, N_out, residual, y, st);
        if (rc == 0 && sumsq_out != nullptr) rc = launch_strip_sumsq(y, rows, N_out, sumsq_out, st);
        return rc;
    }
    LLMOPS_REQUIRE(out_parts == 1);  // (up to 8 rows: a slice of a row is as good as a row of its own)
    return launch_gemv_fused(reinterpret_cast<const uint8_t*>(weiq), x, y, reinterpret_cast<float*>(ws + lay.off_part),
                             reinterpret_cast<unsigned*>(ws), rows, Ng, Kg, group_k, N_out, residual, norm_w, eps, glu,
                             sumsq_in, (int)sumsq_parts, sumsq_out, as_stream(stream));
}

extern "C" int llmops_fc_Q4A_decode(const float* x, int64_t rows, int64_t K, const int8_t* weiq, int64_t Ng, int64_t Kg,
                                    int group_k, int64_t N_out, const float* norm_w, float eps, const float* residual,
                                    int glu, const float* sumsq_in, int64_t sumsq_parts, float* sumsq_out, float* y,
                                    void* workspace, size_t workspace_bytes, llmops_stream_t stream) {
    return fc_decode_impl(x, rows, K, weiq, Ng, Kg, group_k, N_out, norm_w, eps, residual, glu, sumsq_in, sumsq_parts, sumsq_out, y,
                          1, workspace, workspace_bytes, stream);
}

extern "C" int llmops_fc_Q4A_decode_parts(const float* x, int64_t rows, int64_t K, const int8_t* weiq, int64_t Ng, int64_t Kg,
                                          int group_k, int64_t N_out, const float* norm_w, float eps, int glu, int64_t out_parts,
                                          float* y, void* workspace, size_t workspace_bytes, llmops_stream_t stream) {
    LLMOPS_REQUIRE(rows > kMaxGemvRows);
    return fc_decode_impl(x, rows, K, weiq, Ng, Kg, group_k, N_out, norm_w, eps, nullptr, glu, nullptr, 0, nullptr, y, out_parts,
                          workspace, workspace_bytes, stream);
}

static int fc_decode_attn(const float* rec_stats, const float* rec_outs, int64_t chunks, int64_t H, const int8_t* weiq,
                          int64_t Ng, int64_t Kg, int64_t N_out, const float* residual, float* sumsq_out, float* y,
                          void* workspace, size_t workspace_bytes, llmops_stream_t stream, const DumpBufs* dump) {
    LLMOPS_REQUIRE(rec_stats != nullptr && rec_outs != nullptr && weiq != nullptr && y != nullptr && workspace != nullptr);
    LLMOPS_REQUIRE(chunks > 0 && chunks <= 8 && H > 0 && Ng > 0 && Kg > 0 && Kg == H);  // K = H * 128, group 128
    LLMOPS_REQUIRE(N_out > (Ng - 1) * kGroupN && N_out <= Ng * kGroupN);
    LLMOPS_REQUIRE(Ng <= kTicketBytes / 4 && Ng * 64 < ((int64_t)1 << 31));
    LLMOPS_REQUIRE(aligned(weiq, 16) && aligned(workspace, 256) && aligned(rec_stats, 16) && aligned(rec_outs, 16));
    const FcWorkspace lay = fc_layout(1, Ng, Kg, 128);
    if (workspace_bytes < lay.total)
        return fail(LLMOPS_EWORKSPACE, "fc_Q4A needs %zu workspace bytes, got %zu", lay.total, workspace_bytes);
    uint8_t* ws = reinterpret_cast<uint8_t*>(workspace);
    return launch_gemv_fused(reinterpret_cast<const uint8_t*>(weiq), rec_outs, y, reinterpret_cast<float*>(ws + lay.off_part),
                             reinterpret_cast<unsigned*>(ws), 1, Ng, Kg, 128, N_out, residual, nullptr, 0.0f, 0, nullptr, 0,
                             sumsq_out, as_stream(stream), dump, rec_stats, rec_outs, (int)chunks);
}

extern "C" int llmops_fc_Q4A_decode_attn(const float* rec_stats, const float* rec_outs, int64_t chunks, int64_t H,
                                         const int8_t* weiq, int64_t Ng, int64_t Kg, int64_t N_out, const float* residual,
                                         float* sumsq_out, float* y, void* workspace, size_t workspace_bytes,
                                         llmops_stream_t stream) {
    return fc_decode_attn(rec_stats, rec_outs, chunks, H, weiq, Ng, Kg, N_out, residual, sumsq_out, y, workspace, workspace_bytes,
                          stream, nullptr);
}

// the same kernel in its dump build (what it merged and quantized, and its int32 sums)
extern "C" int llmops_test_fc_decode_attn_dump(const float* rec_stats, const float* rec_outs, int64_t chunks, int64_t H,
                                               const int8_t* weiq, int64_t Ng, int64_t Kg, int64_t N_out, float* y, int8_t* xq,
                                               float* xd, float* gsum, int32_t* acc, void* workspace, size_t workspace_bytes,
                                               llmops_stream_t stream) {
    LLMOPS_TEST_HOOK();
    LLMOPS_REQUIRE(xq != nullptr && xd != nullptr && gsum != nullptr && acc != nullptr && aligned(xq, 4));
    const DumpBufs dump{xq, xd, gsum, acc};
    return fc_decode_attn(rec_stats, rec_outs, chunks, H, weiq, Ng, Kg, N_out, nullptr, nullptr, y, workspace, workspace_bytes,
                          stream, &dump);
}

extern "C" int llmops_fc_Q4A_prequantized(const int8_t* xq, const float* xd, const float* gsum, int64_t rows,
                                          const int8_t* weiq, int64_t Ng, int64_t Kg, int group_k, int64_t N, float* y,
                                          void* workspace, size_t workspace_bytes, llmops_stream_t stream) {
    LLMOPS_REQUIRE(valid_group(group_k));
    LLMOPS_REQUIRE(xq != nullptr && xd != nullptr && gsum != nullptr && weiq != nullptr && y != nullptr);
    LLMOPS_REQUIRE(workspace != nullptr);
    LLMOPS_REQUIRE(rows > 0 && Ng > 0 && Kg > 0);
    LLMOPS_REQUIRE(N > (Ng - 1) * kGroupN && N <= Ng * kGroupN);
    LLMOPS_REQUIRE(Ng <= kTicketBytes / 4);
    LLMOPS_REQUIRE(aligned(weiq, 16) && aligned(xq, 16) && aligned(workspace, 256));
    const FcWorkspace lay = fc_layout(rows, Ng, Kg, group_k);
    if (workspace_bytes < lay.total)
        return fail(LLMOPS_EWORKSPACE, "fc_Q4A needs %zu workspace bytes, got %zu", lay.total, workspace_bytes);
    uint8_t* ws = reinterpret_cast<uint8_t*>(workspace);
    float* part = reinterpret_cast<float*>(ws + lay.off_part);
    const uint8_t* w = reinterpret_cast<const uint8_t*>(weiq);
    hipStream_t st = as_stream(stream);
    if (rows <= kMaxGemvRows)
        return launch_gemv(w, xq, xd, gsum, y, part, reinterpret_cast<unsigned*>(ws), rows, Ng, Kg, group_k, N, st);
    return launch_gemm(w, xq, xd, gsum, nullptr, y, part, reinterpret_cast<unsigned*>(ws), rows, Ng, Kg, group_k, N, nullptr, st);
}

extern "C" int llmops_fc_Q4A_partials(const int8_t* xq, int64_t rows, const int8_t* weiq, int64_t Ng, int64_t Kg,
                                      int group_k, int32_t* acc, int use_mfma, llmops_stream_t stream) {
    LLMOPS_REQUIRE(valid_group(group_k));
    LLMOPS_REQUIRE(xq != nullptr && weiq != nullptr && acc != nullptr);
    LLMOPS_REQUIRE(rows > 0 && Ng > 0 && Kg > 0);
    LLMOPS_REQUIRE(aligned(weiq, 16) && aligned(xq, 16));
    LLMOPS_REQUIRE(Ng * Kg < ((int64_t)1 << 31));
    const uint8_t* w = reinterpret_cast<const uint8_t*>(weiq);
    LLMOPS_REQUIRE(use_mfma >= 0 && use_mfma <= 3 && (use_mfma < 2 || group_k == 128));
    if (use_mfma == 3) {
        LLMOPS_REQUIRE(rows <= 32);
        return launch_fc_rows_partials(w, xq, acc, rows, Ng, Kg, as_stream(stream));
    }
    if (use_mfma) return launch_gemm_partials(w, xq, acc, rows, Ng, Kg, group_k, use_mfma == 2, as_stream(stream));
    return launch_gemv_partials(w, xq, acc, rows, Ng, Kg, group_k, as_stream(stream));
}

extern "C" void llmops_test_fc_set_row_routing(int rows_from_small, int rows_from_large) {
    if (!test_hooks_enabled(__func__)) return;
    g_rows_from_small = rows_from_small >= 2 ? rows_from_small : 4;
    g_rows_from_large = rows_from_large >= 2 ? rows_from_large : 3;
}

// ---- fc_Q4A for callers that cannot allocate ---------------------------------------------------
// The workspace of llmops_fc_Q4A (arrival counters and exchange slots, activation codes and scales,
// split-K partial sums) lives in a fixed array in the library's device image instead of coming from
// the caller.  Each device holds its own copy of the array at its own address; the address is looked
// up once per device and only that pointer is ever handed to kernels (the array's name is a host-side
// handle, not a device address).
namespace llmops {

static __device__ __align__(256) unsigned char scratch[LLMOPS_FC_NOALLOC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
static void* g_scratch_ptr[kMaxDevices];
static std::mutex g_scratch_mutex;

// device pointer of this device's copy of `scratch`, resolved on first use with that device current
static int scratch_of_current_device(void** out) {
    int dev = -1;
    LLMOPS_HIP_CHECK(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return fail(LLMOPS_EINVAL, "device ordinal %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        void* ptr = nullptr;
        LLMOPS_HIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        if (ptr == nullptr) return fail(LLMOPS_EHIP, "hipGetSymbolAddress returned no address for the scratch array");
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return LLMOPS_OK;
}

// zero fill with plain vector stores (a kernel rather than a memset node: callers may be capturing a graph)
__global__ __launch_bounds__(256) void zero16_kernel(uint4* p, int64_t n16) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n16) p[i] = make_uint4(0, 0, 0, 0);
}

}  // namespace llmops

extern "C" size_t llmops_fc_Q4A_noalloc_scratch_bytes(void) { return LLMOPS_FC_NOALLOC_SCRATCH_BYTES; }

extern "C" int llmops_fc_workspace_reset(void* workspace, size_t workspace_bytes, llmops_stream_t stream) {
    LLMOPS_REQUIRE(workspace != nullptr && aligned(workspace, 256) && workspace_bytes >= 16);
    const size_t head = workspace_bytes < (size_t)LLMOPS_FC_COUNTER_BYTES ? workspace_bytes : (size_t)LLMOPS_FC_COUNTER_BYTES;
    const int64_t n16 = (int64_t)(head / 16);
    zero16_kernel<<<(unsigned)((n16 + 255) / 256), 256, 0, as_stream(stream)>>>(reinterpret_cast<uint4*>(workspace), n16);
    LLMOPS_LAUNCH_CHECK();
    return LLMOPS_OK;
}

extern "C" int llmops_fc_Q4A_noalloc(const float* x, int64_t rows, int64_t K, const int8_t* weiq, int64_t Ng, int64_t Kg,
                                     int group_k, int64_t N, float* y, llmops_stream_t stream) {
    // everything fc_impl will check is checked here first: a refused call must not enqueue the zero fill either
    const int bad = fc_check_args(x, rows, K, weiq, Ng, Kg, group_k, N, y);
    if (bad) return bad;
    const size_t need = fc_layout(rows, Ng, Kg, group_k).total;
    if (need > (size_t)LLMOPS_FC_NOALLOC_SCRATCH_BYTES)
        return fail(LLMOPS_EWORKSPACE,
                    "llmops_fc_Q4A_noalloc: rows=%lld, strips=%lld, k-groups=%lld need %zu scratch bytes, the built-in "
                    "scratch holds %zu; use llmops_fc_Q4A with a caller-provided workspace",
                    (long long)rows, (long long)Ng, (long long)Kg, need, (size_t)LLMOPS_FC_NOALLOC_SCRATCH_BYTES);
    void* ws = nullptr;
    const int rc = scratch_of_current_device(&ws);
    if (rc) return rc;
    // The array keeps whatever the last call on this device left in it.  Counters and exchange slots must
    // start at zero; the kernels leave them so, but a launch that failed half-way would not.
    const int64_t n16 = LLMOPS_FC_COUNTER_BYTES / 16;
    zero16_kernel<<<(unsigned)((n16 + 255) / 256), 256, 0, as_stream(stream)>>>(reinterpret_cast<uint4*>(ws), n16);
    LLMOPS_LAUNCH_CHECK();
    return fc_impl(x, rows, K, weiq, Ng, Kg, group_k, N, nullptr, y, ws, LLMOPS_FC_NOALLOC_SCRATCH_BYTES, stream);
}

// The production decode kernel in its dump build: y as llmops_fc_Q4A computes it for rows <= 8 with the kernel
// that quantizes on the fly, plus what that kernel quantized and its int32 sums.
extern "C" int llmops_test_fc_decode_dump(const float* x, int64_t rows, int64_t K, const int8_t* weiq, int64_t Ng, int64_t Kg,
                                          int group_k, int64_t N, float* y, int8_t* xq, float* xd, float* gsum, int32_t* acc,
                                          void* workspace, size_t workspace_bytes, llmops_stream_t stream) {
    LLMOPS_TEST_HOOK();
    LLMOPS_REQUIRE(valid_group(group_k));
    LLMOPS_REQUIRE(x != nullptr && weiq != nullptr && y != nullptr && workspace != nullptr);
    LLMOPS_REQUIRE(xq != nullptr && xd != nullptr && gsum != nullptr && acc != nullptr);
    LLMOPS_REQUIRE(rows > 0 && rows <= kMaxGemvRows && K > 0 && Ng > 0 && Kg > 0 && K == Kg * group_k);
    LLMOPS_REQUIRE(N > (Ng - 1) * kGroupN && N <= Ng * kGroupN);
    LLMOPS_REQUIRE(Ng <= kTicketBytes / 4 && Ng * Kg * kGroupN * rows < ((int64_t)1 << 31));
    LLMOPS_REQUIRE(aligned(weiq, 16) && aligned(workspace, 256) && aligned(x, 8) && aligned(xq, 4));
    const FcWorkspace lay = fc_layout(rows, Ng, Kg, group_k);
    if (workspace_bytes < lay.total)
        return fail(LLMOPS_EWORKSPACE, "fc_Q4A needs %zu workspace bytes, got %zu", lay.total, workspace_bytes);
    uint8_t* ws = reinterpret_cast<uint8_t*>(workspace);
    const DumpBufs dump{xq, xd, gsum, acc};
    return launch_gemv_fused(reinterpret_cast<const uint8_t*>(weiq), x, y, reinterpret_cast<float*>(ws + lay.off_part),
                             reinterpret_cast<unsigned*>(ws), rows, Ng, Kg, group_k, N, nullptr, nullptr, 0.0f, 0, nullptr, 0,
                             nullptr, as_stream(stream), &dump);
}
