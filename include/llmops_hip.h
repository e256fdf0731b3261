/* llmops_hip.h -- C ABI of the gfx950 (MI355X) implementation of the Q4_1 fully-connected path
 * and of the KV-cache attention op that wraps it.
 *
 * Every entry point replaces one function the reference binds into its `llmops` Python module
 * (PYBIND11_MODULE, /root/reference/ops/main.cpp:62-179); the citation beside each declaration
 * names that function.  A binding layer (pybind11, ctypes, cgo ...) passes plain device
 * pointers and sizes; no framework types cross this boundary.
 *
 * Conventions
 *  - All data pointers are DEVICE pointers on the current HIP device unless marked host.
 *  - Tensors are dense row-major with the reference's shapes and dtypes.
 *  - `stream` is a hipStream_t passed as void* (NULL = the default stream).  Calls only enqueue
 *    work; they never synchronise and never allocate device memory.
 *  - Every function returns 0 on success and a non-zero LLMOPS_E* code on failure; the message
 *    is available from llmops_last_error() (thread local).  Argument validation mirrors the
 *    reference's ASSERTs (ops/tensor.hpp:20-36) and happens before anything is enqueued.
 *  - group_k is 32 or 128 (the reference fixes it at compile time, ops/op_fc.hpp:109; here it
 *    is a run-time argument recoverable from the packed tensor's last dimension).
 *
 * Packed weight format == the reference's q4_1_block<G> (ops/op_fc.hpp:14-62), byte for byte:
 *   int8 [ceil(N/32)][ceil(K/G)][ (G/8)*128 nibble bytes | 32 x fp16 d | 32 x fp16 m ]
 *   element (k,n) of a block: byte (k>>3)*128 + n*4 + (k&3), high nibble iff (k>>2)&1.
 */
#ifndef LLMOPS_HIP_H
#define LLMOPS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LLMOPS_OK 0
#define LLMOPS_EINVAL 1   /* bad argument (shape, group size, null pointer, misalignment) */
#define LLMOPS_EWORKSPACE 2 /* workspace too small */
#define LLMOPS_EHIP 3     /* a HIP runtime call or kernel launch failed */

#define LLMOPS_CACHE_F32 0
#define LLMOPS_CACHE_F16 1

typedef void* llmops_stream_t;

const char* llmops_last_error(void);
int llmops_abi_version(void);

/* bytes of one packed block for group_k (640 / 2176); 0 if group_k is not supported */
int64_t llmops_q4a_block_bytes(int group_k);

/* ------------------------------------------------------------------------------------------
 * Q4_1 weight packing
 * ------------------------------------------------------------------------------------------ */

/* offline_FC_quant_Q4A (ops/op_fc.hpp:151-219, bound at ops/main.cpp:158).
 * wei fp32 [N,K], row stride `ld` elements -> weiq int8 [ceil(N/32), ceil(K/G), blk(G)].
 * Byte-exact with the reference for every real (n,k); nibbles of padded rows (n >= N), which the
 * reference leaves uninitialised, are written as 0. */
int llmops_offline_FC_quant_Q4A(const float* wei, int64_t N, int64_t K, int64_t ld, int group_k,
                                int8_t* weiq, llmops_stream_t stream);

/* offline_FC_dequant_Q4A (ops/op_fc.hpp:124-149, ops/main.cpp:159).
 * weiq [Ng,Kg,blk] -> out fp32 [Ng*32, Kg*G] = fp32(d)*q + fp32(m). */
int llmops_offline_FC_dequant_Q4A(const int8_t* weiq, int64_t Ng, int64_t Kg, int group_k,
                                  float* out, llmops_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Q8 dynamic activation quantization
 * ------------------------------------------------------------------------------------------ */

/* FC_dynamic_quantize_x (ops/op_fc.hpp:221-272; get_amax ops/utils.hpp:177-197, quant_row_q8_0
 * ops/utils.hpp:200-220).  x fp32 [rows,K] -> xq int8 [rows,Kg*G] (round half to even, zero
 * padded), xd fp32 [rows,Kg] = amax/127, gsum fp32 [rows,Kg] = left-to-right fp32 sum of the raw
 * group.  All three outputs are bit-exact with the reference.  K is any positive value: the last K % 8
 * values of a short last group take the reference's scalar tail, which rounds half away from zero
 * (ops/utils.hpp:217-219). */
int llmops_FC_dynamic_quantize_x(const float* x, int64_t rows, int64_t K, int group_k, int8_t* xq,
                                 float* xd, float* gsum, llmops_stream_t stream);

/* The form of FC_dynamic_quantize_x that the prefill FC runs (many rows, K % group_k == 0): xq and
 * xd bit-exact as above; gsum is summed as a tree (it only feeds the fp32 output, ops/op_fc.hpp:408). */
int llmops_FC_dynamic_quantize_x_rows(const float* x, int64_t rows, int64_t K, int group_k, int8_t* xq,
                                      float* xd, float* gsum, llmops_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Q4_1 x Q8 fully connected
 * ------------------------------------------------------------------------------------------ */

/* workspace bytes llmops_fc_Q4A needs for these sizes (activation codes, split-K partial sums and
 * the hand-off area of the k-splits: arrival counters and exchange slots).  The first
 * LLMOPS_FC_COUNTER_BYTES bytes of the workspace must be zero when the library first sees it; the
 * library leaves them zero after every call.  One workspace must not be shared by calls that can
 * overlap on the device. */
#define LLMOPS_FC_COUNTER_BYTES 3145728
size_t llmops_fc_Q4A_workspace_bytes(int64_t rows, int64_t K, int64_t Ng, int64_t Kg, int group_k);

/* fc_Q4A (ops/op_fc.hpp:286-426, bound at ops/main.cpp:160).
 * x fp32 [rows,K] (rows = B*M), weiq [Ng,Kg,blk] -> y fp32 [rows,N]:
 *   y[r,n] = sum_kb  fp32(d[n,kb])*dx[r,kb] * float(acc[r,n,kb]) + fp32(m[n,kb])*gsum[r,kb]
 * with acc the exact int32 dot product of 4-bit codes and int8 activation codes.  One or two rows (at
 * group 32 up to 8; at group 128 three rows of tensors of up to 256 strips as well) run the
 * HBM-streaming dot4 kernel, larger row counts the int8 MFMA kernels.  K may be any value in (Kg*G-G, Kg*G]: a short
 * last k-group is zero padded as the reference does (ops/op_fc.hpp:259-261; a separate quantization launch then,
 * not the tuned path: no shape the reference is used with has such a K); N any value in (Ng*32-32, Ng*32]. */
int llmops_fc_Q4A(const float* x, int64_t rows, int64_t K, const int8_t* weiq, int64_t Ng, int64_t Kg,
                  int group_k, int64_t N, float* y, void* workspace, size_t workspace_bytes,
                  llmops_stream_t stream);

/* Zero the hand-off area at the head of an FC or attention workspace (arrival counters, exchange slots: the first
 * min(workspace_bytes, LLMOPS_FC_COUNTER_BYTES) bytes) with a fill kernel on `stream`.  The kernels leave that area
 * zero after every call that runs to its end; a launch that did not (a device error in the middle of an op) may
 * leave parked values behind, after which two k-splits no longer meet and outputs are wrong.  Call this once, with no
 * op in flight on the workspace, before using it again.  No counterpart in the reference (its scratch is host
 * memory owned by one call). */
int llmops_fc_workspace_reset(void* workspace, size_t workspace_bytes, llmops_stream_t stream);

/* fc_Q4A for callers that cannot allocate device memory or carry a workspace around: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the
 * reference.  Same arguments, kernels and results as llmops_fc_Q4A, but the workspace is a fixed array of
 * LLMOPS_FC_NOALLOC_SCRATCH_BYTES inside the library's device image (every device the library runs on
 * holds its own copy until the process ends).  The call allocates and frees nothing.  Sizes whose
 * workspace (llmops_fc_Q4A_workspace_bytes) exceeds the array are refused with LLMOPS_EWORKSPACE.
 * Every call on a device shares that device's array: calls that can overlap on one device (two streams,
 * two host threads) race and must use llmops_fc_Q4A with a workspace each instead.  The first call on a
 * device looks the array's address up (hipGetSymbolAddress); make that call outside stream capture. */
#define LLMOPS_FC_NOALLOC_SCRATCH_BYTES (32u << 20)
size_t llmops_fc_Q4A_noalloc_scratch_bytes(void);
int llmops_fc_Q4A_noalloc(const float* x, int64_t rows, int64_t K, const int8_t* weiq, int64_t Ng, int64_t Kg,
                          int group_k, int64_t N, float* y, llmops_stream_t stream);

/* fc_Q4A followed by iadd(y, residual) (ops/op_misc.hpp:55-79) in one launch for rows <= 8:
 * y = fc_Q4A(x) + residual, residual fp32 [rows,N].  The decode step uses it for the o and down
 * projections (chatllama/main.py:355-357,372-375).  residual may be y itself (the add in place the
 * reference does), except when K is not a multiple of group_k and rows <= 8: that combination adds
 * the residual in a second launch and is refused with LLMOPS_EINVAL if the two alias. */
int llmops_fc_Q4A_residual(const float* x, int64_t rows, int64_t K, const int8_t* weiq, int64_t Ng, int64_t Kg,
                           int group_k, int64_t N, const float* residual, float* y, void* workspace,
                           size_t workspace_bytes, llmops_stream_t stream);

/* fc_Q4A with the neighbouring ops of chatllama/main.py:344-375 folded in.  Up to 8 rows (a decode step) it is
 * one launch.  With more rows (a batch of decode steps, a prompt) the producer of the input -- rmsnorm, or
 * silu(gate)*up -- runs inside the quantization launch, so that its fp32 result never passes through memory,
 * the residual is added in the product's stores and the sums of squares take a launch of their own; the codes,
 * scales and results are those of the separate ops (llmops_rmsnorm_out / llmops_silu_mul, then llmops_fc_Q4A).
 * More than 8 rows need whole 16-byte aligned rows, take glu 0 or 2 (2 with group 128 only), hidden sizes up to
 * 16384 with norm_w, and compute the rmsnorm's statistic from the row (sumsq_in is accepted and not read).
 * Each option may be left out (NULL / 0):
 *   norm_w, eps : x is rmsnorm'ed first (clone + rmsnorm, ops/op_misc.hpp:142-181); needs K % 4 == 0
 *   residual    : y += residual (iadd, ops/op_misc.hpp:55-79), fp32 [rows,N_out]
 *   glu == 1    : weiq holds gate and up strips interleaved (strip 2i = gate strip i, 2i+1 = up strip i,
 *                 Ng even) and y[r,n] = silu(gate[r,n]) * up[r,n] (itrans "silu" + imul), N_out = F
 *   glu == 2    : the same two ops on the input side: x is fp32 [rows,2K], a gate|up row (gate in columns
 *                 [0,K), up in [K,2K)), and the FC's input is silu(gate)*up; not with norm_w.  The FC in front
 *                 then runs without glu on the gate and up weights stacked along N.
 *   sumsq_out   : fp32 [rows,Ng], receives the sum of squares of every strip's 32 outputs (after the
 *                 residual add); not with glu == 1
 *   sumsq_in, sumsq_parts : with norm_w: fp32 [rows,sumsq_parts] whose row sums are sum(x^2) -- what the
 *                 FC that produced x left in its sumsq_out -- so that the rmsnorm does not read the row again
 *                 (up to 256 parts; with more the statistic is computed from the row as without sumsq_in)
 * N_out is the number of output columns (Ng*32-ish; Ng/2*32-ish with glu == 1). */
int llmops_fc_Q4A_decode(const float* x, int64_t rows, int64_t K, const int8_t* weiq, int64_t Ng, int64_t Kg,
                         int group_k, int64_t N_out, const float* norm_w, float eps, const float* residual, int glu,
                         const float* sumsq_in, int64_t sumsq_parts, float* sumsq_out, float* y, void* workspace,
                         size_t workspace_bytes, llmops_stream_t stream);

/* llmops_fc_Q4A_decode for more than 8 rows whose result is wanted as out_parts dense matrices, y laid out
 * [out_parts][rows][N_out / out_parts] (Ng % out_parts == 0, N_out == Ng*32): the strips of part p are strips
 * p*Ng/out_parts .. of weiq.  A q|k|v projection over weights stacked along N (chatllama/main.py:347-349 runs three
 * FCs on the same input) thus leaves q, k and v as the three dense [rows, H*S] matrices the attention op takes,
 * with one quantization of the input.  norm_w / eps / glu (0 or 2) as above; no residual, no sums of squares. */
int llmops_fc_Q4A_decode_parts(const float* x, int64_t rows, int64_t K, const int8_t* weiq, int64_t Ng, int64_t Kg,
                               int group_k, int64_t N_out, const float* norm_w, float eps, int glu, int64_t out_parts,
                               float* y, void* workspace, size_t workspace_bytes, llmops_stream_t stream);

/* fc_Q4A (one row, group 128) on the output of llmops_attention_rope_decode_records: the o projection of a decode
 * step (chatllama/main.py:353-355) with the merge of the attention chunks (ops/op_attn.hpp:1012-1025 computes the
 * same softmax-weighted sum in one piece) folded into the FC's input side.  K = H*128 = Kg*128; residual and
 * sumsq_out as in llmops_fc_Q4A_decode. */
int llmops_fc_Q4A_decode_attn(const float* rec_stats, const float* rec_outs, int64_t chunks, int64_t H, const int8_t* weiq,
                              int64_t Ng, int64_t Kg, int64_t N_out, const float* residual, float* sumsq_out, float* y,
                              void* workspace, size_t workspace_bytes, llmops_stream_t stream);

/* The second half of fc_Q4A on its own (ops/op_fc.hpp:318-423): the product for activations that
 * llmops_FC_dynamic_quantize_x has already quantized (xq int8 [rows,Kg*G], xd and gsum fp32
 * [rows,Kg]).  llmops_fc_Q4A == llmops_FC_dynamic_quantize_x into the workspace + this. */
int llmops_fc_Q4A_prequantized(const int8_t* xq, const float* xd, const float* gsum, int64_t rows,
                               const int8_t* weiq, int64_t Ng, int64_t Kg, int group_k, int64_t N, float* y,
                               void* workspace, size_t workspace_bytes, llmops_stream_t stream);

/* The integer core of fc_Q4A on its own (ops/op_fc.hpp:337-363): acc int32 [rows, Ng*32, Kg].
 * `use_mfma` selects which of the production inner loops computes it (0 = dot4 streaming kernel,
 * 1 = int8 MFMA kernel, 2 = the 256-row int8 MFMA kernel with two wave groups in alternating phases,
 * 3 = the weight-streaming int8 MFMA kernel of 3..32 rows; 2 and 3 group 128 only) so that each can be
 * checked bit-for-bit. */
int llmops_fc_Q4A_partials(const int8_t* xq, int64_t rows, const int8_t* weiq, int64_t Ng, int64_t Kg,
                           int group_k, int32_t* acc, int use_mfma, llmops_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Rotary embedding, KV cache, attention
 * ------------------------------------------------------------------------------------------ */

/* rope_embed (ops/op_attn.hpp:44-94, ops/main.cpp:152): in place on x fp32 [B,H,L,S];
 * pairs (i, i+half) for i < half rotated by inv_freq[i]*(position_id+l); dims >= 2*half untouched. */
int llmops_rope_embed(float* x, int64_t B, int64_t H, int64_t L, int64_t S, const float* inv_freq,
                      int64_t half, int position_id, llmops_stream_t stream);

/* workspace bytes for llmops_attention_rope (arrival counters, slot map, split-KV partial results).
 * The first LLMOPS_ATTN_COUNTER_BYTES bytes must be zero when the library first sees the workspace;
 * the library leaves them zero after every call.  One workspace must not be shared by calls that
 * can overlap on the device. */
#define LLMOPS_ATTN_COUNTER_BYTES 65536
size_t llmops_attention_workspace_bytes(int64_t B, int64_t qL, int64_t H, int64_t S, int64_t maxlen);

/* attention_rope2 / attention_rope (ops/op_attn.hpp:721-1029 and :518-718; ops/main.cpp:154-155;
 * same contract).  q,k,v fp32 [B,qL,H*S]; kv_cache [planes,B,H,maxlen,S] in fp32
 * (LLMOPS_CACHE_F32, the reference's layout) or fp16 (LLMOPS_CACHE_F16, an extension: fp32 math
 * on fp16-rounded K/V); slots int32 [qL] (device).  Effects: q,k rotated in place (k stays
 * rotated), k,v rows written to cache[2*layer_id+{0,1}, b, h, slots[p], :], and q overwritten by
 * softmax((q.K^T)/sqrt(S) with in-chunk causal mask via slots) . V over
 * kvLen = min(position_id+qL, maxlen) cache rows.  One query token (qL == 1, the decode form) and 32 or more
 * (the tiled prompt kernel, S == 128) need maxlen*S*sizeof(cache element) < 4 GiB (LLMOPS_EINVAL otherwise); more
 * than 65535 heads in all (B*H) with one query token are served by the general kernels (three launches instead
 * of two).  Arithmetic: fp32 throughout, except that the tiled prompt kernel multiplies on the fp16 matrix cores
 * with every fp32 operand carried as two fp16 halves (22 bits, fp32 accumulation): its results agree with fp32
 * evaluation to about 1e-6 of the largest output (tests assert 1e-5; the contract is 1e-3), and q, k, v and cache
 * values must lie inside the fp16 range (|x| < 65504) there. */
int llmops_attention_rope(float* q, float* k, const float* v, int64_t B, int64_t qL, int64_t H, int64_t S,
                          const float* inv_freq, int64_t half, void* kv_cache, int cache_dtype,
                          int64_t planes, int64_t maxlen, const int32_t* slots, int position_id,
                          int layer_id, void* workspace, size_t workspace_bytes, llmops_stream_t stream);

/* attention_rope2 (ops/op_attn.hpp:721-1029) for one query token per sequence (qL = 1) with the token's position
 * in device memory: `slot` and `position_id` are int32 [1] on the device and are read by the kernels, so a HIP
 * graph that captured the call can be replayed for every following token after the two values have been
 * updated (the reference passes position_id by value, chatllama/main.py:353).  kvLen = min(position_id + 1,
 * maxlen).  The launch is sized for a full cache.  Needs half % 4 == 0.  Otherwise as llmops_attention_rope. */
int llmops_attention_rope_decode(float* q, float* k, const float* v, int64_t B, int64_t H, int64_t S,
                                 const float* inv_freq, int64_t half, void* kv_cache, int cache_dtype, int64_t planes,
                                 int64_t maxlen, const int32_t* slot, const int32_t* position_id, int layer_id,
                                 void* workspace, size_t workspace_bytes, llmops_stream_t stream);

/* attention_rope2 for one query token (B sequences of one token) that leaves the merge of its split-KV chunks to
 * the consumer: instead of overwriting q with softmax(qK^T)V (ops/op_attn.hpp:1012-1025) it writes, per head,
 * up to 8 chunk records -- rec_stats fp32 [B*H][8][2] (max score, sum of exp) and rec_outs fp32 [B*H][8][128]
 * (sum of exp-weighted V rows) -- which llmops_fc_Q4A_decode_attn merges while it loads its input.  q is left as
 * it came in; k is rotated in place and the cache updated as usual.  The position is `position_id`, or, when
 * position_id_dev is not NULL, the int32 it points at in device memory.  llmops_attention_records_chunks returns 8
 * when a cache of `maxlen` rows can be served this way (fp32: up to 2048 rows, fp16: up to 4096), else 0. */
int64_t llmops_attention_records_chunks(int64_t maxlen, int cache_dtype);
/* cache rows that one chunk record of llmops_attention_rope_decode_records covers for a cache of `maxlen` rows (0: such
 * a cache cannot be served this way).  A call at kv length L writes ceil(L / rows) records per head -- with the
 * position in device memory ceil(maxlen / rows), empty ones (sum 0) beyond the current length included -- and that
 * count is the `chunks` argument of llmops_fc_Q4A_decode_attn. */
int64_t llmops_attention_records_chunk_rows(int64_t maxlen, int cache_dtype);
int llmops_attention_rope_decode_records(float* q, float* k, const float* v, int64_t B, int64_t H, int64_t S,
                                         const float* inv_freq, int64_t half, void* kv_cache, int cache_dtype,
                                         int64_t planes, int64_t maxlen, const int32_t* slot, int position_id,
                                         const int32_t* position_id_dev, int layer_id, float* rec_stats, float* rec_outs,
                                         void* workspace, size_t workspace_bytes, llmops_stream_t stream);

/* softmax (ops/op_misc.hpp:183-194, ops/utils.hpp:484-490): in place over rows of length K */
int llmops_softmax(float* x, int64_t rows, int64_t K, llmops_stream_t stream);

/* mm_qk, mm_qk42, mm_qk81, mm_qk24 (ops/op_attn.hpp:149-193, 195-298, 300-422, 424-515; bound at
 * ops/main.cpp:163-166): the reference's four benchmark variants of one product,
 *   attn_w[b,h,pq,pk] = dot(q[b,h,pq,:], kcache[b,h,pk,:]) / sqrt(S),   pk < kvLen <= kv_max.
 * q is addressed as q + b*q_stride_b + h*q_stride_h + pq*q_stride_q (elements, multiples of 4):
 * [B,qL,H*S] for mm_qk/81/24 -> (qL*H*S, S, H*S); [B,H,qL,S] for mm_qk42 -> (H*qL*S, qL*S, S).
 * kcache fp32 [B,H,kv_max,S]; attn_w fp32 [B,H,qL,kvLen] dense; S % 8 == 0 (ops/op_attn.hpp:205). */
int llmops_mm_qk(const float* q, int64_t q_stride_b, int64_t q_stride_h, int64_t q_stride_q, const float* kcache,
                 int64_t kv_max, float* attn_w, int64_t B, int64_t H, int64_t qL, int64_t kvLen, int64_t S,
                 llmops_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Neighbours needed for one decode step (ops/op_misc.hpp, ops/op_embedding.hpp)
 * ------------------------------------------------------------------------------------------ */

/* rmsnorm (ops/op_misc.hpp:142-181): x[r,:] *= rsqrt(mean(x[r,:]^2)+eps) * w, in place */
int llmops_rmsnorm(float* x, int64_t rows, int64_t hidden, const float* w, float eps, llmops_stream_t stream);
/* clone + rmsnorm (chatllama/main.py:345-346) in one launch: out = rmsnorm(x), x untouched */
int llmops_rmsnorm_out(const float* x, float* out, int64_t rows, int64_t hidden, const float* w, float eps,
                       llmops_stream_t stream);
/* itrans(gate,"silu") + imul(up,gate) (chatllama/main.py:363-367) on a row that holds gate and up
 * side by side: out[r,i] = silu(gate_up[r,i]) * gate_up[r,F+i] */
int llmops_silu_mul(const float* gate_up, float* out, int64_t rows, int64_t F, llmops_stream_t stream);
/* the same two ops on a row whose strips of 32 columns alternate gate, up, gate, up ... (what an FC over interleaved
 * gate/up strips leaves): out[r,i] = silu(gate_up[r,(i/32)*64 + i%32]) * gate_up[r,(i/32)*64 + 32 + i%32]; F % 32 == 0 */
int llmops_silu_mul_interleaved(const float* gate_up, float* out, int64_t rows, int64_t F, llmops_stream_t stream);
/* sum of squares of every strip of 32 columns of y fp32 [rows,N] -> out fp32 [rows, ceil(N/32)]: the partial sums of
 * the rmsnorm statistic (ops/op_misc.hpp:158-166) in the form llmops_fc_Q4A_decode's sumsq_out / sumsq_in exchange,
 * for more rows than that entry takes */
int llmops_strip_sumsq(const float* y, int64_t rows, int64_t N, float* out, llmops_stream_t stream);
/* iadd / imul (ops/op_misc.hpp:55-107): a (+|*)= b; b is [rows,inner] or, if b_is_row, [inner] */
int llmops_iadd(float* a, const float* b, int64_t rows, int64_t inner, int b_is_row, llmops_stream_t stream);
int llmops_imul(float* a, const float* b, int64_t rows, int64_t inner, int b_is_row, llmops_stream_t stream);
/* itrans "silu" (ops/op_misc.hpp:127-138): a = a * sigmoid(a), in place */
int llmops_itrans_silu(float* a, int64_t n, llmops_stream_t stream);
/* embedding_q8c_quant_w (ops/op_embedding.hpp:51-78): w fp32 [V,E] -> q int8 [V,E], scales [V] */
int llmops_embedding_q8c_quant_w(const float* w, int64_t V, int64_t E, int8_t* q, float* scales, llmops_stream_t stream);
/* embedding_q8c (ops/op_embedding.hpp:108-137): out[i,:] = scales[ids[i]] * q[ids[i],:]; ids int64 */
int llmops_embedding_q8c(float* out, const int64_t* ids, int64_t n, const int8_t* q, const float* scales,
                         int64_t V, int64_t E, llmops_stream_t stream);
/* embedding (ops/op_embedding.hpp:24-49): out[i,:] = w[ids[i],:]; ids int64 */
int llmops_embedding(float* out, const int64_t* ids, int64_t n, const float* w, int64_t V, int64_t E, llmops_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* LLMOPS_HIP_H */
