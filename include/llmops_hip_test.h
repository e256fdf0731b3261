/* llmops_hip_test.h -- hooks for tests and benchmarks of libllmops_hip.so.
 *
 * None of these has a counterpart in the reference and none is part of the product ABI
 * (include/llmops_hip.h): they change process-wide planner state or run measurement kernels, so a
 * program that serves requests must not call them -- and cannot by accident: every hook is refused
 * (LLMOPS_EINVAL; the setters do nothing and say so once on stderr) unless the process was started with
 * the environment variable LLMOPS_TEST_HOOKS=1, which the tests and bench.py set.  Tests flip a knob, run one op, and restore the
 * default in a finally block; bench.py uses the read/copy kernels for the measured HBM ceiling and
 * to calibrate the traffic counters.
 */
#ifndef LLMOPS_HIP_TEST_H
#define LLMOPS_HIP_TEST_H

#include "llmops_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------------------------------
 * Measurement helpers (used by bench.py and the profiles)
 * ------------------------------------------------------------------------------------------ */

/* read / copy `bytes` (multiple of 16) with `workgroups` workgroups of 256 threads streaming
 * contiguous slabs: the machine's measured HBM ceiling and the calibration of traffic counters */
int llmops_test_calib_read(const void* src, int64_t bytes, int workgroups, void* out4, llmops_stream_t stream);
int llmops_test_calib_copy(const void* src, void* dst, int64_t bytes, int workgroups, llmops_stream_t stream);

/* split-K planner knobs of the streaming FC kernel: number of workgroups to aim for and
 * wavefronts per workgroup (4, 8, 16; 0 = default).  Values <= 0 / < 0 leave a knob unchanged.
 * target_workgroups == -2 / -3 instead selects how two k-splits of a strip meet: through one 64-bit
 * exchange per output (default) / through the arrival ticket like larger split counts. */
void llmops_test_fc_set_tuning(int target_workgroups, int waves_per_workgroup);

/* prefill GEMM planner knob: force the row-tile factor of the LDS-tiled MFMA kernel (1, 2 or 4:
 * 32, 64 or 128 rows per workgroup; 8: the 256-row kernel whose two wave groups alternate between
 * MFMA and fold phases, which the planner takes from 512 rows on); 0 = choose per shape; -1 = choose
 * per shape and send 9..16 rows to the tiled kernel too instead of the weight-streaming MFMA kernel */
void llmops_test_gemm_set_tuning(int row_tile_factor);

/* prefill GEMM with split-K: the product kernel adds the partial sums itself (the last split of a tile to
 * arrive adds all of them in index order) when the split count is at most 12 x in_kernel; otherwise, and
 * always with 0, a second launch adds them.  Default 1.  Same result either way; kept for comparisons and tests. */
void llmops_test_gemm_set_reduce(int in_kernel);

/* prefill GEMM: force the split-K factor (clamped to the number of k-groups); 0 = choose per shape.  Together
 * with a forced row-tile factor it pins the tiling, so that the two ways of adding the partial sums can be
 * compared bit for bit. */
void llmops_test_gemm_set_split(int splits);

/* prefill GEMM: what the planner chooses for a product of `rows` rows with a packed tensor of Ng strips x Kg
 * k-groups (host arithmetic only, no launch): the row-tile factor (1, 2, 4: 32, 64, 128 rows per workgroup of
 * the four-wave kernel; 8: the 256-row kernel) and the split-K factor.  Reads the knobs above. */
int llmops_test_gemm_plan(int64_t rows, int64_t Ng, int64_t Kg, int group_k, int* row_tile_factor, int* splits);

/* weight-streaming MFMA kernel (3..16 rows, 17..32 for tensors of fewer than 256 strips): two workgroups per strip with half of K each for tensors of
 * fewer than 256 strips (default on; 0 switches it off, for comparisons and tests) */
void llmops_test_fc_rows_set_split(int on);

/* llmops_fc_Q4A with 2..8 rows, group 128: from how many rows the weight-streaming MFMA kernel (separate
 * quantization launch) replaces the streaming kernel that quantizes on the fly, for tensors of up to
 * 256 strips and for larger ones (defaults 4 and 3; values below 2 restore them) */
void llmops_test_fc_set_row_routing(int rows_from_small, int rows_from_large);

/* decode attention (one query token): force the cache rows per wavefront (fp32 cache 4, 8, 16; fp16 cache 8, 16,
 * 32; a chunk is 4 times that); 0 = choose */
void llmops_test_attn_set_decode_plan(int rows_per_wave);

/* The decode kernel of llmops_fc_Q4A (rows <= 8, the one that quantizes the activations on the fly) in its
 * dump build: y as llmops_fc_Q4A computes it, plus what the kernel itself quantized -- xq int8 [rows,Kg*G],
 * xd and gsum fp32 [rows,Kg] (FC_dynamic_quantize_x, ops/op_fc.hpp:221-272; gsum is a tree sum here) -- and
 * its int32 dot products acc [rows,Ng*32,Kg] (ops/op_fc.hpp:337-363), so that the production loop can be
 * compared bit for bit.  Every workgroup stores the activations it quantized (they must all agree). */
int llmops_test_fc_decode_dump(const float* x, int64_t rows, int64_t K, const int8_t* weiq, int64_t Ng, int64_t Kg,
                               int group_k, int64_t N, float* y, int8_t* xq, float* xd, float* gsum, int32_t* acc,
                               void* workspace, size_t workspace_bytes, llmops_stream_t stream);

/* llmops_fc_Q4A_decode_attn in the same dump build: the codes and scales of the attention output the kernel merged
 * from the chunk records, and its int32 sums */
int llmops_test_fc_decode_attn_dump(const float* rec_stats, const float* rec_outs, int64_t chunks, int64_t H,
                                    const int8_t* weiq, int64_t Ng, int64_t Kg, int64_t N_out, float* y, int8_t* xq, float* xd,
                                    float* gsum, int32_t* acc, void* workspace, size_t workspace_bytes, llmops_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* LLMOPS_HIP_TEST_H */
