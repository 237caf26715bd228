// Internal launchers shared with the decode-step driver.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace feather {

// As feather_paged_attn_fp8, but the result can be written (any subset) as fp32 (out_f32), as
// packed FP8 words of the same mode (out_packed, [n_seq, n_q_heads * d / 4]) and as fp16 holding
// the values of those codes (out_q16, [n_seq, n_q_heads * d]): the operand of the next GEMV in
// its two accepted forms.  Arguments are assumed validated.
int paged_attn_launch(const void *q, const void *k_cache, const void *v_cache, const void *block_tables,
                      const void *ctx_lens, float *out_f32, uint32_t *out_packed, _Float16 *out_q16, void *scratch, int64_t n_seq,
                      int64_t n_q_heads, int64_t n_kv_heads, int64_t d, int64_t block_size, int64_t max_blocks,
                      int64_t n_blocks, int64_t max_ctx, int mode, float scale, hipStream_t stream);

// The decode step's attention with the rotary embedding, the query packing and the append of the new
// token's K / V row fused into its prologue (see paged_attn_split_kernel, FUSED).  `plan` and `cs` are
// written once per step by the step's prologue kernel; plan entries are 4 + 512 / block_size ints:
// {sequence or -1, split, tokens of the sequence including an appended new one, owner flag, block ids of
// the split}, one per (sequence, split) item in launch order.  ctx_after [n_seq] is what the merge reads.
bool paged_attn_fused_supported(int64_t n_seq, int64_t n_q_heads, int64_t n_kv_heads, int64_t d, int64_t block_size,
                                int64_t n_part);
int64_t paged_attn_plan_ints(int64_t n_seq, int64_t block_size, int64_t max_ctx);
int paged_attn_fused_launch(const int32_t *plan, const int32_t *ctx_after, void *k_cache, void *v_cache, const float *qkv,
                            int n_part, int64_t part_stride, const float *cs, uint32_t *out_packed, void *scratch,
                            int64_t n_seq, int64_t n_q_heads, int64_t n_kv_heads, int64_t block_size, int64_t max_blocks,
                            int64_t n_blocks, int64_t max_ctx, int mode, float scale, hipStream_t stream);

// Batched GEMV with the K range cut into `splits` slices: slice s writes its partial sums to
// out_f32 + s * part_stride ([nvec, M] each); the consumer adds the slices in index order.
// Needs K % 256 == 0 and 16-byte aligned w and x; splits is clamped to K / 256.  Returns the
// number of slices actually written through *splits_out.
int gemv_batched_launch(const void *w, const void *x, float *out_f32, int64_t M, int64_t K, int64_t nvec, int mode,
                        int splits, int64_t part_stride, int *splits_out, hipStream_t stream);

// As gemv_batched_launch for w = [gate rows; up rows] ([2 * inter, K]) with the SwiGLU activation
// and the FP8 quantisation fused: act_packed [nvec, inter / 4] words.  Needs K % 256 == 0,
// inter % 4 == 0, 16-byte aligned w and x.  act_f32 (optional, [nvec, inter]) receives the fp32 values the
// codes were rounded from.
int gemv_batched_swiglu_launch(const void *w, const void *x, uint32_t *act_packed, float *act_f32, int64_t inter,
                               int64_t K, int64_t nvec, int mode, hipStream_t stream);

}  // namespace feather
