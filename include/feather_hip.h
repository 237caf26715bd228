/*
 * feather_hip.h -- C ABI of libfeather_hip.so: hand-written gfx950 (MI355X)
 * kernels for the packed-low-precision routines of SuriyaaMM/feather.
 *
 * Conventions
 *   - Every pointer is a DEVICE pointer unless the name says host.  The library
 *     never allocates, frees or synchronises; outputs and scratch are caller
 *     owned.  Kernels are enqueued on `stream` (a hipStream_t passed as void*,
 *     NULL = the default stream) and the call returns at once.
 *   - Return value: FEATHER_OK (0) or a negative FEATHER_E* code; a message for
 *     the last failure on the calling thread is available from
 *     feather_last_error().
 *   - Packed layout (reference feather/packers/fp8.py:134, fp16.py:39): element
 *     4j+i of the flattened source is byte i (bits [8i, 8i+8)) of 32-bit word
 *     j; two fp16 values per word with the first in the low half.
 *   - `mode`: FEATHER_E5M2 / FEATHER_E4M3.  Decode inside the compute kernels
 *     follows the reference kernels: E5M2 code c -> fp16 bits c << 8
 *     (feather/routines/gemv.py:31-58); E4M3 -> sign | (e ? e + 8 : 0) << 10 |
 *     m << 7 (feather/routines/gemv.py:83-88).
 *
 * Each entry point cites the reference interface it replaces (paths relative
 * to the reference checkout).
 */
#ifndef FEATHER_HIP_H
#define FEATHER_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FEATHER_OK 0
#define FEATHER_EINVAL (-1)       /* null / misaligned pointer, negative size, bad flag */
#define FEATHER_EMODE (-2)        /* unknown mode (reference: NotImplementedError, fp8.py:114) */
#define FEATHER_ESHAPE (-3)       /* shape the kernels do not support (K % 4, head dim, ...) */
#define FEATHER_ELAUNCH (-4)      /* hipGetLastError() after a launch */

#define FEATHER_E5M2 0
#define FEATHER_E4M3 1

#define FEATHER_ROUND_RNE 0       /* pack_fp8_tensor (round to nearest even) */
#define FEATHER_ROUND_TRUNC 1     /* *_legacy packers (E5M2 only, drop the low byte) */

#define FEATHER_SEM_KERNEL 0      /* decode of the GPU kernels (gemv.py:83-88) */
#define FEATHER_SEM_IEEE 1        /* decode of the CPU unpack_* API (fp8.py:381-391) */

#define FEATHER_OUT_F32 0
#define FEATHER_OUT_F16 1

#define FEATHER_TAIL_MASK 0       /* keys past seq_len are excluded from the softmax */
#define FEATHER_TAIL_REFERENCE 1  /* keys past seq_len in the last 64-key tile count as zero rows
                                     (attention.py:57-59) */

/* Library version (major * 10000 + minor * 100 + patch); FEATHER_HIP_VERSION is the version of this header.
 * A change of any signature or struct below raises the minor number: a binding must refuse a library whose
 * feather_version() differs from the header it was written against in major or minor. */
#define FEATHER_HIP_VERSION 10400
int feather_version(void);

/* Message for the last non-zero return code on this thread ("" if none). */
const char *feather_last_error(void);

/* fp16[n] -> u32[ceil(n/4)], four FP8 codes per word, tail padded with +0.
 * Replaces pack_fp8_tensor / pack_fp8_ndarray / pack_fp8_into_fp32
 * (feather/packers/fp8.py:260-281, :178-210, :69-136) with rounding = RNE, and
 * the *_legacy packers (:8-66, :139-175, :213-257) with rounding = TRUNC.
 * src must be 2-byte aligned, dst 4-byte aligned. */
int feather_pack_fp8(const void *src_f16, void *dst_u32, int64_t n, int mode, int rounding, void *stream);

/* fp32[n] -> u32[ceil(n/4)]: each value rounded fp32 -> fp16 -> FP8 (round to nearest even twice,
 * i.e. pack_fp8_tensor applied to x.half()), tail padded with +0.  No reference counterpart: the
 * reference packs on the CPU from fp16 (feather/packers/fp8.py:260-281); this is the rounding chain
 * every fp32 producer that feeds a packed GEMV uses (the norm, SwiGLU, rotary and attention
 * epilogues below), as an operation of its own. */
int feather_quant_pack_f32(const void *src_f32, void *dst_u32, int64_t n, int mode, void *stream);

/* u32[n_words] -> fp32 or fp16 [4 * n_words] in element order.
 * Replaces unpack_fp8_from_fp32 / unpack_into_fp8_ndarray
 * (feather/packers/fp8.py:336-392, :395-432) with semantics = IEEE, the legacy
 * unpack (:284-333) and the kernels' in-register decode with semantics =
 * KERNEL.  relu != 0 applies max(0, x) (relu1d_fp8_ret_fp32_feather_gpu,
 * feather/routines/activations.py:9-42). */
int feather_unpack_fp8(const void *src_u32, void *dst, int64_t n_words, int mode, int semantics, int out_dtype,
                       int relu, void *stream);

/* fp16[n] -> u32[ceil(n/2)] (first element in the low half, odd tail + 0) and
 * back.  Replaces pack_fp16_ndarray / pack_fp16_into_fp32 and
 * unpack_into_fp16_ndarray / unpack_fp32_into_fp16
 * (feather/packers/fp16.py:83-116, :8-43, :119-151, :46-80). */
int feather_pack_fp16(const void *src_f16, void *dst_u32, int64_t n, void *stream);
int feather_unpack_fp16(const void *src_u32, void *dst_f16, int64_t n_words, void *stream);

/* out[r] = sum_k dec(m[r, k]) * dec(v[k]), fp32 accumulate, fp32 out[M].
 * m: M*K/4 words row-major, v: K/4 words; K % 4 == 0; m, v 4-byte aligned
 * (16-byte aligned rows take the fast path).
 * Replaces gemv_fp8_e5m2_acc_fp32_gpu / gemv_fp8_e4m3_acc_fp32_gpu
 * (feather/routines/gemv.py:136-184, :187-235). */
int feather_gemv_fp8(const void *m, const void *v, void *out_f32, int64_t M, int64_t K, int mode, void *stream);

/* out[b, r] = sum_k dec(w[r, k]) * dec(x[b, k]) for b < nvec (1 <= nvec <= 64):
 * the weight matrix is streamed once for all vectors.  No reference
 * counterpart (the reference runs one vector per launch, gemv.py:179-183);
 * used by the batched decode step. */
int feather_gemv_fp8_batched(const void *w, const void *x, void *out_f32, int64_t M, int64_t K, int64_t nvec, int mode,
                             void *stream);

/* act[b, i] = silu(g) * u with g = sum_k dec(w[i, k]) dec(x[b, k]), u = sum_k dec(w[inter + i, k]) dec(x[b, k]),
 * written as packed FP8 words act_packed [nvec, inter / 4] (fp32 -> fp16 -> FP8 as feather_quant_pack_f32)
 * and, if act_f32 is not NULL, also as the fp32 values [nvec, inter] the codes were rounded from.
 * w_gate_up is [2 * inter, K] packed: gate rows, then up rows.  silu(g) = g / (1 + 2^(-g log2 e)) with the
 * hardware exp2 and reciprocal.  K % 256 == 0, inter % 4 == 0, 1 <= nvec <= 64, 16-byte aligned w and x.
 * No reference counterpart (quantise + pack fused into the producing GEMV). */
int feather_gemv_fp8_batched_swiglu(const void *w_gate_up, const void *x, void *act_packed, void *act_f32, int64_t inter,
                                    int64_t K, int64_t nvec, int mode, void *stream);

/* Bytes of scratch feather_dot_* need (one buffer per stream in flight; 64-byte
 * aligned; contents need no initialisation). */
int64_t feather_dot_scratch_bytes(void);

/* out[0] = sum_k dec(x1[k]) * dec(x2[k]) over n_words packed words, fp32.
 * Deterministic: per-workgroup partials are combined in a fixed order by a
 * second small kernel (the reference adds them with fp32 atomics).
 * Replaces dot_fp8_e5m2_acc_fp32_gpu (feather/routines/dot.py:220-260); mode
 * E4M3 has no reference kernel and uses the GEMV decode. */
int feather_dot_fp8(const void *x1, const void *x2, void *out_f32, void *scratch, int64_t n_words, int mode,
                    void *stream);

/* FP16-packed dot, summed in fp32.  fp16_products != 0: per word
 * fp16(lo1*lo2) +fp16 fp16(hi1*hi2) as in the reference GPU kernel
 * (dot_fp16_acc_fp32_gpu, feather/routines/dot.py:194-218, :134-141);
 * fp16_products == 0: exact fp32 products as in the reference's CPU variants
 * (dot_fp16_acc_fp32_vec / _numba, feather/routines/dot.py:9-50, :53-106). */
int feather_dot_fp16(const void *x1, const void *x2, void *out_f32, void *scratch, int64_t n_words, int fp16_products,
                     void *stream);

/* Non-causal attention forward on packed Q/K/V of fixed length: for each of n_heads
 * independent heads, out[h] = softmax(Q K^T * scale) V, Q/K/V [L, d/4] words,
 * out [L, d] fp32; scores fp32, P rounded to fp16 before P.V, fp32 output.
 * d in {32, 64, 128, 256, 512}; any other head dim returns FEATHER_ESHAPE (the reference kernel takes
 * power-of-two d >= 64, attention.py:28-41, :145: its tl.dot needs d / 4 >= 16).  kv_group > 1 maps query head h to K/V head
 * h / kv_group (K/V then hold n_heads / kv_group heads).  scale must be positive.
 * Replaces flash_attention_fp8_e5m2_acc_fp32_gpu
 * (feather/routines/attention.py:110-179) at n_heads = 1, mode = E5M2,
 * scale = 1/sqrt(d), tail = REFERENCE. */
int feather_flash_attn_fp8(const void *q, const void *k, const void *v, void *out_f32, int64_t n_heads, int64_t L,
                           int64_t d, int64_t kv_group, int mode, float scale, int tail, void *stream);

/* The same attention with an optional device workspace.  One head, or a few short wide heads, make a grid that leaves
 * most of the 256 CUs idle (the reference function is one head, attention.py:110-179: 8192 rows at d = 64 are 32
 * workgroups here; 8 heads x 1024 rows at d = 512 are 128).  With a workspace of
 * feather_flash_attn_workspace_bytes(n_heads, L, d) bytes (0: the shape does not profit; d >= 64) the key loop of every
 * query tile is cut into 2, 4 or 8 ranges that run as separate workgroups, and a second small kernel combines them
 * (same result up to the rounding of P against another reference point and of the fp32 additions; identical from call
 * to call).  workspace == NULL, or a workspace smaller than asked for, runs fewer ranges or the plain kernel; nothing
 * is kept in the workspace between calls, and calls that share a workspace must not overlap.  No reference counterpart
 * (the reference launches one program per 64 queries of one head, attention.py:172-179). */
int64_t feather_flash_attn_workspace_bytes(int64_t n_heads, int64_t L, int64_t d);
int feather_flash_attn_fp8_ws(const void *q, const void *k, const void *v, void *out_f32, void *workspace,
                              int64_t workspace_bytes, int64_t n_heads, int64_t L, int64_t d, int64_t kv_group, int mode,
                              float scale, int tail, void *stream);

/* Attention forward on packed variable-length sequences, optionally causal.  No reference
 * counterpart (the reference kernel, feather/routines/attention.py:14-108, is one
 * fixed-length non-causal head); numerics as feather_flash_attn_fp8 with the exact tail.
 *   q            [n_heads, total_rows, d/4] words; k, v [n_heads / kv_group, total_rows, d/4]
 *   cu_seqlens   [n_seq + 1] int32 on the device, non-decreasing row offsets: sequence s is
 *                rows cu[s] .. cu[s+1]-1 of every head and attends only to itself
 *   max_seqlen   upper bound of cu[s+1] - cu[s]: it sizes the grid, so rows of a sequence beyond its first
 *                max_seqlen rows are NOT computed and keep whatever `out` held (the caller must pass a
 *                true bound; the kernel cannot report a longer sequence)
 *   out          [n_heads, total_rows, d] fp32; rows outside every sequence are left untouched
 *   causal       1: query i of a sequence sees keys 0..i of that sequence
 * A fixed-length batch is n_seq = 1, cu = {0, L}, n_heads = batch * heads. */
int feather_flash_attn_fp8_varlen(const void *q, const void *k, const void *v, void *out_f32, const void *cu_seqlens,
                                  int64_t n_seq, int64_t max_seqlen, int64_t total_rows, int64_t n_heads, int64_t d,
                                  int64_t kv_group, int mode, float scale, int causal, void *stream);

/* Scatter the K and V rows of packed variable-length sequences (the layout of
 * feather_flash_attn_fp8_varlen) into a paged cache.  No reference counterpart.
 *   k_src, v_src  src_f16 = 0: packed words [n_kv_heads, total_rows, d/4];
 *                 src_f16 = 1: fp16 [n_kv_heads, total_rows, d], encoded to `mode` on the way
 *                 (round to nearest even, as feather_pack_fp8)
 *   k_cache       [n_blocks, n_kv_heads, block_size, d/4] words (v_cache same)
 *   block_tables  [n_seq, max_blocks] int32; cu_seqlens [n_seq + 1] int32
 *   start_pos     [n_seq] int32 or NULL (all 0): cache position of each sequence's first row
 * Row cu[s] + i goes to position start_pos[s] + i of sequence s.  Positions below 0 or at or beyond
 * max_blocks * block_size have no table entry and are dropped, and so are rows whose table entry
 * is not a block of the cache (outside [0, n_blocks): padding, -1).  d % 16 == 0. */
int feather_paged_cache_write(const void *k_src, const void *v_src, int src_f16, void *k_cache, void *v_cache,
                              const void *block_tables, const void *cu_seqlens, const void *start_pos, int64_t n_seq,
                              int64_t total_rows, int64_t n_kv_heads, int64_t d, int64_t block_size, int64_t max_blocks,
                              int64_t n_blocks, int mode, void *stream);

/* Bytes of scratch feather_paged_attn_fp8 needs for the given problem. */
int64_t feather_paged_attn_scratch_bytes(int64_t n_seq, int64_t n_q_heads, int64_t d, int64_t max_ctx);

/* Single-query (decode) attention over a paged FP8 KV cache.  No reference
 * counterpart.
 *   q            [n_seq, n_q_heads, d/4] words
 *   k_cache      [n_blocks, n_kv_heads, block_size, d/4] words (v_cache same)
 *   block_tables [n_seq, max_blocks] int32, ctx_lens [n_seq] int32
 *   out_f32      [n_seq, n_q_heads, d] fp32, and / or
 *   out_packed   [n_seq, n_q_heads * d / 4] words: the same result rounded fp32 -> fp16 -> FP8 of `mode`
 *                (as feather_quant_pack_f32), the packed operand of a following GEMV; either may be NULL
 * d in {64, 128, 256, 512} (any other head dim returns FEATHER_ESHAPE); at most 16 query heads per KV head.
 * Query head h uses KV head h / (n_q_heads / n_kv_heads).  Table entries of positions below
 * ctx_lens[s] must be blocks of the cache; an entry outside [0, n_blocks) is read as the last block
 * (a wrong result for that sequence, never an access outside the cache).  Entries past the context
 * are not used.  Negative context lengths count as 0 (a zero result). */
int feather_paged_attn_fp8(const void *q, const void *k_cache, const void *v_cache, const void *block_tables,
                           const void *ctx_lens, void *out_f32, void *out_packed, void *scratch, int64_t n_seq,
                           int64_t n_q_heads, int64_t n_kv_heads, int64_t d, int64_t block_size, int64_t max_blocks,
                           int64_t n_blocks, int64_t max_ctx, int mode, float scale, void *stream);

/* feather_paged_attn_fp8 for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): no counterpart in the reference.
 * Same arguments without `scratch`: the split partials go to a buffer of
 * FEATHER_PAGED_ATTN_STATIC_SCRATCH_BYTES that is part of the library's device image (every GPU the
 * library runs on holds it until the process ends).  A problem whose
 * feather_paged_attn_scratch_bytes() exceeds that size is rejected with FEATHER_ESHAPE.  The call
 * allocates and frees nothing.  All calls on one GPU share the buffer: calls that overlap on one
 * GPU (different streams, or threads) race; calls on one stream are ordered and safe.  Nothing in
 * the buffer needs clearing between calls.  Results are bit-identical to feather_paged_attn_fp8.
 * The first call on a device looks up the buffer's device address (hipGetSymbolAddress: no allocation, no stream
 * work, but it may load the code object): make that call before a stream capture begins; later calls only
 * enqueue kernels and can be captured. */
#define FEATHER_PAGED_ATTN_STATIC_SCRATCH_BYTES (4 << 20)
int feather_paged_attn_fp8_static(const void *q, const void *k_cache, const void *v_cache, const void *block_tables,
                                  const void *ctx_lens, void *out_f32, void *out_packed, int64_t n_seq,
                                  int64_t n_q_heads, int64_t n_kv_heads, int64_t d, int64_t block_size,
                                  int64_t max_blocks, int64_t n_blocks, int64_t max_ctx, int mode, float scale,
                                  void *stream);

/* ---- decode step of a Llama-shaped model on packed weights (no reference counterpart) ----
 *
 * The reference has no model code; this entry point runs one token step for a batch with
 * every linear layer as a packed-FP8 batched GEMV (decode as feather_gemv_fp8) and attention
 * over the paged FP8 cache (feather_paged_attn_fp8).  Activations that feed a GEMV are
 * rounded fp32 -> fp16 -> FP8 (round to nearest even, as pack_fp8_tensor) in the producing
 * kernel.  Per layer: RMSNorm, fused QKV projection, rotary embedding (rotate-half
 * convention), append of the new K/V to the cache at position ctx_lens[b], attention over
 * ctx_lens[b] + 1 tokens, output projection, residual, RMSNorm, gate/up projection,
 * silu(gate) * up, down projection, residual; then the final norm and the lm_head GEMV.
 * The structs live in HOST memory; every pointer inside them is a device pointer. */
typedef struct feather_decoder_layer {
    const void *w_qkv;      /* [(n_q_heads + 2 n_kv_heads) * head_dim, hidden] packed: q rows, k rows, v rows */
    const void *w_o;        /* [hidden, n_q_heads * head_dim] packed */
    const void *w_gate_up;  /* [2 * inter, hidden] packed: gate rows, then up rows */
    const void *w_down;     /* [hidden, inter] packed */
    const float *norm_attn; /* [hidden] fp32 RMSNorm weight before attention */
    const float *norm_mlp;  /* [hidden] fp32 RMSNorm weight before the MLP */
    void *k_cache;          /* [n_blocks, n_kv_heads, block_size, head_dim / 4] packed words, written by the step */
    void *v_cache;          /* same shape */
} feather_decoder_layer_t;

typedef struct feather_decoder {
    int32_t n_layers, hidden, n_q_heads, n_kv_heads, head_dim, inter, vocab;
    int32_t block_size, max_blocks; /* KV paging: block_tables is [batch, max_blocks] */
    int32_t n_blocks;               /* blocks in every layer's k_cache / v_cache */
    int32_t mode;                   /* FEATHER_E5M2 / FEATHER_E4M3 for weights, activations and cache */
    float rms_eps, rope_theta;
    const feather_decoder_layer_t *layers; /* host array of n_layers entries */
    const void *embed_f16;                 /* [vocab, hidden] fp16 embedding table */
    const float *norm_final;               /* [hidden] */
    const void *w_lm_head;                 /* [vocab, hidden] packed */
} feather_decoder_t;

/* Bytes of scratch feather_decode_step needs (256-byte aligned buffer); -1 for a bad configuration. */
int64_t feather_decode_step_scratch_bytes(const feather_decoder_t *dec, int64_t batch, int64_t max_ctx);

/* Which attention path feather_decode_step takes for this configuration: 1 = the attention kernel with the
 * rotary embedding, query packing and K/V append in its prologue (head_dim 64, power-of-two block_size >= 4,
 * batch <= 64: the new token is scored from registers after the cached ones), 0 = separate rotary / append kernel
 * followed by feather_paged_attn_fp8 (the new token is read back from the cache in position order), -1 = bad
 * configuration.  The two differ in the order of the softmax's additions only.  No reference counterpart. */
int feather_decode_step_attention_path(const feather_decoder_t *dec, int64_t batch, int64_t max_ctx);

/* token_ids [batch] int32, block_tables [batch, max_blocks] int32, ctx_lens [batch] int32 (tokens
 * already in the cache; the caller adds 1 after the step), logits [batch, vocab] fp32.
 * batch <= 64; max_ctx (<= max_blocks * block_size) bounds ctx_lens + 1.
 * seq_status [batch] int32 or NULL: 0 = the new token's K/V were appended; 1 = the new position
 * ctx_lens[b] is negative or not below max_ctx (no room for it); 2 = the table entry of the new position is
 * not a block of the cache (outside [0, n_blocks)).  With 1 or 2 nothing is written to the cache for
 * that sequence and its logits come from the tokens already cached: the caller must not use them. */
int feather_decode_step(const feather_decoder_t *dec, const void *token_ids, const void *block_tables,
                        const void *ctx_lens, int64_t batch, int64_t max_ctx, void *scratch, void *logits_f32,
                        void *seq_status, void *stream);

/* The fused producers of the decode step as operations of their own (no reference counterpart: the
 * reference has no device-side quantisation; they are the callers' side of the packed GEMV, where the
 * fp32 -> FP8 rounding and the packing happen in the kernel that produces the values).
 *
 * feather_add_rmsnorm_pack: for each of `batch` rows, h += sum of the n_part slices of delta (slice s at
 * delta + s * part_stride floats, [batch, hidden] each, added in slice order; delta may be NULL), then
 * y = h * (1 / sqrt(mean(h^2) + eps)) * gain and xq = packed FP8 of y ([batch, hidden / 4] words).
 * y_f32 (optional, [batch, hidden]) receives the fp32 values the codes were rounded from.  hidden % 4 == 0. */
int feather_add_rmsnorm_pack(void *h_f32, const void *delta_f32, int64_t n_part, int64_t part_stride,
                             const void *gain_f32, void *xq_u32, void *y_f32, int64_t batch, int64_t hidden, float eps,
                             int mode, void *stream);

/* feather_rope_append: qkv [batch, (n_q + 2 n_kv) * d] fp32 (q heads, k heads, v heads; given as n_part
 * slices part_stride floats apart that are added in slice order) -> rotary embedding at position
 * ctx_lens[b] on the q and k heads (rotate-half: element j pairs with j + d/2, angle pos * theta^(-2j/d)),
 * q written as packed FP8 words q_packed [batch, n_q, d/4], k and v encoded and appended to the paged
 * cache ([n_blocks, n_kv, block_size, d/4] words) at position ctx_lens[b] through block_tables
 * [batch, max_blocks]; ctx_after[b] = ctx_lens[b] + 1.  seq_status (optional) as in feather_decode_step:
 * a token without a valid slot is not written and ctx_after[b] keeps the old length.  rot_f32 (optional,
 * [batch, n_q + 2 n_kv, d]) receives the fp32 values the codes were rounded from.  d % 8 == 0. */
int feather_rope_append(const void *qkv_f32, int64_t n_part, int64_t part_stride, const void *ctx_lens,
                        const void *block_tables, void *q_packed, void *k_cache, void *v_cache, void *ctx_after,
                        void *seq_status, void *rot_f32, int64_t batch, int64_t n_q_heads, int64_t n_kv_heads, int64_t d,
                        int64_t block_size, int64_t max_blocks, int64_t n_blocks, float rope_theta, int mode,
                        void *stream);

#ifdef __cplusplus
}
#endif
#endif /* FEATHER_HIP_H */
