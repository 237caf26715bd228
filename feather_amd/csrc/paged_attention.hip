// Single-query (decode) attention over a paged FP8 KV cache, grouped-query
// aware.  The kernel is an HBM gather-stream of the K and V blocks; every cache
// byte is read once per group of query heads that share its KV head.
//
// Work split (flash-decoding): one wave per (sequence, KV head, context split).
// The query heads of the group (up to 16) are the 16 columns of a 16x16 MFMA
// tile and the tokens are its rows:
//     S^T[tok, qh]  = K[tok, :] . Q[qh, :]
//     O^T_c[i, qh] += V^T_c[i, tok] P^T[tok, qh],   dd = 4 i + c, c = 0..3
// K rows are contiguous 16-byte pieces per lane straight from the cache block
// (no LDS).  V needs the token index along the MFMA k dimension while memory
// has the head dimension contiguous; instead of transposing through LDS the
// lane loads the SAME packed word of 8 tokens and uses byte c of every word
// for the c-th MFMA (the four bytes of a word are four different head dims),
// so the transpose is the byte select that decoding does anyway.
//
// Each split writes (m, l, unnormalised O) to scratch; a second tiny kernel
// merges the splits of a (sequence, head).
#include "common.h"

namespace feather {

constexpr int kSplit = 256;  // tokens per wave

__device__ __forceinline__ float4_t pa_mfma16(half8_t a, half8_t b, float4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}

template <int MODE>
__device__ __forceinline__ half8_t pa_dec8(uint32_t w0, uint32_t w1) {
    u32x4 r;
    uint32_t a, b;
    dec_word<MODE>(w0, a, b);
    r.x = a; r.y = b;
    dec_word<MODE>(w1, a, b);
    r.z = a; r.w = b;
    return __builtin_bit_cast(half8_t, r);
}

// fp16 pairs (tok a, tok b) for head-dim byte c of two packed words
template <int MODE>
__device__ __forceinline__ void v_pairs(uint32_t wa, uint32_t wb, uint32_t out[4]) {
    if constexpr (MODE == FEATHER_E5M2) {
#pragma unroll
        for (int c = 0; c < 4; c++)
            out[c] = perm(wb, wa, 0x000c000cu | ((uint32_t)c << 8) | ((uint32_t)(4 + c) << 24));
    } else {
        uint32_t a01, a23, b01, b23;
        dec_word<MODE>(wa, a01, a23);
        dec_word<MODE>(wb, b01, b23);
        out[0] = perm(b01, a01, 0x05040100u);
        out[1] = perm(b01, a01, 0x07060302u);
        out[2] = perm(b23, a23, 0x05040100u);
        out[3] = perm(b23, a23, 0x07060302u);
    }
}

// scratch per (seq, q head, split): [0] = m (log2 domain), [1] = l, [2 .. 2+D) = O
template <int D, int MODE>
__global__ __launch_bounds__(64) void paged_attn_split_kernel(
    const uint32_t *__restrict__ q, const uint32_t *__restrict__ k_cache, const uint32_t *__restrict__ v_cache,
    const int32_t *__restrict__ block_tables, const int32_t *__restrict__ ctx_lens, float *__restrict__ scratch,
    int n_q_heads, int n_kv_heads, int block_size, int max_blocks, int n_splits, int max_ctx, float scale_log2e) {
    constexpr int DW = D / 4;       // words per token row
    constexpr int RB = D / 64;      // 16-word row blocks of V per token
    constexpr int STEPS = D / 32;   // MFMA k-steps of the score product
    const int split = blockIdx.x % n_splits;
    const int kvh = (blockIdx.x / n_splits) % n_kv_heads;
    const int seq = blockIdx.x / (n_splits * n_kv_heads);
    const int group = n_q_heads / n_kv_heads;
    const int ctx = min(ctx_lens[seq], max_ctx);  // never index past the block table
    const int t_begin = split * kSplit;
    const int lane = threadIdx.x, j = lane & 15, kb = lane >> 4;
    const int t_end = min(t_begin + kSplit, ctx);

    const int qh = kvh * group + j;  // this lane's query head (valid if j < group)
    float *my = scratch + ((int64_t)(seq * n_q_heads + qh) * n_splits + split) * (D + 2);
    if (t_begin >= ctx) {            // empty split: neutral element for the merge
        if (j < group && kb == 0) { my[0] = -INFINITY; my[1] = 0.f; }
        return;
    }

    // Q fragments: lane (qh = j, kb) holds dims 16 kb + 8 s' + {0..7} of 32-dim chunk pairs:
    // k-slot mapping of step st: dims 64 (st / 2) + 16 kb + 8 (st % 2) + {0..7}
    half8_t qf[STEPS];
#pragma unroll
    for (int st = 0; st < STEPS; st++) {
        u32x2 w = u32x2{0, 0};
        if (j < group)
            w = *reinterpret_cast<const u32x2 *>(q + (int64_t)(seq * n_q_heads + qh) * DW + 16 * (st / 2) + 4 * kb +
                                                 2 * (st % 2));
        qf[st] = pa_dec8<MODE>(w.x, w.y);
    }

    float4_t o[RB][4];
#pragma unroll
    for (int rb = 0; rb < RB; rb++)
#pragma unroll
        for (int c = 0; c < 4; c++) o[rb][c] = float4_t{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;
    const int32_t *bt = block_tables + (int64_t)seq * max_blocks;

    for (int t0 = t_begin; t0 < t_end; t0 += 32) {
        // ---- scores of 32 tokens: two 16-token row blocks
        float4_t s[2];
#pragma unroll
        for (int a = 0; a < 2; a++) {
            int tok = t0 + 16 * a + j;                    // A-operand row of this lane
            int tc = min(tok, ctx - 1);                   // clamp: masked below
            int64_t base = ((int64_t)bt[tc / block_size] * n_kv_heads + kvh) * block_size + tc % block_size;
            const uint32_t *kr = k_cache + base * DW;
            s[a] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c64 = 0; c64 < RB; c64++) {
                u32x4 w = *reinterpret_cast<const u32x4 *>(kr + 16 * c64 + 4 * kb);  // 16 codes, 64 B per token
                s[a] = pa_mfma16(pa_dec8<MODE>(w.x, w.y), qf[2 * c64], s[a]);
                s[a] = pa_mfma16(pa_dec8<MODE>(w.z, w.w), qf[2 * c64 + 1], s[a]);
            }
        }
        // ---- V words: lane (i = j, kb) takes word i of tokens 16 a + 4 kb + r
        uint32_t vw[RB][2][4];
#pragma unroll
        for (int a = 0; a < 2; a++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                int tok = t0 + 16 * a + 4 * kb + r;
                int tc = min(tok, ctx - 1);
                int64_t base = ((int64_t)bt[tc / block_size] * n_kv_heads + kvh) * block_size + tc % block_size;
#pragma unroll
                for (int rb = 0; rb < RB; rb++) vw[rb][a][r] = tok < ctx ? v_cache[base * DW + 16 * rb + j] : 0u;
            }
        // ---- online softmax (lane column = query head)
        float mx = -INFINITY;
#pragma unroll
        for (int a = 0; a < 2; a++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                float x = s[a][r] * scale_log2e;
                if (t0 + 16 * a + 4 * kb + r >= t_end) x = -INFINITY;
                s[a][r] = x;
                mx = fmaxf(mx, x);
            }
        mx = fmaxf(mx, __shfl_xor(mx, 16, kWave));
        mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
        float m_new = fmaxf(m_run, mx);
        float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        m_run = m_new;
        half8_t p8;
        float rs = 0.f;
#pragma unroll
        for (int a = 0; a < 2; a++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                float e = __builtin_amdgcn_exp2f(s[a][r] - m_new);
                rs += e;
                p8[4 * a + r] = (_Float16)e;
            }
        l_run = l_run * alpha + rs;
        // ---- O^T_c += V^T_c P^T
#pragma unroll
        for (int rb = 0; rb < RB; rb++) {
            uint32_t pr[4][4];  // [pair index][c]
            v_pairs<MODE>(vw[rb][0][0], vw[rb][0][1], pr[0]);
            v_pairs<MODE>(vw[rb][0][2], vw[rb][0][3], pr[1]);
            v_pairs<MODE>(vw[rb][1][0], vw[rb][1][1], pr[2]);
            v_pairs<MODE>(vw[rb][1][2], vw[rb][1][3], pr[3]);
#pragma unroll
            for (int c = 0; c < 4; c++) {
                u32x4 vf = u32x4{pr[0][c], pr[1][c], pr[2][c], pr[3][c]};
                o[rb][c] = pa_mfma16(__builtin_bit_cast(half8_t, vf), p8, o[rb][c] * alpha);
            }
        }
    }

    // ---- write the split's partial: lane (qh = j, kb) holds O rows i = 4 kb + r -> dd = 64 rb + 4 i + c
    float l = l_run;
    l += __shfl_xor(l, 16, kWave);
    l += __shfl_xor(l, 32, kWave);
    if (j < group) {
        if (kb == 0) { my[0] = m_run; my[1] = l; }
#pragma unroll
        for (int rb = 0; rb < RB; rb++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                float4_t x = float4_t{o[rb][0][r], o[rb][1][r], o[rb][2][r], o[rb][3][r]};
                *reinterpret_cast<float4_t *>(my + 2 + 64 * rb + 4 * (4 * kb + r)) = x;
            }
    }
}

// out[seq, qh, :] = sum_s 2^(m_s - m) O_s / sum_s 2^(m_s - m) l_s
template <int D>
__global__ __launch_bounds__(64) void paged_attn_merge_kernel(const float *__restrict__ scratch,
                                                             float *__restrict__ out, int n_splits) {
    const int64_t item = blockIdx.x;  // seq * n_q_heads + qh
    const float *base = scratch + item * n_splits * (D + 2);
    float m = -INFINITY;
    for (int s = 0; s < n_splits; s++) m = fmaxf(m, base[(int64_t)s * (D + 2)]);
    float acc[D / 64];
#pragma unroll
    for (int i = 0; i < D / 64; i++) acc[i] = 0.f;
    float l = 0.f;
    for (int s = 0; s < n_splits; s++) {
        const float *p = base + (int64_t)s * (D + 2);
        float ms = p[0];
        if (ms == -INFINITY) continue;
        float w = __builtin_amdgcn_exp2f(ms - m);
        l += w * p[1];
#pragma unroll
        for (int i = 0; i < D / 64; i++) acc[i] += w * p[2 + 64 * i + threadIdx.x];
    }
#pragma unroll
    for (int i = 0; i < D / 64; i++) out[item * D + 64 * i + threadIdx.x] = l > 0.f ? acc[i] / l : 0.f;
}

template <int D, int MODE>
static int launch_paged(const void *q, const void *kc, const void *vc, const void *bt, const void *cl, void *out,
                        void *scratch, int64_t n_seq, int64_t n_q_heads, int64_t n_kv_heads, int64_t block_size,
                        int64_t max_blocks, int64_t max_ctx, float scale, hipStream_t s) {
    int n_splits = (int)((max_ctx + kSplit - 1) / kSplit);
    if (n_splits < 1) n_splits = 1;
    int64_t blocks = n_seq * n_kv_heads * n_splits;
    FEATHER_CHECK(blocks < (1ll << 31), FEATHER_ESHAPE, "feather_paged_attn_fp8: grid too large");
    const float log2e = 1.4426950408889634f;
    hipLaunchKernelGGL((paged_attn_split_kernel<D, MODE>), dim3((unsigned)blocks), dim3(64), 0, s,
                       (const uint32_t *)q, (const uint32_t *)kc, (const uint32_t *)vc, (const int32_t *)bt,
                       (const int32_t *)cl, (float *)scratch, (int)n_q_heads, (int)n_kv_heads, (int)block_size,
                       (int)max_blocks, n_splits, (int)max_ctx, scale * log2e);
    int rc = check_launch("feather_paged_attn_fp8");
    if (rc != FEATHER_OK) return rc;
    hipLaunchKernelGGL((paged_attn_merge_kernel<D>), dim3((unsigned)(n_seq * n_q_heads)), dim3(64), 0, s,
                       (const float *)scratch, (float *)out, n_splits);
    return check_launch("feather_paged_attn_fp8 (merge)");
}

}  // namespace feather

using namespace feather;

extern "C" int64_t feather_paged_attn_scratch_bytes(int64_t n_seq, int64_t n_q_heads, int64_t d, int64_t max_ctx) {
    if (n_seq < 0 || n_q_heads < 0 || d < 0 || max_ctx < 0) return 0;
    int64_t n_splits = (max_ctx + kSplit - 1) / kSplit;
    if (n_splits < 1) n_splits = 1;
    return n_seq * n_q_heads * n_splits * (d + 2) * 4;
}

extern "C" int feather_paged_attn_fp8(const void *q, const void *k_cache, const void *v_cache, const void *block_tables,
                                      const void *ctx_lens, void *out_f32, void *scratch, int64_t n_seq,
                                      int64_t n_q_heads, int64_t n_kv_heads, int64_t d, int64_t block_size,
                                      int64_t max_blocks, int64_t max_ctx, int mode, float scale, void *stream) {
    const char *me = "feather_paged_attn_fp8";
    FEATHER_CHECK(mode == FEATHER_E5M2 || mode == FEATHER_E4M3, FEATHER_EMODE, "%s: mode %d not supported", me, mode);
    FEATHER_CHECK(n_seq >= 0 && n_q_heads > 0 && n_kv_heads > 0 && block_size > 0 && max_blocks >= 0 && max_ctx >= 0,
                  FEATHER_EINVAL, "%s: bad shape", me);
    FEATHER_CHECK(n_q_heads % n_kv_heads == 0, FEATHER_ESHAPE, "%s: n_q_heads=%lld not a multiple of n_kv_heads=%lld",
                  me, (long long)n_q_heads, (long long)n_kv_heads);
    FEATHER_CHECK(n_q_heads / n_kv_heads <= 16, FEATHER_ESHAPE, "%s: at most 16 query heads per KV head", me);
    FEATHER_CHECK(d == 64 || d == 128 || d == 256, FEATHER_ESHAPE, "%s: head dim %lld not supported (64, 128, 256)", me,
                  (long long)d);
    FEATHER_CHECK(max_ctx <= max_blocks * block_size, FEATHER_ESHAPE, "%s: max_ctx exceeds the block table", me);
    if (n_seq == 0) return FEATHER_OK;
    FEATHER_CHECK(q && k_cache && v_cache && block_tables && ctx_lens && out_f32 && scratch, FEATHER_EINVAL,
                  "%s: null pointer", me);
    FEATHER_CHECK(aligned(q, 8) && aligned(k_cache, 16) && aligned(v_cache, 16) && aligned(out_f32, 4) &&
                      aligned(scratch, 16) && aligned(block_tables, 4) && aligned(ctx_lens, 4),
                  FEATHER_EINVAL, "%s: misaligned pointer", me);
    hipStream_t s = (hipStream_t)stream;
#define FEATHER_PA(DD, MM)                                                                                          \
    return launch_paged<DD, MM>(q, k_cache, v_cache, block_tables, ctx_lens, out_f32, scratch, n_seq, n_q_heads,     \
                                n_kv_heads, block_size, max_blocks, max_ctx, scale, s)
    if (mode == FEATHER_E5M2) {
        if (d == 64) FEATHER_PA(64, FEATHER_E5M2);
        if (d == 128) FEATHER_PA(128, FEATHER_E5M2);
        FEATHER_PA(256, FEATHER_E5M2);
    }
    if (d == 64) FEATHER_PA(64, FEATHER_E4M3);
    if (d == 128) FEATHER_PA(128, FEATHER_E4M3);
    FEATHER_PA(256, FEATHER_E4M3);
#undef FEATHER_PA
}
