// Single-query (decode) attention over a paged FP8 KV cache, grouped-query
// aware.  The kernel is an HBM gather-stream of the K and V blocks; every cache
// byte is read once per group of query heads that share its KV head.
//
// Work split (flash-decoding): one workgroup of 4 waves per (sequence, KV head,
// split of 512 tokens); the waves take the 32-token steps of the split round
// robin and are merged through LDS, the splits of a sequence by a second small
// kernel (skipped when the whole context fits one split).  Inside a wave the
// query heads of the group (up to 16) are the 16 columns of a 16x16 MFMA tile
// and the tokens are its rows:
//     S^T[tok, qh]  = K[tok, :] . Q[qh, :]
//     O^T_c[i, qh] += V^T_c[i, tok] P^T[tok, qh],   dd = 4 i + c, c = 0..3
// K rows are contiguous 16-byte pieces per lane straight from the cache block
// (no LDS).  V needs the token index along the MFMA k dimension while memory
// has the head dimension contiguous; instead of transposing through LDS the
// lane loads the SAME packed word of 8 tokens and uses byte c of every word
// for the c-th MFMA (the four bytes of a word are four different head dims),
// so the transpose is the byte select that decoding does anyway.
// A wave issues the loads of all its steps (up to four) before it consumes the
// first, so the dependent chains block id -> row address -> data of the steps
// overlap instead of adding up.
// (Letting the last split of a sequence to finish do the merge, with the partials
// and an arrival counter handled by device-scope atomics, gives the same results
// without the second launch but was slower: write-through stores, the ticket and
// the read-back are three memory-side round trips in a row, +7 us per call
// against ~4 us for the merge kernel.)
#include <mutex>

#include "internal.h"
#include "common.h"

namespace feather {

constexpr int kPaWaves = 4;
constexpr int kPaThreads = kPaWaves * kWave;
constexpr int kSplit = 512;   // tokens per workgroup
constexpr int kStepTok = 32;  // tokens per wave step

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
        // interleave the codes of the two tokens first ((a0 b0 a1 b1), (a2 b2 a3 b3)): the decoder's own
        // pairs are then the (tok a, tok b) pairs
        dec_word<MODE>(perm(wb, wa, 0x05010400u), out[0], out[1]);
        dec_word<MODE>(perm(wb, wa, 0x07030602u), out[2], out[3]);
    }
}

// scratch per (seq, q head, split): [0] = m (log2 domain), [1] = l, [2 .. 2+D) = unnormalised O
// FAST: block_size is a power of two >= 4: token -> block / slot by shift and mask, and an aligned
// group of 4 tokens never straddles a block (one table lookup per group)
// (parameter order: what a wave needs before its first loads -- the lengths, the table, the operands
// and the shape -- fills the 16 dwords of kernel arguments that arrive preloaded in SGPRs; the rest
// is fetched with s_load while those loads are in flight)
//
// FUSED (the decode step's attention; needs FAST and D = 64): the kernel also does what the step otherwise
// runs as a separate kernel in front of it.  `ctx_lens` then points to the step's work plan (one entry per
// workgroup item, written once per step: sequence, split, token count, owner flag and the block ids of the
// split, so that a workgroup knows its work and its blocks after ONE memory round trip), `q` is unused and the
// query comes from the fused QKV projection's fp32 partial sums `qkv` (n_part slices, part_stride floats
// apart): the workgroup adds the slices in slice order, applies the rotary embedding with the step's cos / sin
// table `cs` ([n_seq, D / 2] pairs), rounds to FP8 (quant4) and keeps the packed query heads in LDS.  The
// workgroup whose split holds the new token's position ("owner") does the same for that token's K and V row of
// its KV head, appends them to the cache and scores the token from LDS after the cached ones (wave 0, one extra
// one-token step), so the cached tokens are read from memory and the new one never is.
constexpr int kEarly = 2;             // FUSED: steps of a wave whose rows are requested before the query is ready
constexpr int kFusedMaxPairs = 96;   // (group + 2) * n_part the LDS staging of the FUSED prologue holds

template <int D, int MODE, bool FAST, bool FUSED = false>
__global__ __launch_bounds__(kPaThreads) void paged_attn_split_kernel(
    const int32_t *__restrict__ ctx_lens, const int32_t *__restrict__ block_tables, const uint32_t *__restrict__ q,
    const uint32_t *__restrict__ k_cache, const uint32_t *__restrict__ v_cache, int n_q_heads, int n_kv_heads,
    int block_size, int max_blocks, int n_splits, int max_ctx, float scale_log2e, float *__restrict__ scratch,
    float *__restrict__ out_f32, uint32_t *__restrict__ out_packed, _Float16 *__restrict__ out_q16, uint32_t max_blk,
    const float *__restrict__ qkv, int n_part, int64_t part_stride, const float *__restrict__ cs,
    uint32_t *__restrict__ k_cache_w, uint32_t *__restrict__ v_cache_w) {
    static_assert(!FUSED || (FAST && D == 64), "the fused prologue is written for D = 64 and power-of-two blocks");
    const int bs_shift = FAST ? __builtin_ctz((unsigned)block_size) : 0;
    constexpr int DW = D / 4;       // words per token row
    constexpr int RB = D / 64;      // 16-word row blocks of V per token
    constexpr int STEPS = D / 32;   // MFMA k-steps of the score product
    __shared__ float ml_lds[kPaWaves][2][16];
    __shared__ float4_t o_lds[kPaWaves - 1][RB * 4][kWave];
    __shared__ float4_t part_lds[FUSED ? kFusedMaxPairs * (D / 8) * 2 : 1];   // [slice][head slot][D/8 threads][lo, hi]
    __shared__ uint32_t q_lds[FUSED ? 16 * DW : 1];                             // packed query heads of the group
    __shared__ uint32_t kv_new[FUSED ? 2 * DW : 1];                             // packed K and V row of the new token

    // Work item of this workgroup.  With one split per sequence the grid is exactly the
    // (sequence, KV head) pairs.  Otherwise the grid is sized for max_ctx and most sequences use
    // fewer splits: the workgroups that have work are the FIRST ones in launch order (items are
    // numbered over the splits that exist, found from a prefix sum over the context lengths that
    // every wave computes for itself), so the hardware spreads them over all XCDs and CUs in its
    // first pass and the rest exit at once.  (Numbering items over the full grid left the CUs
    // unevenly loaded; and with the split index fastest all first splits landed on one XCD,
    // because consecutive workgroups go to consecutive XCDs.)
    const int lane = threadIdx.x & 63, wave = wave_id(), j = lane & 15, kb = lane >> 4;
    const int kvh = blockIdx.x % n_kv_heads;
    int seq = blockIdx.x / n_kv_heads, split = 0;
    int ctx_raw;
    bool owner = false;                                     // FUSED: this workgroup appends and scores the new token
    const int32_t *entry = nullptr;
    if constexpr (FUSED) {
        // plan entry: {sequence (-1: no work), split, tokens of the sequence incl. the new one, owner flag, block ids of the split}
        // (an entry without work has sequence -1; the test waits until the block ids of the entry have been
        // requested, so that header and ids arrive in one round trip: every entry has all its id slots)
        entry = ctx_lens + (int64_t)(blockIdx.x / n_kv_heads) * (4 + (kSplit >> bs_shift));
        seq = entry[0];
        split = entry[1];
        ctx_raw = entry[2];
        owner = entry[3] != 0;
    } else if (n_splits > 1) {
        const int n_seq = gridDim.x / (n_splits * n_kv_heads);
        const int item = blockIdx.x / n_kv_heads;          // index over the (sequence, split) pairs that exist
        seq = -1;
        ctx_raw = 0;
        if (n_seq <= kWave) {
            // Largest items first: all full splits in sequence order, then the partial last splits by
            // size, largest first.  Every workgroup with work is resident at once and the hardware deals
            // them to the CUs in launch order, so when the items are not a multiple of the CUs the CUs
            // that get one more than the others get the smallest ones (with sequence order a full split
            // could be the extra one and its CU finished last: 15 us against 10 us for the median).
            const int c = lane < n_seq ? max(ctx_lens[lane], 0) : 0;
            const int cc = min(c, max_ctx);
            const int nf = cc / kSplit, ps = cc % kSplit;   // full splits, tokens of the partial one
            int inc = nf;                                   // inclusive prefix sum over the lanes
#pragma unroll
            for (int off = 1; off < kWave; off <<= 1) {
                const int t = __shfl_up(inc, off, kWave);
                if (lane >= off) inc += t;
            }
            const int n_full = __builtin_amdgcn_readlane(inc, kWave - 1);
            uint64_t hit;
            if (item < n_full) {
                const int exc = inc - nf;
                hit = __builtin_amdgcn_ballot_w64(item >= exc && item < exc + nf);
                if (hit) split = item - __builtin_amdgcn_readlane(exc, __builtin_ctzll(hit));
            } else {
                int rank = 0;                               // partial splits larger than this lane's (ties: lower sequence first)
                for (int t = 0; t < n_seq; t++) {
                    const int pt = __builtin_amdgcn_readlane(ps, t);
                    rank += (pt > ps || (pt == ps && t < lane)) ? 1 : 0;
                }
                hit = __builtin_amdgcn_ballot_w64(ps > 0 && rank == item - n_full);
                if (hit) split = __builtin_amdgcn_readlane(nf, __builtin_ctzll(hit));
            }
            if (hit) {
                seq = __builtin_ctzll(hit);
                ctx_raw = __builtin_amdgcn_readlane(c, seq);
            }
        } else {
        int base = 0;
        for (int s0 = 0; s0 < n_seq && seq < 0; s0 += kWave) {
            const int s = s0 + lane;
            const int c = s < n_seq ? max(ctx_lens[s], 0) : 0;
            const int ns = (min(c, max_ctx) + kSplit - 1) / kSplit;
            int inc = ns;                                   // inclusive prefix sum over the lanes
#pragma unroll
            for (int off = 1; off < kWave; off <<= 1) {
                const int t = __shfl_up(inc, off, kWave);
                if (lane >= off) inc += t;
            }
            const int exc = base + inc - ns;
            const uint64_t hit = __builtin_amdgcn_ballot_w64(item >= exc && item < exc + ns);
            if (hit) {
                const int src = __builtin_ctzll(hit);
                seq = s0 + src;
                split = item - __builtin_amdgcn_readlane(exc, src);
                ctx_raw = __builtin_amdgcn_readlane(c, src);
            }
            base += __builtin_amdgcn_readlane(inc, kWave - 1);
        }
        }
        if (seq < 0) return;                                // beyond the last item (whole workgroup)
    } else {
        ctx_raw = ctx_lens[seq];
    }
    const int group = n_q_heads / n_kv_heads;
    const int t_begin = split * kSplit;
    auto blk_of = [&](int tok) { return FAST ? tok >> bs_shift : tok / block_size; };
    auto slot_of = [&](int tok) { return FAST ? tok & (block_size - 1) : tok % block_size; };
    const int32_t *bt = block_tables + (int64_t)seq * max_blocks;

    const int qh = kvh * group + j;  // this lane's query head (valid if j < group)
    // Q fragments: k-slot mapping of step st: dims 64 (st / 2) + 16 kb + 8 (st % 2) + {0..7}
    u32x2 qw[STEPS];
#pragma unroll
    for (int st = 0; st < STEPS; st++) {
        qw[st] = u32x2{0, 0};
        if constexpr (!FUSED)
            if (j < group)
                qw[st] = *reinterpret_cast<const u32x2 *>(q + (int64_t)(seq * n_q_heads + qh) * DW + 16 * (st / 2) +
                                                          4 * kb + 2 * (st % 2));
    }

    // One step = packed K (16 codes of the lane's token per 64-dim chunk) and V (word j of 8 tokens).
    // A step is a chain of dependent memory accesses: block id -> row address -> data.  The ids of
    // all steps in flight are fetched (and waited for) before the first data load, because memory
    // returns in order and a lookup issued behind another step's data would wait for it; and the
    // ids of the first round are fetched without waiting for the context length (any token index
    // below max_ctx is inside the table; entries past the context are replaced below), so that the
    // length, the query and the ids arrive together instead of one after the other.
    struct Step {
        int kid[2], vid[2][FAST ? 1 : 4];
        u32x4 kw[2][RB];
        uint32_t vw[RB][2][4];
    };
    constexpr int NF = D == 64 ? 4 : (D == 128 ? 2 : 1);
    Step steps[NF];
    const int t_cap = max(max_ctx - 1, 0);
    auto fetch_ids = [&](Step &T, int t0) {
#pragma unroll
        for (int a = 0; a < 2; a++) {
            if constexpr (FUSED) {                // the split's ids sit in the plan entry (every slot of it is filled)
                T.kid[a] = entry[4 + ((t0 - t_begin + 16 * a + j) >> bs_shift)];
                T.vid[a][0] = entry[4 + ((t0 - t_begin + 16 * a + 4 * kb) >> bs_shift)];
            } else {
                T.kid[a] = bt[blk_of(min(t0 + 16 * a + j, t_cap))];
#pragma unroll
                for (int r = 0; r < (FAST ? 1 : 4); r++) T.vid[a][r] = bt[blk_of(min(t0 + 16 * a + 4 * kb + r, t_cap))];
            }
        }
    };
    int fallback = 0;                             // block of the split's first token: valid whenever the split has work
    if (max_ctx > 0) {
        fallback = FUSED ? entry[4] : bt[blk_of(min(t_begin, t_cap))];
#pragma unroll
        for (int f = 0; f < NF; f++) fetch_ids(steps[f], t_begin + kStepTok * (wave + kPaWaves * f));
    }
    if constexpr (FUSED)
        if (seq < 0) return;                      // beyond the last item (whole workgroup)

    const int ctx = min(ctx_raw, max_ctx);        // never index past the block table
    if (t_begin >= ctx) {                         // empty split: the merge never reads it
        if (n_splits == 1) {                      // no merge pass: an empty context gives a zero result
            for (int i = threadIdx.x; i < group * DW; i += kPaThreads) {
                int64_t w = ((int64_t)seq * n_q_heads + kvh * group) * DW + i;
                if (out_f32) *reinterpret_cast<float4_t *>(out_f32 + 4 * w) = float4_t{0.f, 0.f, 0.f, 0.f};
                if (out_packed) out_packed[w] = 0u;
                if (out_q16) *reinterpret_cast<u32x2 *>(out_q16 + 4 * w) = u32x2{0u, 0u};
            }
        }
        return;
    }
    // tokens of this split that are read from the cache: the owner's new token (position ctx - 1) is not among them
    const int t_end = min(t_begin + kSplit, owner ? ctx - 1 : ctx);
    const int n_steps = (t_end - t_begin + kStepTok - 1) / kStepTok;

    half8_t qf[STEPS];
    if constexpr (!FUSED) {
#pragma unroll
        for (int st = 0; st < STEPS; st++) qf[st] = pa_dec8<MODE>(qw[st].x, qw[st].y);
    }

    float4_t o[RB][4];
#pragma unroll
    for (int rb = 0; rb < RB; rb++)
#pragma unroll
        for (int c = 0; c < 4; c++) o[rb][c] = float4_t{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;

    // Row addresses are formed right before the loads (only the block ids of the steps in flight
    // stay in registers).  Rows past the context read the fallback block (valid memory) and are
    // masked later.
    // row index inside the cache in 32 bits (a cache of 2^31 rows of d codes is >= 128 GB)
    // block ids come from the caller's table: an id outside the cache (padding, -1) is clamped to the last block,
    // so that a bad table gives a wrong result for that sequence and never an access outside the cache
    auto row_base = [&](int blk, int tok) {
        return (int64_t)(uint32_t)((min((uint32_t)blk, max_blk) * n_kv_heads + kvh) * block_size + slot_of(tok));
    };
    auto load_step = [&](Step &S, int t0) {
        const bool full = t0 + kStepTok <= t_end; // wave-uniform: every token of the step exists
#pragma unroll
        for (int a = 0; a < 2; a++) {
            const int tk = t0 + 16 * a + j;
            const uint32_t *kr = k_cache + row_base(full || tk < t_end ? S.kid[a] : fallback, tk) * DW;
#pragma unroll
            for (int c64 = 0; c64 < RB; c64++) S.kw[a][c64] = *reinterpret_cast<const u32x4 *>(kr + 16 * c64 + 4 * kb);
            const int tq = t0 + 16 * a + 4 * kb;
            const uint32_t *vq = nullptr;
            if constexpr (FAST)                   // an aligned group of 4 tokens shares a block
                vq = v_cache + row_base(full || tq < t_end ? S.vid[a][0] : fallback, tq) * DW + j;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const uint32_t *vr = vq + r * DW;
                if constexpr (!FAST) vr = v_cache + row_base(full || tq + r < t_end ? S.vid[a][r] : fallback, tq + r) * DW + j;
                if (full) {
#pragma unroll
                    for (int rb = 0; rb < RB; rb++) S.vw[rb][a][r] = vr[16 * rb];
                } else {
#pragma unroll
                    for (int rb = 0; rb < RB; rb++) S.vw[rb][a][r] = tq + r < t_end ? vr[16 * rb] : 0u;
                }
            }
        }
    };
    auto compute_step = [&](const Step &S, int t0) {
        float4_t s[2];
#pragma unroll
        for (int a = 0; a < 2; a++) {
            s[a] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c64 = 0; c64 < RB; c64++) {
                s[a] = pa_mfma16(pa_dec8<MODE>(S.kw[a][c64].x, S.kw[a][c64].y), qf[2 * c64], s[a]);
                s[a] = pa_mfma16(pa_dec8<MODE>(S.kw[a][c64].z, S.kw[a][c64].w), qf[2 * c64 + 1], s[a]);
            }
        }
        mfma_settle<2>(s);   // the first readers of the scores are asm statements (max3_raw)
        // online softmax (lane column = query head), log2 domain; only the last step of a split
        // can hold tokens past its end (wave-uniform test)
        if (t0 + kStepTok > t_end) {
            // token 16 a + 4 kb + r of the step is past the end if 16 a + r >= rel; rel is made opaque
            // so that this rarely taken branch stays a branch (if-converted, its compares and selects
            // run in every step)
            int rel = t_end - t0 - 4 * kb;
            asm volatile("" : "+v"(rel));
#pragma unroll
            for (int a = 0; a < 2; a++)
#pragma unroll
                for (int r = 0; r < 4; r++)
                    if (16 * a + r >= rel) s[a][r] = -INFINITY;
        }
        float mx = max3_raw(max3_raw(s[0][0], s[0][1], s[0][2]), s[0][3], s[1][0]);
        mx = max_raw(max3_raw(mx, s[1][1], s[1][2]), s[1][3]);
        mx = max_xor32(max_xor16(mx));
        const float m_new = max_raw(m_run, mx * scale_log2e);    // scale > 0: the maximum commutes with it
        half8_t p8;
        float rs = 0.f;
#pragma unroll
        for (int a = 0; a < 2; a++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                float e = __builtin_amdgcn_exp2f(__builtin_fmaf(s[a][r], scale_log2e, -m_new));
                rs += e;
                p8[4 * a + r] = (_Float16)e;
            }
        // rescale only when some query head of the wave saw a new maximum (wave-uniform test)
        const bool moved = __builtin_amdgcn_ballot_w64(m_new != m_run) != 0;
        float alpha = 1.0f;
        if (moved) {
            alpha = __builtin_amdgcn_exp2f(m_run - m_new);
            m_run = m_new;
#pragma unroll
            for (int rb = 0; rb < RB; rb++)
#pragma unroll
                for (int c = 0; c < 4; c++) o[rb][c] *= alpha;
        }
        l_run = l_run * alpha + rs;
#pragma unroll
        for (int rb = 0; rb < RB; rb++) {
            uint32_t pr[4][4];  // [pair index][c]
            v_pairs<MODE>(S.vw[rb][0][0], S.vw[rb][0][1], pr[0]);
            v_pairs<MODE>(S.vw[rb][0][2], S.vw[rb][0][3], pr[1]);
            v_pairs<MODE>(S.vw[rb][1][0], S.vw[rb][1][1], pr[2]);
            v_pairs<MODE>(S.vw[rb][1][2], S.vw[rb][1][3], pr[3]);
#pragma unroll
            for (int c = 0; c < 4; c++) {
                u32x4 vf = u32x4{pr[0][c], pr[1][c], pr[2][c], pr[3][c]};
                o[rb][c] = pa_mfma16(__builtin_bit_cast(half8_t, vf), p8, o[rb][c]);
            }
        }
    };

    float4_t cs01 = float4_t{0.f, 0.f, 0.f, 0.f}, cs23 = cs01;     // FUSED: (cos, sin) of this thread's four element pairs
    if constexpr (FUSED) {
        // ---- query (and, for the owner, the new token's K / V row) from the QKV projection's partial sums.
        // Phase A: every (slice, head slot, 4 + 4 elements) unit is fetched by some thread -- spread over the
        // whole workgroup so that a thread holds two or three units, not every slice of its element -- and
        // parked in LDS; the cos / sin pairs of the threads that will rotate are fetched in the same round.
        constexpr int T8 = D / 8;                                  // threads per head slot: 4 low + 4 high elements each
        const int heads = n_q_heads + 2 * n_kv_heads;
        const int slots = group + (owner ? 2 : 0);                 // query heads of the group, then the K and the V head
        const int units = n_part * slots * T8;
        auto src_row = [&](int slot) {
            return slot < group ? kvh * group + slot : (slot == group ? n_q_heads + kvh : n_q_heads + n_kv_heads + kvh);
        };
        constexpr int kUnitsPerThread = (kFusedMaxPairs * T8 + kPaThreads - 1) / kPaThreads;
        float4_t plo[kUnitsPerThread], phi[kUnitsPerThread];
#pragma unroll
        for (int it = 0; it < kUnitsPerThread; it++) {
            const int u = min((int)threadIdx.x + it * kPaThreads, units - 1);   // surplus threads repeat the last unit
            const int tt = u % T8, slot = (u / T8) % slots, slice = u / (T8 * slots);
            const float *x = qkv + ((int64_t)seq * heads + src_row(slot)) * D + (int64_t)slice * part_stride;
            plo[it] = *reinterpret_cast<const float4_t *>(x + 4 * tt);
            phi[it] = *reinterpret_cast<const float4_t *>(x + D / 2 + 4 * tt);
        }
        const int my_tt = threadIdx.x % T8;
        const float4_t *csp = reinterpret_cast<const float4_t *>(cs + ((int64_t)seq * (D / 2) + 4 * my_tt) * 2);
        cs01 = csp[0];                                             // (cos, sin) of elements 4 tt .. 4 tt + 3
        cs23 = csp[1];
        // the wave's first step goes out behind the partial sums (memory returns in order: parking the sums waits for
        // them, not for the rows), so the cache rows start to stream one round trip earlier than the query allows
#pragma unroll
        for (int f = 0; f < kEarly; f++)   // (a wave without such a step reads the split's first block: no branch, so the wait below counts loads)
            load_step(steps[f], t_begin + kStepTok * (wave + kPaWaves * f));
#pragma unroll
        for (int it = 0; it < kUnitsPerThread; it++) {
            const int u = threadIdx.x + it * kPaThreads;
            if (u < units) {
                part_lds[2 * u] = plo[it];
                part_lds[2 * u + 1] = phi[it];
            }
        }
    }
    // Phase B runs behind the loads of the wave's first step.  (Only that step: with the rows of all four steps
    // requested before the partial sums are parked, their 64 destination registers are live together with the
    // partial sums' and one workgroup less fits a CU.)
    auto fused_phase_b = [&]() {
        constexpr int T8 = D / 8;
        const int slots = group + (owner ? 2 : 0);
        const bool rotates = (int)threadIdx.x < slots * T8;
        const int my_slot = rotates ? threadIdx.x / T8 : 0, my_tt = threadIdx.x % T8;
        __syncthreads();
        // Phase B: one thread per (head slot, 4 + 4 elements) adds the slices in slice order, rotates (query and
        // K heads), rounds to FP8 and packs: the arithmetic of the stand-alone rotary kernel, value for value.
        if (rotates) {
            float4_t lo = part_lds[2 * (my_slot * T8 + my_tt)], hi = part_lds[2 * (my_slot * T8 + my_tt) + 1];
            for (int sl = 1; sl < n_part; sl++) {
                lo += part_lds[2 * ((sl * slots + my_slot) * T8 + my_tt)];
                hi += part_lds[2 * ((sl * slots + my_slot) * T8 + my_tt) + 1];
            }
            if (my_slot <= group) {                                // query heads and the K head; V is not rotated
                const float c4[4] = {cs01[0], cs01[2], cs23[0], cs23[2]}, s4[4] = {cs01[1], cs01[3], cs23[1], cs23[3]};
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float a = lo[i], bb = hi[i];
                    lo[i] = a * c4[i] - bb * s4[i];
                    hi[i] = bb * c4[i] + a * s4[i];
                }
            }
            const uint32_t wlo = quant4<MODE>(lo[0], lo[1], lo[2], lo[3]), whi = quant4<MODE>(hi[0], hi[1], hi[2], hi[3]);
            if (my_slot < group) {
                q_lds[my_slot * DW + my_tt] = wlo;
                q_lds[my_slot * DW + my_tt + T8] = whi;
            } else {                                               // owner only: append the row and keep it for the extra step
                const int which = my_slot - group, pos = ctx - 1;
                kv_new[which * DW + my_tt] = wlo;
                kv_new[which * DW + my_tt + T8] = whi;
                uint32_t *row = (which ? v_cache_w : k_cache_w) + row_base(entry[4 + ((pos - t_begin) >> bs_shift)], pos) * DW;
                row[my_tt] = wlo;
                row[my_tt + T8] = whi;
            }
        }
        __syncthreads();
#pragma unroll
        for (int st = 0; st < STEPS; st++) {
            if (j < group) qw[st] = *reinterpret_cast<const u32x2 *>(&q_lds[j * DW + 16 * (st / 2) + 4 * kb + 2 * (st % 2)]);
            qf[st] = pa_dec8<MODE>(qw[st].x, qw[st].y);
        }
    };

    // Phase B: the query is rotated and packed while the rows of the wave's first step are in flight (every wave
    // takes part: the phase holds workgroup barriers).
    if constexpr (FUSED) fused_phase_b();

    // The wave's steps are wave, wave + 4, ...; NF of them are in flight together: a wave has only a handful of
    // steps, so their chains must overlap each other.  The loads of a turn go out kAhead steps ahead of the
    // arithmetic instead of all up front: when every workgroup of the grid asks for its rows at once the memory
    // system is the bottleneck and a wave sits in the issue of its loads until there is room for them, so the
    // arithmetic of the early steps fits under the stream of the later ones.
    constexpr int kAhead = NF < 3 ? NF : 3;
    for (int st = wave; st < n_steps; st += kPaWaves * NF) {
        const bool first_turn = st == wave;
        if (!first_turn) {
#pragma unroll
            for (int f = 0; f < NF; f++)
                if (st + kPaWaves * f < n_steps) fetch_ids(steps[f], t_begin + kStepTok * (st + kPaWaves * f));
        }
#pragma unroll
        for (int f = 0; f < kAhead; f++)
            if (st + kPaWaves * f < n_steps && !(FUSED && first_turn && f < kEarly))
                load_step(steps[f], t_begin + kStepTok * (st + kPaWaves * f));
#pragma unroll
        for (int f = 0; f < NF; f++) {
            if (f + kAhead < NF && st + kPaWaves * (f + kAhead) < n_steps && !(FUSED && first_turn && f + kAhead < kEarly))
                load_step(steps[f + kAhead], t_begin + kStepTok * (st + kPaWaves * (f + kAhead)));
            if (st + kPaWaves * f < n_steps) compute_step(steps[f], t_begin + kStepTok * (st + kPaWaves * f));
        }
    }

    if constexpr (FUSED) {
        // ---- the new token, scored from LDS by wave 0 of its owner as one more step of one token
        if (owner && wave == 0) {
            float sc = 0.f;
#pragma unroll
            for (int st = 0; st < STEPS; st++) {
                const u32x2 kw = *reinterpret_cast<const u32x2 *>(&kv_new[16 * (st / 2) + 4 * kb + 2 * (st % 2)]);
                const u32x4 kd = __builtin_bit_cast(u32x4, pa_dec8<MODE>(kw.x, kw.y)), qd = __builtin_bit_cast(u32x4, qf[st]);
                sc = dot2(kd.x, qd.x, sc);
                sc = dot2(kd.y, qd.y, sc);
                sc = dot2(kd.z, qd.z, sc);
                sc = dot2(kd.w, qd.w, sc);
            }
            sc += __shfl_xor(sc, 16, kWave);                       // the four lanes of a head hold a quarter of the dims each
            sc += __shfl_xor(sc, 32, kWave);
            const float m_new = max_raw(m_run, sc * scale_log2e);
            const float e = __builtin_amdgcn_exp2f(__builtin_fmaf(sc, scale_log2e, -m_new));
            const float pf = (float)(_Float16)e;                   // P is rounded to fp16 before it multiplies V
            const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
            m_run = m_new;
            l_run = l_run * alpha + (kb == 0 ? e : 0.f);           // the lanes' sums are added over kb at the end
#pragma unroll
            for (int rb = 0; rb < RB; rb++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    // accumulator row 4 kb + r of block c is head dim 64 rb + 4 (4 kb + r) + c: word 16 rb + 4 kb + r, byte c
                    const u32x2 vd = dequant4<MODE>(kv_new[DW + 16 * rb + 4 * kb + r]);
                    const half2_t v01 = as_half2(vd.x), v23 = as_half2(vd.y);
                    o[rb][0][r] = o[rb][0][r] * alpha + pf * (float)v01.x;
                    o[rb][1][r] = o[rb][1][r] * alpha + pf * (float)v01.y;
                    o[rb][2][r] = o[rb][2][r] * alpha + pf * (float)v23.x;
                    o[rb][3][r] = o[rb][3][r] * alpha + pf * (float)v23.y;
                }
        }
    }

    // ---- merge the four waves through LDS (wave 0 finishes)
    float l = l_run;
    l += __shfl_xor(l, 16, kWave);
    l += __shfl_xor(l, 32, kWave);
    if (kb == 0) {
        ml_lds[wave][0][j] = m_run;
        ml_lds[wave][1][j] = l;
    }
    if (wave > 0) {
#pragma unroll
        for (int rb = 0; rb < RB; rb++)
#pragma unroll
            for (int c = 0; c < 4; c++) o_lds[wave - 1][rb * 4 + c][lane] = o[rb][c];
    }
    __syncthreads();
    if (wave != 0) return;
    float m_all = m_run;
#pragma unroll
    for (int w = 1; w < kPaWaves; w++) m_all = fmaxf(m_all, ml_lds[w][0][j]);
    float wgt = __builtin_amdgcn_exp2f(m_run - m_all);
    float l_all = wgt * l;
#pragma unroll
    for (int rb = 0; rb < RB; rb++)
#pragma unroll
        for (int c = 0; c < 4; c++) o[rb][c] *= wgt;
#pragma unroll
    for (int w = 1; w < kPaWaves; w++) {
        float mw = ml_lds[w][0][j];
        float ww = mw == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mw - m_all);
        l_all += ww * ml_lds[w][1][j];
#pragma unroll
        for (int rb = 0; rb < RB; rb++)
#pragma unroll
            for (int c = 0; c < 4; c++) o[rb][c] += ww * o_lds[w - 1][rb * 4 + c][lane];
    }
    if (j >= group) return;
    // lane (qh = j, kb) holds O rows i = 4 kb + r of every c: dims dd = 64 rb + 4 i + c
    if (n_splits == 1) {   // the whole context was here: normalise and write the result
        const float inv = 1.0f / l_all;
        const int64_t item = (int64_t)seq * n_q_heads + qh;
#pragma unroll
        for (int rb = 0; rb < RB; rb++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                float4_t x = float4_t{o[rb][0][r], o[rb][1][r], o[rb][2][r], o[rb][3][r]} * inv;
                int w4 = 16 * rb + 4 * kb + r;       // float4 / packed-word index inside the head
                if (out_f32) *reinterpret_cast<float4_t *>(out_f32 + item * D + 4 * w4) = x;
                if (out_packed || out_q16) {
                    const uint32_t word = quant4<MODE>(x[0], x[1], x[2], x[3]);
                    if (out_packed) out_packed[item * DW + w4] = word;
                    if (out_q16) *reinterpret_cast<u32x2 *>(out_q16 + item * D + 4 * w4) = dequant4<MODE>(word);
                }
            }
        return;
    }
    float *my = scratch + ((int64_t)(seq * n_q_heads + qh) * n_splits + split) * (D + 2);
    if (kb == 0) { my[0] = m_all; my[1] = l_all; }
#pragma unroll
    for (int rb = 0; rb < RB; rb++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
            float4_t x = float4_t{o[rb][0][r], o[rb][1][r], o[rb][2][r], o[rb][3][r]};
            *reinterpret_cast<float4_t *>(my + 2 + 64 * rb + 4 * (4 * kb + r)) = x;
        }
}

// out[seq, qh, :] = sum_s 2^(m_s - m) O_s / sum_s 2^(m_s - m) l_s over the splits that hold tokens.
// One thread per 4 consecutive dims.  Splits are read eight at a time with every load issued
// before the first use (a loop of dependent loads would pay one memory latency per split).
template <int D, int MODE>
__global__ __launch_bounds__(256) void paged_attn_merge_kernel(const float *__restrict__ scratch,
                                                              const int32_t *__restrict__ ctx_lens,
                                                              float *__restrict__ out_f32,
                                                              uint32_t *__restrict__ out_packed,
                                                              _Float16 *__restrict__ out_q16, int n_items,
                                                              int n_q_heads, int n_splits, int max_ctx) {
    constexpr int DW = D / 4;
    constexpr int G = 8;
    const int gid = blockIdx.x * 256 + threadIdx.x;
    const int item = gid / DW, w4 = gid % DW;      // item = seq * n_q_heads + qh
    if (item >= n_items) return;
    // The context length and the partials of the first eight splits are requested together (the number
    // of splits that hold tokens is only needed to mask the values afterwards): one memory round trip
    // instead of two.  Partials of splits without tokens are whatever the buffer held and are replaced,
    // never used in arithmetic.
    const int ctx_raw = ctx_lens[item / n_q_heads];
    const float *base = scratch + (int64_t)item * n_splits * (D + 2);
    float ms[G], ls[G];
    float4_t os[G];
#pragma unroll
    for (int g = 0; g < G; g++) {
        const float *p = base + (int64_t)min(g, n_splits - 1) * (D + 2);
        ms[g] = p[0];
        ls[g] = p[1];
        os[g] = *reinterpret_cast<const float4_t *>(p + 2 + 4 * w4);
    }
    const int ctx = min(ctx_raw, max_ctx);
    const int used = min(n_splits, (ctx + kSplit - 1) / kSplit);
    float m = -INFINITY, l = 0.f;
    float4_t acc = float4_t{0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < used; s0 += G) {
        if (s0 > 0) {
#pragma unroll
            for (int g = 0; g < G; g++) {
                const float *p = base + (int64_t)min(s0 + g, n_splits - 1) * (D + 2);
                ms[g] = p[0];
                ls[g] = p[1];
                os[g] = *reinterpret_cast<const float4_t *>(p + 2 + 4 * w4);
            }
        }
#pragma unroll
        for (int g = 0; g < G; g++) {
            if (s0 + g >= used) {
                ms[g] = -INFINITY;
                ls[g] = 0.f;
                os[g] = float4_t{0.f, 0.f, 0.f, 0.f};
            }
        }
        float mg = m;
#pragma unroll
        for (int g = 0; g < G; g++) mg = fmaxf(mg, ms[g]);
        const float keep = m == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m - mg);
        l *= keep;
        acc *= keep;
#pragma unroll
        for (int g = 0; g < G; g++) {
            const float w = ms[g] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(ms[g] - mg);
            l += w * ls[g];
            acc += w * os[g];
        }
        m = mg;
    }
    if (used > 0) acc = acc * (1.0f / l);
    if (out_f32) *reinterpret_cast<float4_t *>(out_f32 + (int64_t)item * D + 4 * w4) = acc;
    if (out_packed || out_q16) {
        const uint32_t word = quant4<MODE>(acc[0], acc[1], acc[2], acc[3]);
        if (out_packed) out_packed[(int64_t)item * DW + w4] = word;
        if (out_q16) *reinterpret_cast<u32x2 *>(out_q16 + (int64_t)item * D + 4 * w4) = dequant4<MODE>(word);
    }
}

template <int D, int MODE>
static int launch_paged(const void *q, const void *kc, const void *vc, const void *bt, const void *cl, float *out_f32,
                        uint32_t *out_packed, _Float16 *out_q16, void *scratch, int64_t n_seq, int64_t n_q_heads, int64_t n_kv_heads,
                        int64_t block_size, int64_t max_blocks, int64_t n_blocks, int64_t max_ctx, float scale, hipStream_t s) {
    int n_splits = (int)((max_ctx + kSplit - 1) / kSplit);
    if (n_splits < 1) n_splits = 1;
    int64_t blocks = n_seq * n_kv_heads * n_splits;
    FEATHER_CHECK(blocks < (1ll << 31), FEATHER_ESHAPE, "feather_paged_attn_fp8: grid too large");
    int bs_shift = -1;
    for (int sh = 0; sh < 31; sh++)
        if ((1ll << sh) == block_size) bs_shift = sh;
    const float log2e = 1.4426950408889634f;
    if (bs_shift >= 2)
        hipLaunchKernelGGL((paged_attn_split_kernel<D, MODE, true>), dim3((unsigned)blocks), dim3(kPaThreads), 0, s,
                           (const int32_t *)cl, (const int32_t *)bt, (const uint32_t *)q, (const uint32_t *)kc,
                           (const uint32_t *)vc, (int)n_q_heads, (int)n_kv_heads, (int)block_size, (int)max_blocks, n_splits,
                           (int)max_ctx, scale * log2e, (float *)scratch, out_f32, out_packed, out_q16, (uint32_t)(n_blocks - 1),
                           (const float *)nullptr, 0, (int64_t)0, (const float *)nullptr, (uint32_t *)nullptr, (uint32_t *)nullptr);
    else
        hipLaunchKernelGGL((paged_attn_split_kernel<D, MODE, false>), dim3((unsigned)blocks), dim3(kPaThreads), 0, s,
                           (const int32_t *)cl, (const int32_t *)bt, (const uint32_t *)q, (const uint32_t *)kc,
                           (const uint32_t *)vc, (int)n_q_heads, (int)n_kv_heads, (int)block_size, (int)max_blocks, n_splits,
                           (int)max_ctx, scale * log2e, (float *)scratch, out_f32, out_packed, out_q16, (uint32_t)(n_blocks - 1),
                           (const float *)nullptr, 0, (int64_t)0, (const float *)nullptr, (uint32_t *)nullptr, (uint32_t *)nullptr);
    int rc = check_launch("feather_paged_attn_fp8");
    if (rc != FEATHER_OK || n_splits == 1) return rc;
    int64_t threads = n_seq * n_q_heads * (D / 4);
    hipLaunchKernelGGL((paged_attn_merge_kernel<D, MODE>), dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s,
                       (const float *)scratch, (const int32_t *)cl, out_f32, out_packed, out_q16, (int)(n_seq * n_q_heads),
                       (int)n_q_heads, n_splits, (int)max_ctx);
    return check_launch("feather_paged_attn_fp8 (merge)");
}

bool paged_attn_fused_supported(int64_t n_seq, int64_t n_q_heads, int64_t n_kv_heads, int64_t d, int64_t block_size,
                                int64_t n_part) {
    bool pow2 = block_size >= 4 && block_size <= kSplit && (block_size & (block_size - 1)) == 0;
    return d == 64 && pow2 && n_seq <= kWave && n_part >= 1 &&
           (n_q_heads / n_kv_heads + 2) * n_part <= kFusedMaxPairs;
}

int64_t paged_attn_plan_ints(int64_t n_seq, int64_t block_size, int64_t max_ctx) {
    int64_t n_splits = (max_ctx + kSplit - 1) / kSplit;
    if (n_splits < 1) n_splits = 1;
    return n_seq * n_splits * (4 + kSplit / block_size);
}

int paged_attn_fused_launch(const int32_t *plan, const int32_t *ctx_after, void *k_cache, void *v_cache, const float *qkv,
                            int n_part, int64_t part_stride, const float *cs, uint32_t *out_packed, void *scratch,
                            int64_t n_seq, int64_t n_q_heads, int64_t n_kv_heads, int64_t block_size, int64_t max_blocks,
                            int64_t n_blocks, int64_t max_ctx, int mode, float scale, hipStream_t s) {
    int n_splits = (int)((max_ctx + kSplit - 1) / kSplit);
    if (n_splits < 1) n_splits = 1;
    const int64_t blocks = n_seq * n_kv_heads * n_splits;
    FEATHER_CHECK(blocks < (1ll << 31), FEATHER_ESHAPE, "feather_decode_step: attention grid too large");
    const float log2e = 1.4426950408889634f;
#define FEATHER_PAF(MM)                                                                                                \
    hipLaunchKernelGGL((paged_attn_split_kernel<64, MM, true, true>), dim3((unsigned)blocks), dim3(kPaThreads), 0, s, plan, \
                       (const int32_t *)nullptr, (const uint32_t *)nullptr, (const uint32_t *)k_cache,                 \
                       (const uint32_t *)v_cache, (int)n_q_heads, (int)n_kv_heads, (int)block_size, (int)max_blocks,   \
                       n_splits, (int)max_ctx, scale * log2e, (float *)scratch, (float *)nullptr, out_packed,         \
                       (_Float16 *)nullptr, (uint32_t)(n_blocks - 1), qkv, n_part, part_stride, cs, (uint32_t *)k_cache, \
                       (uint32_t *)v_cache)
    if (mode == FEATHER_E5M2) FEATHER_PAF(FEATHER_E5M2); else FEATHER_PAF(FEATHER_E4M3);
#undef FEATHER_PAF
    int rc = check_launch("feather_decode_step (attention)");
    if (rc != FEATHER_OK || n_splits == 1) return rc;
    const int64_t threads = n_seq * n_q_heads * (64 / 4);
#define FEATHER_PAM(MM)                                                                                                \
    hipLaunchKernelGGL((paged_attn_merge_kernel<64, MM>), dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s,   \
                       (const float *)scratch, ctx_after, (float *)nullptr, out_packed, (_Float16 *)nullptr,          \
                       (int)(n_seq * n_q_heads), (int)n_q_heads, n_splits, (int)max_ctx)
    if (mode == FEATHER_E5M2) FEATHER_PAM(FEATHER_E5M2); else FEATHER_PAM(FEATHER_E4M3);
#undef FEATHER_PAM
    return check_launch("feather_decode_step (attention merge)");
}

int paged_attn_launch(const void *q, const void *k_cache, const void *v_cache, const void *block_tables,
                      const void *ctx_lens, float *out_f32, uint32_t *out_packed, _Float16 *out_q16, void *scratch,
                      int64_t n_seq,
                      int64_t n_q_heads, int64_t n_kv_heads, int64_t d, int64_t block_size, int64_t max_blocks,
                      int64_t n_blocks, int64_t max_ctx, int mode, float scale, hipStream_t s) {
#define FEATHER_PA(DD, MM)                                                                                           \
    return launch_paged<DD, MM>(q, k_cache, v_cache, block_tables, ctx_lens, out_f32, out_packed, out_q16, scratch,  \
                                n_seq, n_q_heads, n_kv_heads, block_size, max_blocks, n_blocks, max_ctx, scale, s)
    if (mode == FEATHER_E5M2) {
        if (d == 64) FEATHER_PA(64, FEATHER_E5M2);
        if (d == 128) FEATHER_PA(128, FEATHER_E5M2);
        if (d == 256) FEATHER_PA(256, FEATHER_E5M2);
        FEATHER_PA(512, FEATHER_E5M2);
    }
    if (d == 64) FEATHER_PA(64, FEATHER_E4M3);
    if (d == 128) FEATHER_PA(128, FEATHER_E4M3);
    if (d == 256) FEATHER_PA(256, FEATHER_E4M3);
    FEATHER_PA(512, FEATHER_E4M3);
#undef FEATHER_PA
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
                                      const void *ctx_lens, void *out_f32, void *out_packed, void *scratch, int64_t n_seq,
                                      int64_t n_q_heads, int64_t n_kv_heads, int64_t d, int64_t block_size,
                                      int64_t max_blocks, int64_t n_blocks, int64_t max_ctx, int mode, float scale,
                                      void *stream) {
    const char *me = "feather_paged_attn_fp8";
    FEATHER_CHECK(mode == FEATHER_E5M2 || mode == FEATHER_E4M3, FEATHER_EMODE, "%s: mode %d not supported", me, mode);
    FEATHER_CHECK(n_seq >= 0 && n_q_heads > 0 && n_kv_heads > 0 && block_size > 0 && max_blocks >= 0 && max_ctx >= 0,
                  FEATHER_EINVAL, "%s: bad shape", me);
    FEATHER_CHECK(n_blocks >= 1 && n_blocks < (1ll << 31), FEATHER_EINVAL, "%s: n_blocks=%lld: the cache must hold at least one block",
                  me, (long long)n_blocks);
    FEATHER_CHECK(n_q_heads % n_kv_heads == 0, FEATHER_ESHAPE, "%s: n_q_heads=%lld not a multiple of n_kv_heads=%lld",
                  me, (long long)n_q_heads, (long long)n_kv_heads);
    FEATHER_CHECK(n_q_heads / n_kv_heads <= 16, FEATHER_ESHAPE, "%s: at most 16 query heads per KV head", me);
    FEATHER_CHECK(d == 64 || d == 128 || d == 256 || d == 512, FEATHER_ESHAPE,
                  "%s: head dim %lld not supported (64, 128, 256, 512)", me, (long long)d);
    FEATHER_CHECK(max_ctx <= max_blocks * block_size, FEATHER_ESHAPE, "%s: max_ctx exceeds the block table", me);
    FEATHER_CHECK(scale > 0.f, FEATHER_EINVAL, "%s: scale must be positive (the running maximum is kept on raw scores)", me);
    if (n_seq == 0) return FEATHER_OK;
    FEATHER_CHECK(q && k_cache && v_cache && block_tables && ctx_lens && scratch, FEATHER_EINVAL, "%s: null pointer", me);
    FEATHER_CHECK(out_f32 || out_packed, FEATHER_EINVAL, "%s: no output (out_f32 and out_packed are both null)", me);
    FEATHER_CHECK(aligned(q, 8) && aligned(k_cache, 16) && aligned(v_cache, 16) && aligned(out_f32, 16) &&
                      aligned(out_packed, 4) && aligned(scratch, 16) && aligned(block_tables, 4) && aligned(ctx_lens, 4),
                  FEATHER_EINVAL, "%s: misaligned pointer", me);
    return paged_attn_launch(q, k_cache, v_cache, block_tables, ctx_lens, (float *)out_f32, (uint32_t *)out_packed, nullptr,
                             scratch, n_seq, n_q_heads, n_kv_heads, d, block_size, max_blocks, n_blocks, max_ctx, mode, scale,
                             (hipStream_t)stream);
}

// ---- the same attention for callers that cannot allocate -------------------------------------
// The split partials live in a file-scope device array instead of a caller-supplied buffer.  Every
// device that loads the library holds its own copy of the array at its own address, which
// hipGetSymbolAddress returns for the current device; host code only ever uses that address (the
// array's name is a host-side handle, not device memory).
namespace feather {

static __device__ __align__(256) unsigned char g_pa_static_scratch[FEATHER_PAGED_ATTN_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
static void *g_pa_static_ptr[kMaxDevices];   // device address of the array, per device; set once
static std::mutex g_pa_static_mutex;

static int pa_static_scratch(void **out, const char *me) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    FEATHER_CHECK(e == hipSuccess, FEATHER_ELAUNCH, "%s: hipGetDevice: %s", me, hipGetErrorString(e));
    FEATHER_CHECK(dev >= 0 && dev < kMaxDevices, FEATHER_EINVAL, "%s: device index %d outside 0..%d", me, dev,
                  kMaxDevices - 1);
    std::lock_guard<std::mutex> lock(g_pa_static_mutex);
    if (!g_pa_static_ptr[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(g_pa_static_scratch));
        FEATHER_CHECK(e == hipSuccess && p, FEATHER_ELAUNCH, "%s: hipGetSymbolAddress: %s", me, hipGetErrorString(e));
        g_pa_static_ptr[dev] = p;
    }
    *out = g_pa_static_ptr[dev];
    return FEATHER_OK;
}

}  // namespace feather

extern "C" int feather_paged_attn_fp8_static(const void *q, const void *k_cache, const void *v_cache,
                                             const void *block_tables, const void *ctx_lens, void *out_f32,
                                             void *out_packed, int64_t n_seq, int64_t n_q_heads, int64_t n_kv_heads,
                                             int64_t d, int64_t block_size, int64_t max_blocks, int64_t n_blocks,
                                             int64_t max_ctx, int mode, float scale, void *stream) {
    const char *me = "feather_paged_attn_fp8_static";
    const int64_t need = feather_paged_attn_scratch_bytes(n_seq, n_q_heads, d, max_ctx);
    FEATHER_CHECK(need <= (int64_t)FEATHER_PAGED_ATTN_STATIC_SCRATCH_BYTES, FEATHER_ESHAPE,
                  "%s: the split partials of this problem need %lld bytes, the built-in buffer holds %lld "
                  "(n_seq * n_q_heads * ceil(max_ctx / 512) * (d + 2) * 4); use feather_paged_attn_fp8 with a "
                  "caller-owned scratch",
                  me, (long long)need, (long long)FEATHER_PAGED_ATTN_STATIC_SCRATCH_BYTES);
    void *scratch = nullptr;
    if (n_seq > 0) {
        int rc = pa_static_scratch(&scratch, me);
        if (rc != FEATHER_OK) return rc;
    }
    // nothing in the buffer has to start at zero: the merge reads only the partials of splits that
    // hold tokens, and the split kernel of the same call writes exactly those
    return feather_paged_attn_fp8(q, k_cache, v_cache, block_tables, ctx_lens, out_f32, out_packed, scratch, n_seq,
                                  n_q_heads, n_kv_heads, d, block_size, max_blocks, n_blocks, max_ctx, mode, scale, stream);
}
