// Flash-attention forward on FP8-packed Q/K/V (prefill): fixed-length heads, or variable-length
// sequences packed back to back with an optional causal mask.
//
// Two kernels: flash_attn_kernel (this comment; head dims 128, 256, 512) on the 16x16x32 matrix
// instructions, and flash_attn64_wide_kernel (head dim 64, further down) on the 32x32 ones, which
// shares the work split, the staging scheme and the numerics and documents what differs.
//
// Work split.  One workgroup (WAVES waves, 4 or 8) owns a tile of 16*QB*WAVES/KSPLIT
// queries of one head; each wave owns 16*QB of them for the whole key loop (with KSPLIT = 2 two
// waves share them and each scores one half of the keys of every tile).  Keys/values are
// streamed in tiles of BN keys: the PACKED tile is fetched from global memory
// into registers two tiles ahead (so HBM/L2 latency overlaps the MFMA work of
// the tiles before it), decoded to fp16 on its way into the other LDS buffer one tile
// ahead, and read from LDS as MFMA operands by every wave.
//
// Matrix cores.  Everything is computed transposed so that one lane keeps one
// query for the whole kernel:
//     S^T[key, q] = K[key, :] . Q[q, :]     v_mfma_f32_16x16x32_f16, A = K tile
//     O^T[dd, q] += V^T[dd, key] P^T[key, q]  same instruction, A = V^T tile
// In the 16x16 accumulator layout lane l holds column l % 16 (the query) and
// rows 4 * (l / 16) + {0..3}; the B operand of the next MFMA wants, for the
// same column, 8 consecutive k-slots per lane.  The two layouts are matched by
// permuting the key order in which V^T is written to LDS, so the softmax
// output feeds the second MFMA straight from registers: no shuffle, no LDS
// round trip for P.  Row maxima need one exchange across the 4 lanes that
// share a query (a row swap and a half-wave swap); the row sums (softmax denominators) are
// accumulated by one more MFMA per step whose A operand is a constant block of
// ones, so they cost no vector-ALU work.
//
// E5M2 is the matrix core's bf8 operand format, so in that mode S^T runs on
// v_mfma_f32_16x16x32_bf8_bf8 straight from the packed K and Q bytes (no decode
// of K, half the LDS bytes; the instruction takes the same 16 cycles as the fp16
// one, as SQ_VALU_MFMA_BUSY_CYCLES shows); the products are the same
// exact fp16 x fp16 products, accumulated in fp32.
//
// Numerics follow the reference kernel (feather/routines/attention.py:24-108):
// fp16 x fp16 products accumulated in fp32, scores scaled in fp32, online
// softmax in fp32 (computed as 2^x with log2(e) folded into the scale), P
// rounded to fp16 before P.V, fp32 output.  One difference inside the stated
// tolerance: the denominator sums the fp16-rounded P (the values that multiply
// V) where the reference sums P before rounding.  The point the exponentials
// refer to is a running maximum that is raised lazily (see softmax_block): the
// quotient O / l does not depend on it.
#include <type_traits>
#include "common.h"

namespace feather {

typedef float float2v_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float4_t mfma16(half8_t a, half8_t b, float4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}

// 8 codes (two packed words) -> 8 fp16
template <int MODE>
__device__ __forceinline__ half8_t dec8(uint32_t w0, uint32_t w1) {
    u32x4 r;
    uint32_t a, b;
    dec_word<MODE>(w0, a, b);
    r.x = a; r.y = b;
    dec_word<MODE>(w1, a, b);
    r.z = a; r.w = b;
    return __builtin_bit_cast(half8_t, r);
}

// QB  16-query blocks per wave (a workgroup owns 16 * QB * WAVES queries)
// SB  query blocks scored together (SB divides QB)
// BN  keys per tile
// OCC workgroups per CU the register budget is sized for (2 keeps every MFMA
//     accumulator in architectural VGPRs, so rescaling needs no AGPR copies)
// VC  variable-length / causal variant: every head holds total_rows rows, sequence s of
//     cu_seqlens (n_seq + 1 row offsets) occupies rows [cu[s], cu[s+1]) of every head and
//     attends only to itself; with causal != 0 query i sees keys 0..i of its sequence.
//     tiles_per_head = n_seq * tiles_per_seq; L, keys_scored and mask_tail are not used.
// KSPLIT  wave groups that share the workgroup's queries: group g scores keys [g, g + 1) * BN / KSPLIT of
//         every tile with its own running maximum, sum and accumulators, merged through LDS at the
//         end (finer work items for grids that would leave CUs idle; every wave is busy in every
//         tile, where groups that took whole tiles in turn idled at the tile barrier while the other
//         one worked).  A group of 16 keys multiplies P and V on the 16x16x16 MFMA.  Group 0 always has
//         key 0, so its running maximum is finite whenever the sequence has a key; not combined with
//         the causal mask.
// ZS  the key loop is cut into n_kchunks ranges of kchunk_keys keys (a multiple of BN, every range starting
//     below L) that go to separate workgroups, for grids that would leave most CUs idle: workgroup
//     (tile, z) scores range z and writes its unnormalised accumulators, reference point and row sum to
//     `part` ([z][row][D] floats, then [z][row] pairs (m, l)); flash_attn_merge_kernel combines the ranges.
//     Fixed-length heads only.
template <int D, int MODE, int QB, int SB, int BN, int OCC, bool VC, int WAVES = 4, int KSPLIT = 1, bool ZS = false>
__global__ __launch_bounds__(64 * WAVES, OCC) void flash_attn_kernel(
    const uint32_t *__restrict__ q, const uint32_t *__restrict__ k, const uint32_t *__restrict__ v,
    float *__restrict__ out, int L, int n_heads, int kv_group, int tiles_per_head, float scale_log2e,
    int keys_scored, int mask_tail, const int32_t *__restrict__ cu_seqlens, int tiles_per_seq, int total_rows,
    int causal, float *__restrict__ part, int kchunk_keys, int n_kchunks) {
    static_assert(!(ZS && VC), "key ranges over workgroups are for fixed-length heads");
    constexpr int DW = D / 4;              // packed words per row
    // E5M2 codes ARE the bf8 operand format of the matrix core: the score product runs on
    // v_mfma_f32_16x16x32_bf8_bf8 straight from the packed bytes (exact products, fp32 accumulation,
    // no decode, half the LDS bytes for K); V still goes through fp16
    // because P is an fp16 operand (the reference rounds P to fp16, attention.py:90).
    constexpr bool BF8 = MODE == FEATHER_E5M2;
    constexpr int KS = BF8 ? (D + 16) / 2 : D + 8;   // K row pitch in LDS, in fp16 units (bf8: D + 16 bytes)
    constexpr int VS = BN;                 // fp16 per V^T row in LDS (16-byte chunks XOR-swizzled by row)
    constexpr int CH = BN / 8;             // 16-byte chunks per V^T row
    constexpr int kAttnThreads = 64 * WAVES;
    constexpr int QWAVES = WAVES / KSPLIT; // waves that own distinct queries
    constexpr int QT = 16 * QB * QWAVES;   // queries per workgroup
    constexpr int UNITS = BN * D / 16;     // 16-code units of a K (or V) tile
    constexpr int NU = UNITS >= kAttnThreads ? UNITS / kAttnThreads : 1;  // units per thread per tile
    // a tile with fewer units than threads is staged by the first UNITS threads (whole waves)
    constexpr bool ALL_STAGE = UNITS >= kAttnThreads;
    static_assert(UNITS % 64 == 0 && (ALL_STAGE ? UNITS % kAttnThreads == 0 : true), "tile / workgroup mismatch");
    constexpr int DB = D / 16, STEPS = D / 32;
    constexpr int GBN = BN / KSPLIT;       // keys of a tile that one key group scores
    static_assert(GBN == 16 || GBN % 32 == 0, "a key group scores 16 keys or whole groups of 32");
    constexpr bool K16 = GBN == 16;
    constexpr int GKB16 = GBN / 16, GKB32 = K16 ? 1 : GBN / 32;
    using pfrag_t = std::conditional_t<K16, half4_t, half8_t>;   // P of one 16- or 32-key MFMA step

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    // two buffers of (K tile, V^T tile): tile i+1 is written while tile i is being read
    constexpr int kBufHalfs = BN * KS + D * VS;
    _Float16 *const lds = reinterpret_cast<_Float16 *>(smem);
    // V^T swizzle: chunk c of row r lives at chunk c ^ swz(r).  Eight lanes that read the same
    // chunk of eight consecutive rows, and the lanes that write the same key group of rows four
    // apart, then fall on different LDS banks.
    auto swz = [](int row) { return (row ^ (row >> 2)) & (CH - 1); };

    // XCD-aware block mapping: consecutive workgroup ids go round-robin over the 8
    // XCDs (each with its own L2); remap so that an XCD works through a contiguous
    // range of (head, tile) pairs and the K/V of a head stay in one L2.
    int bid = blockIdx.x;
    const int total = gridDim.x;
    if (total % 8 == 0) bid = (bid % 8) * (total / 8) + bid / 8;
    int zchunk = 0;
    if constexpr (ZS) {   // the key ranges of a query tile are neighbours in this order: same XCD, same L2
        zchunk = bid % n_kchunks;
        bid /= n_kchunks;
    }
    const int head = bid / tiles_per_head;
    int tile = bid % tiles_per_head;
    const int kv_head = head / kv_group;
    int64_t q_row0 = (int64_t)head * L, kv_row0 = (int64_t)kv_head * L;   // first row of this head's sequence
    if constexpr (VC) {
        const int seq = tile / tiles_per_seq;
        tile = tile % tiles_per_seq;
        if (causal) tile = tiles_per_seq - 1 - tile;          // the tiles with the longest key loops start first
        const int r0 = cu_seqlens[seq];
        L = cu_seqlens[seq + 1] - r0;
        if (tile * QT >= L) return;                    // past the end of this sequence (whole workgroup)
        q_row0 = (int64_t)head * total_rows + r0;
        kv_row0 = (int64_t)kv_head * total_rows + r0;
        mask_tail = 1;
        const int last_key = causal ? min(L, (tile + 1) * QT) : L;
        keys_scored = (last_key + BN - 1) / BN * BN;
    }

    const int tid = threadIdx.x, lane = tid & 63, wave = wave_id();
    const int j = lane & 15, kb = lane >> 4;
    const int qwave = KSPLIT == 1 ? wave : wave % QWAVES, kgroup = KSPLIT == 1 ? 0 : wave / QWAVES;
    const int q0 = tile * QT + qwave * (16 * QB);

    const uint32_t *qh = q + q_row0 * DW;
    const uint32_t *kh = k + kv_row0 * DW;
    const uint32_t *vh = v + kv_row0 * DW;

    // ---- Q fragments (B operand of S^T), resident in registers
    half8_t qf[BF8 ? 1 : QB][BF8 ? 1 : STEPS];
    long qf8[BF8 ? QB : 1][BF8 ? STEPS : 1];   // bf8: the raw 8 codes
#pragma unroll
    for (int b = 0; b < QB; b++) {
        int row = q0 + 16 * b + j;
#pragma unroll
        for (int s = 0; s < STEPS; s++) {
            u32x2 w = u32x2{0, 0};
            if (row < L) w = *reinterpret_cast<const u32x2 *>(qh + (int64_t)row * DW + 8 * s + 2 * kb);
            if constexpr (BF8) qf8[b][s] = __builtin_bit_cast(long, w);
            else qf[b][s] = dec8<MODE>(w.x, w.y);
        }
    }

    // o[b][DB] is one extra accumulator block whose A operand is constant: rows 0, 4, 8, 12
    // of it are all ones, so element [0] of every lane accumulates l = sum_k P[k, q] of the
    // lane's query on the matrix core (the softmax denominator costs no VALU adds).  The
    // summands are the fp16-rounded P that also multiply V.
    float4_t o[QB][DB + 1];
    float m_run[QB];
#pragma unroll
    for (int b = 0; b < QB; b++) {
        m_run[b] = -INFINITY;
#pragma unroll
        for (int d = 0; d <= DB; d++) o[b][d] = float4_t{0.f, 0.f, 0.f, 0.f};
    }
    constexpr float kLazy = 8.f;
    const float lazy_raw = kLazy / scale_log2e;   // the same margin in raw-score units
    const _Float16 one_or_zero = (j & 3) == 0 ? (_Float16)1 : (_Float16)0;
    const half8_t ones = {one_or_zero, one_or_zero, one_or_zero, one_or_zero,
                          one_or_zero, one_or_zero, one_or_zero, one_or_zero};

    // ---- register staging of the next packed K / V tile
    u32x4 kreg[NU];
    uint32_t vreg[NU][4];
    auto prefetch = [&](int key0) {
        if (!ALL_STAGE && tid >= UNITS) return;
        // The tile's first row is wave-uniform (scalar base); the lane adds a 32-bit byte offset inside
        // the tile, re-derived from the thread index on every call: the index is made opaque here,
        // otherwise base + offset is hoisted out of the key loop as one 64-bit address per load and
        // those register pairs are what gets spilled at d = 512 (and a spill reload between two global
        // loads waits for the first one).
        const int row0 = __builtin_amdgcn_readfirstlane(key0);
        const char *kt = reinterpret_cast<const char *>(kh + (int64_t)row0 * DW);
        const char *vt = reinterpret_cast<const char *>(vh + (int64_t)row0 * DW);
        int t = tid;
        asm volatile("" : "+v"(t));
#pragma unroll
        for (int i = 0; i < NU; i++) {
            const int u = t + kAttnThreads * i;
            const int krel = u / (D / 16), c16 = u % (D / 16);
            kreg[i] = u32x4{0, 0, 0, 0};
            if (key0 + krel < L) kreg[i] = *reinterpret_cast<const u32x4 *>(kt + (uint32_t)(krel * D + 16 * c16));
            const int ddw = u % DW, kg = u / DW;
            const uint32_t voff = (uint32_t)(4 * kg * D + 4 * ddw);
#pragma unroll
            for (int r = 0; r < 4; r++)
                vreg[i][r] = key0 + 4 * kg + r < L ? *reinterpret_cast<const uint32_t *>(vt + voff + (uint32_t)(r * D)) : 0u;
        }
    };
    auto stage = [&](int buf) {
        _Float16 *k_lds = lds + buf * kBufHalfs;
        _Float16 *vt_lds = k_lds + BN * KS;
        if (!ALL_STAGE && tid >= UNITS) return;
#pragma unroll
        for (int i = 0; i < NU; i++) {
            int u = tid + kAttnThreads * i;
            // K: 16 codes of one key -> 16 fp16, row-major [key][d]
            int key = u / (D / 16), c16 = u % (D / 16);
            if constexpr (BF8) {
                *reinterpret_cast<u32x4 *>(reinterpret_cast<unsigned char *>(k_lds) + key * (2 * KS) + 16 * c16) = kreg[i];
            } else {
                half8_t lo = dec8<MODE>(kreg[i].x, kreg[i].y), hi = dec8<MODE>(kreg[i].z, kreg[i].w);
                half8_t *kd = reinterpret_cast<half8_t *>(k_lds + key * KS + 16 * c16);
                kd[0] = lo;
                kd[1] = hi;
            }
            // V: 4 keys x 4 dims -> V^T[dd][pos], key order permuted inside each
            // group of 32 so that slot (kb, 4a + r) holds key 16a + 4kb + r
            int ddw = u % DW, kg = u / DW;
            int ko = 4 * kg, o32 = ko & 31;
            int pos = (ko & ~31) + ((o32 & 15) >> 2) * 8 + (o32 >> 4) * 4;
            uint32_t lo2[4], hi2[4];
            if constexpr (MODE == FEATHER_E5M2) {
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    // halfs (key r, key r+1) of dim 4*ddw + c: byte c of each word, placed as the high byte
                    uint32_t sel = 0x000c000cu | ((uint32_t)c << 8) | ((uint32_t)(4 + c) << 24);
                    lo2[c] = perm(vreg[i][1], vreg[i][0], sel);
                    hi2[c] = perm(vreg[i][3], vreg[i][2], sel);
                }
            } else {
                uint32_t p01[4], p23[4];
#pragma unroll
                for (int r = 0; r < 4; r++) dec_word<MODE>(vreg[i][r], p01[r], p23[r]);
                lo2[0] = perm(p01[1], p01[0], 0x05040100u); hi2[0] = perm(p01[3], p01[2], 0x05040100u);
                lo2[1] = perm(p01[1], p01[0], 0x07060302u); hi2[1] = perm(p01[3], p01[2], 0x07060302u);
                lo2[2] = perm(p23[1], p23[0], 0x05040100u); hi2[2] = perm(p23[3], p23[2], 0x05040100u);
                lo2[3] = perm(p23[1], p23[0], 0x07060302u); hi2[3] = perm(p23[3], p23[2], 0x07060302u);
            }
#pragma unroll
            for (int c = 0; c < 4; c++) {
                int row = 4 * ddw + c;
                *reinterpret_cast<u32x2 *>(vt_lds + row * VS + (((pos >> 3) ^ swz(row)) << 3) + (pos & 4)) =
                    u32x2{lo2[c], hi2[c]};
            }
        }
    };

    const int key_begin = ZS ? zchunk * kchunk_keys : 0;
    const int key_end = ZS ? min(keys_scored, key_begin + kchunk_keys) : keys_scored;
    prefetch(key_begin);
    stage(0);
    if (key_begin + BN < key_end) prefetch(key_begin + BN);
    __syncthreads();
    int cur = 0;
    for (int key0 = key_begin; key0 < key_end; key0 += BN, cur ^= 1) {
        // tile i+1 goes to the other buffer (its readers passed the barrier that ended the previous
        // iteration) and tile i+2 into registers, both off the critical path of this tile's math
        // At d = 512 the two waves that share a SIMD (w and w + 4 of an eight-wave workgroup) run this
        // in opposite order, math first for the second one: staging is vector-ALU work, the math is LDS
        // reads and MFMAs, and in lock step the pair wants the same unit at the same time (-2..5 % time;
        // the narrower heads lose 1-4 % with it, their staging is a smaller share of a tile).
        const bool math_first = WAVES == 8 && D >= 512 && wave >= 4;
        if (!math_first && key0 + BN < key_end) {
            stage(cur ^ 1);
            if (key0 + 2 * BN < key_end) prefetch(key0 + 2 * BN);
        }
        const _Float16 *k_lds = lds + cur * kBufHalfs;
        const _Float16 *vt_lds = k_lds + BN * KS;
        const bool ragged = mask_tail && key0 + BN > L;   // only the last tile can hold masked keys
        bool diag = false, skip = false;
        if constexpr (VC) {
            diag = causal && key0 + BN - 1 > q0;          // some key of the tile lies past the wave's first query
            skip = causal && key0 > q0 + 16 * QB - 1;     // every key lies past the wave's last query
        }
        if constexpr (KSPLIT > 1) skip = skip || (mask_tail && key0 + kgroup * GBN >= L);   // no key of this group's part exists
        if (!skip) {

        // ---- online softmax of one 16-query block, one query per lane column.  The running maximum
        // is kept on the raw scores; scale * log2(e) is folded into one fma per score:
        // p = 2^(s * c - m * c).  Leaves P (fp16) in pb and rescales the block's accumulators if needed.
        auto softmax_block = [&](int qb, float4_t (&sb)[GKB16], pfrag_t (&pb)[GKB32]) {
            if (ragged || diag) {
                int last = diag ? min(L - 1, q0 + 16 * qb + j) : L - 1;   // last visible key
                // opaque to the optimiser from here on: otherwise the 16 key-index compares below
                // are hoisted out of this rarely taken branch and run for every tile
                asm volatile("" : "+v"(last));
                // key 16 c + 4 kb + r of the group's part of the tile is hidden if 16 c + r > rel
                const int rel = last - key0 - kgroup * GBN - 4 * kb;
#pragma unroll
                for (int c = 0; c < GKB16; c++)
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        if (16 * c + r > rel) sb[c][r] = -INFINITY;
            }
            float mx = max3_raw(sb[0][0], sb[0][1], sb[0][2]);
            mx = max_raw(mx, sb[0][3]);
#pragma unroll
            for (int c = 1; c < GKB16; c++) {
                mx = max3_raw(mx, sb[c][0], sb[c][1]);
                mx = max3_raw(mx, sb[c][2], sb[c][3]);
            }
            mx = max_xor32(max_xor16(mx));   // over the four lanes that share the query
            // The reference point of the exponentials is only raised when some query of the block exceeds it by
            // more than kLazy binary orders of magnitude (P then lies in (0, 2^kLazy], which fp16 holds with the
            // same relative precision; O / l does not depend on the reference point): the rescaling of the
            // block's 4 (DB + 1) accumulator registers, more than its whole softmax from d = 256 on, runs for
            // a few tiles per sequence instead of for a third of them.
            const float m_old = m_run[qb];
            const bool raise = __builtin_amdgcn_ballot_w64(mx > m_old + lazy_raw) != 0;
            const float m_new = raise ? max_raw(m_old, mx) : m_old;
            const float mc = m_new * scale_log2e;
            if constexpr (K16) {
                half4_t p4;
#pragma unroll
                for (int r = 0; r < 4; r++)
                    p4[r] = (_Float16)__builtin_amdgcn_exp2f(__builtin_fmaf(sb[0][r], scale_log2e, -mc));
                pb[0] = p4;
            } else {
#pragma unroll
                for (int t = 0; t < GKB32; t++) {
                    half8_t p8;
#pragma unroll
                    for (int a = 0; a < 2; a++)
#pragma unroll
                        for (int r = 0; r < 4; r++) {
                            float e = __builtin_amdgcn_exp2f(__builtin_fmaf(sb[2 * t + a][r], scale_log2e, -mc));
                            p8[4 * a + r] = (_Float16)e;  // round to nearest even, as P.to(fp16)
                        }
                    pb[t] = p8;
                }
            }
            if (raise) {   // wave-uniform
                const float alpha = __builtin_amdgcn_exp2f((m_old - m_new) * scale_log2e);
                m_run[qb] = m_new;
#pragma unroll
                for (int d = 0; d <= DB; d++) o[qb][d] *= alpha;
            }
        };
        pfrag_t pf[QB][GKB32];
        const int kc0 = kgroup * GKB16;   // first 16-key block of this key group inside the tile
        // query blocks are scored SB at a time: the K fragments are re-used across the SB
        // blocks while only SB * GKB16 score tiles are live in registers
#pragma unroll
        for (int b0 = 0; b0 < QB; b0 += SB) {
            // ---- S^T = K Q^T (raw, unscaled scores)
            float4_t s[SB][GKB16];
#pragma unroll
            for (int c = 0; c < GKB16; c++) {
#pragma unroll
                for (int st = 0; st < STEPS; st++) {
                    if constexpr (BF8) {
                        const long kf = *reinterpret_cast<const long *>(reinterpret_cast<const unsigned char *>(k_lds) +
                                                                       (16 * (kc0 + c) + j) * (2 * KS) + 32 * st + 8 * kb);
#pragma unroll
                        for (int b = 0; b < SB; b++)
                            s[b][c] = __builtin_amdgcn_mfma_f32_16x16x32_bf8_bf8(
                                kf, qf8[b0 + b][st], st == 0 ? float4_t{0.f, 0.f, 0.f, 0.f} : s[b][c], 0, 0, 0);
                    } else {
                        half8_t kf = *reinterpret_cast<const half8_t *>(k_lds + (16 * (kc0 + c) + j) * KS + 32 * st + 8 * kb);
#pragma unroll
                        for (int b = 0; b < SB; b++)
                            s[b][c] = mfma16(kf, qf[b0 + b][st], st == 0 ? float4_t{0.f, 0.f, 0.f, 0.f} : s[b][c]);
                    }
                }
            }
            mfma_settle<SB * GKB16>(&s[0][0]);   // the softmax's first readers are asm statements
#pragma unroll
            for (int b = 0; b < SB; b++) softmax_block(b0 + b, s[b], pf[b0 + b]);
        }

        // ---- O^T += V^T P^T (and the row sums through the constant ones block)
        if constexpr (K16) {
            // keys 16 a + 4 kb + r of 32-key group t sit at slots 8 kb + 4 a + r of a V^T row: the four
            // keys of this lane are half a chunk
            const int t = kgroup / 2, a = kgroup % 2;
            const half4_t ones4 = {one_or_zero, one_or_zero, one_or_zero, one_or_zero};
#pragma unroll
            for (int d = 0; d < DB; d++) {
                half4_t vf = *reinterpret_cast<const half4_t *>(vt_lds + (16 * d + j) * VS +
                                                                (((4 * t + kb) ^ swz(16 * d + j)) << 3) + 4 * a);
#pragma unroll
                for (int b = 0; b < QB; b++) o[b][d] = __builtin_amdgcn_mfma_f32_16x16x16f16(vf, pf[b][0], o[b][d], 0, 0, 0);
            }
#pragma unroll
            for (int b = 0; b < QB; b++) o[b][DB] = __builtin_amdgcn_mfma_f32_16x16x16f16(ones4, pf[b][0], o[b][DB], 0, 0, 0);
        } else {
#pragma unroll
        for (int t = 0; t < GKB32; t++) {
#pragma unroll
            for (int d = 0; d < DB; d++) {
                half8_t vf = *reinterpret_cast<const half8_t *>(vt_lds + (16 * d + j) * VS +
                                                                (((4 * (kgroup * GKB32 + t) + kb) ^ swz(16 * d + j)) << 3));
#pragma unroll
                for (int b = 0; b < QB; b++) o[b][d] = mfma16(vf, pf[b][t], o[b][d]);
            }
#pragma unroll
            for (int b = 0; b < QB; b++) o[b][DB] = mfma16(ones, pf[b][t], o[b][DB]);
        }
        }
        }   // !skip
        if (math_first && key0 + BN < key_end) {
            stage(cur ^ 1);
            if (key0 + 2 * BN < key_end) prefetch(key0 + 2 * BN);
        }
        __syncthreads();  // tile i+1 is visible; every wave is done reading tile i
    }

    if constexpr (KSPLIT > 1) {
        // ---- merge the key groups: groups 1, 2, ... hand (m, O, l) to group 0 through LDS one after
        // the other (a fixed order of additions; the tile buffers are free: the loop ended with a
        // barrier), DCH accumulator blocks per pass
        constexpr int kLdsBytes = kBufHalfs * 2 * 2;
        constexpr int kPerBlock = QWAVES * QB * 64 * 16;                      // bytes of one accumulator block
        constexpr int DCH = (kLdsBytes - QWAVES * QB * 64 * 4) / kPerBlock < DB + 1
                                ? (kLdsBytes - QWAVES * QB * 64 * 4) / kPerBlock : DB + 1;
        static_assert(DCH >= 1, "no room for the merge");
        float *xm = reinterpret_cast<float *>(smem);                          // [QWAVES][QB][64]
        float4_t *xo = reinterpret_cast<float4_t *>(xm + QWAVES * QB * 64);   // [DCH][QWAVES][QB][64]
#pragma unroll
        for (int g = 1; g < KSPLIT; g++) {
            float w0[QB], w1[QB];
#pragma unroll
            for (int d0 = 0; d0 <= DB; d0 += DCH) {
                if (kgroup == g) {
#pragma unroll
                    for (int b = 0; b < QB; b++) {
                        if (d0 == 0) xm[(qwave * QB + b) * 64 + lane] = m_run[b];
#pragma unroll
                        for (int d = d0; d < d0 + DCH && d <= DB; d++)
                            xo[(((d - d0) * QWAVES + qwave) * QB + b) * 64 + lane] = o[b][d];
                    }
                }
                __syncthreads();
                if (kgroup == 0) {
#pragma unroll
                    for (int b = 0; b < QB; b++) {
                        if (d0 == 0) {
                            const float m1 = xm[(qwave * QB + b) * 64 + lane];
                            const float m = fmaxf(m_run[b], m1);
                            w0[b] = m_run[b] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f((m_run[b] - m) * scale_log2e);
                            w1[b] = m1 == -INFINITY ? 0.f : __builtin_amdgcn_exp2f((m1 - m) * scale_log2e);
                            m_run[b] = m;
                        }
#pragma unroll
                        for (int d = d0; d < d0 + DCH && d <= DB; d++)
                            o[b][d] = o[b][d] * w0[b] + xo[(((d - d0) * QWAVES + qwave) * QB + b) * 64 + lane] * w1[b];
                    }
                }
                // the next pass (of this group or the next one) overwrites the exchange area
                if (d0 + DCH <= DB || g + 1 < KSPLIT) __syncthreads();
            }
        }
        if (kgroup != 0) return;
    }

    if constexpr (ZS) {
        // ---- epilogue of a key range: unnormalised accumulators, reference point and row sum
        const int64_t rows_total = (int64_t)n_heads * L;
        float *ph = part + ((int64_t)zchunk * rows_total + q_row0) * D;
        float *ml = part + (int64_t)n_kchunks * rows_total * D + ((int64_t)zchunk * rows_total + q_row0) * 2;
#pragma unroll
        for (int b = 0; b < QB; b++) {
            int row = q0 + 16 * b + j;
            if (row < L) {
#pragma unroll
                for (int d = 0; d < DB; d++)
                    *reinterpret_cast<float4_t *>(ph + (int64_t)row * D + 16 * d + 4 * kb) = o[b][d];
                if (kb == 0) *reinterpret_cast<float2v_t *>(ml + (int64_t)row * 2) = float2v_t{m_run[b], o[b][DB][0]};
            }
        }
        return;
    }

    // ---- epilogue: finish the row sums, normalise, store [q][dd]
    float *oh = out + q_row0 * D;
#pragma unroll
    for (int b = 0; b < QB; b++) {
        const float l = o[b][DB][0];   // row 4 * kb of the ones block: the full sum over keys
        int row = q0 + 16 * b + j;
        if (row < L) {
#pragma unroll
            for (int d = 0; d < DB; d++) {
                *reinterpret_cast<float4_t *>(oh + (int64_t)row * D + 16 * d + 4 * kb) = o[b][d] / l;
            }
        }
    }
}

constexpr int kMaxKeyChunks = 8;

// Combines the Z key ranges of flash_attn_kernel<..., ZS = true> and flash_attn64_wide_kernel<..., ZS = true>:
// one thread per (row, four dims).  Range z of a row
// holds O_z = sum_k 2^((s_k - m_z) c) V_k and l_z = sum_k 2^((s_k - m_z) c); with m = max_z m_z the row is
// sum_z 2^((m_z - m) c) O_z / sum_z 2^((m_z - m) c) l_z, added in range order.
template <int Z>
__global__ __launch_bounds__(256) void flash_attn_merge_kernel(const float *__restrict__ part, float *__restrict__ out,
                                                               int64_t rows_total, int dq, float scale_log2e) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= rows_total * dq) return;
    const int64_t row = idx / dq;
    const float2v_t *ml = reinterpret_cast<const float2v_t *>(part + (int64_t)Z * rows_total * dq * 4);
    const float4_t *po = reinterpret_cast<const float4_t *>(part);
    float2v_t mlz[Z];
    float4_t oz[Z];
#pragma unroll
    for (int z = 0; z < Z; z++) {   // every load goes out before the first use
        mlz[z] = ml[z * rows_total + row];
        oz[z] = __builtin_nontemporal_load(po + z * rows_total * dq + idx);
    }
    float m = mlz[0][0];
#pragma unroll
    for (int z = 1; z < Z; z++) m = fmaxf(m, mlz[z][0]);
    float4_t acc = {0.f, 0.f, 0.f, 0.f};
    float l = 0.f;
#pragma unroll
    for (int z = 0; z < Z; z++) {
        const float w = mlz[z][0] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f((mlz[z][0] - m) * scale_log2e);
        acc += oz[z] * w;
        l += mlz[z][1] * w;
    }
    reinterpret_cast<float4_t *>(out)[idx] = acc / l;
}

// ---- d = 64, E5M2: the FP8-rate kernel -------------------------------------------------------------
// Same work split, staging and numerics as flash_attn_kernel<64, E5M2, ...> (a wave owns 64 queries,
// 64-key tiles, K staged as raw bytes, V^T as fp16), on the 32x32 matrix instructions:
//     S^T[32 keys, 32 q]  = v_mfma_f32_32x32x64_f8f6f4 (both operands BF8 = E5M2): the whole head dim in
//                           one instruction at the FP8 rate, 4 per tile where the 16x16x32 form needs 32;
//     O^T[32 dd, 32 q]   += v_mfma_f32_32x32x16_f16, 16 per tile.
// What it buys is vector-ALU issue time, which bounds this head dim: an MFMA holds the SIMD's vector
// issue for as long as its operands take to read (measured: 8 cycles for a 16x16x32 fp16 MFMA, 4 for
// the bf8 one, about the same 8 for a 32x32x16 that does twice the work), so 20 large MFMAs per tile
// block it for ~170 cycles where 72 small ones block it for ~450; a query is shared by two lanes
// instead of four (one cross-lane step per maximum instead of two), and the row sums are two-term dot
// products on the fp16 pairs of P (v_dot2_f32_f16, 32 per tile) instead of a constant-ones MFMA whose
// 32x32 form would cost 32 accumulator registers.
// Layouts (lane l, n = l % 32, h = l / 32): an MFMA operand row is [n]; operand bytes / halves are the
// k-slots 32 h .. 32 h + 31 (f8f6f4) or 8 h .. 8 h + 7 (f16); accumulator register r of a 32x32 block is
// row 8 (r / 4) + 4 h + r % 4, column n.  So a lane holds, for query n, the scores of keys
// 8 g + 4 h + {0..3} (g = 0..3) of each 32-key block, and registers 8 s .. 8 s + 7 are exactly the eight
// k-slots the second MFMA wants from this lane for the 16-key step s if V^T stores the keys of every
// group of 16 in the order 0 1 2 3 8 9 10 11 | 4 5 6 7 12 13 14 15.  (Both operands of the score MFMA take
// the same bytes of a row, so the order of the k-slots inside the instruction does not matter.)
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef int int8v_t __attribute__((ext_vector_type(8)));

template <int MODE, bool VC, int WAVES, int OCC, bool ZS = false>
__global__ __launch_bounds__(64 * WAVES, OCC) void flash_attn64_wide_kernel(
    const uint32_t *__restrict__ q, const uint32_t *__restrict__ k, const uint32_t *__restrict__ v,
    float *__restrict__ out, int L, int n_heads, int kv_group, int tiles_per_head, float scale_log2e,
    int keys_scored, int mask_tail, const int32_t *__restrict__ cu_seqlens, int tiles_per_seq, int total_rows,
    int causal, float *__restrict__ part, int kchunk_keys, int n_kchunks) {
    static_assert(!(ZS && VC), "key ranges over workgroups are for fixed-length heads");
    constexpr int D = 64, DW = 16, BN = 64;
    constexpr bool BF8 = MODE == FEATHER_E5M2;   // K and Q stay packed bytes; otherwise both are decoded to fp16
    constexpr int KP = (BF8 ? D : 2 * D) + 16;   // K row pitch in LDS, bytes
    constexpr int VS = BN;                 // fp16 per V^T row
    constexpr int kThreads = 64 * WAVES, QT = 64 * WAVES;
    constexpr int UNITS = BN * D / 16;     // 16-code units of a K (or V) tile: 256
    static_assert(UNITS <= kThreads && UNITS % 64 == 0, "the first UNITS threads stage a tile");
    constexpr int kBufBytes = BN * KP + D * VS * 2;

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    // V^T swizzle: 16-byte chunk c of row r lives at chunk c ^ swz(r).  The 16 lanes of a fragment read take
    // the same chunk of 16 consecutive rows (distinct bank groups for rows of equal parity need distinct
    // swz over r / 2 % 8); the writers of a wave take rows 4 apart (bits 2..5 of the row vary)
    auto swz = [](int row) { return ((row >> 1) & 7) ^ ((row >> 4) & 1); };

    int bid = blockIdx.x;
    const int total = gridDim.x;
    if (total % 8 == 0) bid = (bid % 8) * (total / 8) + bid / 8;   // an XCD works through contiguous (head, tile) pairs
    int zchunk = 0;
    if constexpr (ZS) {   // key ranges of a query tile (see flash_attn_kernel): neighbours in this order
        zchunk = bid % n_kchunks;
        bid /= n_kchunks;
    }
    const int head = bid / tiles_per_head;
    int tile = bid % tiles_per_head;
    const int kv_head = head / kv_group;
    int64_t q_row0 = (int64_t)head * L, kv_row0 = (int64_t)kv_head * L;
    if constexpr (VC) {
        const int seq = tile / tiles_per_seq;
        tile = tile % tiles_per_seq;
        if (causal) tile = tiles_per_seq - 1 - tile;          // the tiles with the longest key loops start first
        const int r0 = cu_seqlens[seq];
        L = cu_seqlens[seq + 1] - r0;
        if (tile * QT >= L) return;
        q_row0 = (int64_t)head * total_rows + r0;
        kv_row0 = (int64_t)kv_head * total_rows + r0;
        mask_tail = 1;
        const int last_key = causal ? min(L, (tile + 1) * QT) : L;
        keys_scored = (last_key + BN - 1) / BN * BN;
    }

    const int tid = threadIdx.x, lane = tid & 63, wave = wave_id();
    const int n = lane & 31, h = lane >> 5;
    const int q0 = tile * QT + wave * 64;
    const uint32_t *qh = q + q_row0 * DW;
    const uint32_t *kh = k + kv_row0 * DW;
    const uint32_t *vh = v + kv_row0 * DW;

    // ---- Q operands per 32-query block: 32 bytes of the lane's query row (bf8), or four fp16 fragments of the
    // eight dims 16 st + 8 h .. + 7 (the k-slots of this lane in the st-th 32x32x16 step)
    int8v_t qf[BF8 ? 2 : 1];
    half8_t qh16[BF8 ? 1 : 2][BF8 ? 1 : 4];
#pragma unroll
    for (int b = 0; b < 2; b++) {
        const int row = q0 + 32 * b + n;
        if constexpr (BF8) {
            u32x4 w0 = u32x4{0, 0, 0, 0}, w1 = u32x4{0, 0, 0, 0};
            if (row < L) {
                const u32x4 *src = reinterpret_cast<const u32x4 *>(qh + (int64_t)row * DW + 8 * h);
                w0 = src[0];
                w1 = src[1];
            }
            qf[b] = int8v_t{(int)w0.x, (int)w0.y, (int)w0.z, (int)w0.w, (int)w1.x, (int)w1.y, (int)w1.z, (int)w1.w};
        } else {
#pragma unroll
            for (int st = 0; st < 4; st++) {
                u32x2 w = u32x2{0, 0};
                if (row < L) w = *reinterpret_cast<const u32x2 *>(qh + (int64_t)row * DW + 4 * st + 2 * h);
                qh16[b][st] = dec8<MODE>(w.x, w.y);
            }
        }
    }

    constexpr float kGuard = 4096.f;   // a lane's share of a tile's row sum at which the reference point is renewed
    float16_t o[2][2];      // [query block][32-dim block]
    float m_run[2], mc_run[2], l_run[2];   // reference point of the query's exponentials (raw, and times scale * log2 e); the lane's share of its row sum
#pragma unroll
    for (int b = 0; b < 2; b++) {
        m_run[b] = -INFINITY;
        mc_run[b] = -INFINITY;
        l_run[b] = 0.f;
#pragma unroll
        for (int d = 0; d < 2; d++)
#pragma unroll
            for (int r = 0; r < 16; r++) o[b][d][r] = 0.f;
    }

    // ---- register staging of the next packed K / V tile: 256 threads carry V (4 keys x 4 dims each), 256 threads
    // K (16 bytes of one key each): the same threads in a four-wave workgroup, waves 0-3 and 4-7 in an
    // eight-wave one (all of them then have staging work to fill the wait for the tile's first LDS reads)
    constexpr bool kSplitStaging = kThreads >= 2 * UNITS;
    const bool stages_v = tid < UNITS, stages_k = kSplitStaging ? (tid >= UNITS && tid < 2 * UNITS) : tid < UNITS;
    const int kt_id = kSplitStaging ? tid - UNITS : tid;   // index of the thread among the K stagers
    u32x4 kreg;
    uint32_t vreg[4];
    auto prefetch = [&](int key0) {
        const int row0 = __builtin_amdgcn_readfirstlane(key0);
        const char *kt = reinterpret_cast<const char *>(kh + (int64_t)row0 * DW);
        const char *vt = reinterpret_cast<const char *>(vh + (int64_t)row0 * DW);
        const bool whole = key0 + BN <= L;   // wave-uniform: only the last tile needs per-row guards
        if (stages_k) {
            int t = kt_id;
            asm volatile("" : "+v"(t));   // keeps base + offset from being hoisted out of the key loop as 64-bit pairs
            const int krel = t / 4, c16 = t % 4;
            kreg = u32x4{0, 0, 0, 0};
            if (whole || key0 + krel < L) kreg = *reinterpret_cast<const u32x4 *>(kt + (uint32_t)(krel * D + 16 * c16));
        }
        if (stages_v) {
            int t = tid;
            asm volatile("" : "+v"(t));
            const int ddw = t % DW, kg = t / DW;
            const uint32_t voff = (uint32_t)(4 * kg * D + 4 * ddw);
            if (whole) {
#pragma unroll
                for (int r = 0; r < 4; r++) vreg[r] = *reinterpret_cast<const uint32_t *>(vt + voff + (uint32_t)(r * D));
            } else {
#pragma unroll
                for (int r = 0; r < 4; r++)
                    vreg[r] = key0 + 4 * kg + r < L ? *reinterpret_cast<const uint32_t *>(vt + voff + (uint32_t)(r * D)) : 0u;
            }
        }
    };
    auto stage = [&](int buf) {
        unsigned char *k_lds = smem + buf * kBufBytes;
        _Float16 *vt_lds = reinterpret_cast<_Float16 *>(k_lds + BN * KP);
        if (stages_k) {
            const int key = kt_id / 4, c16 = kt_id % 4;
            if constexpr (BF8) {
                *reinterpret_cast<u32x4 *>(k_lds + key * KP + 16 * c16) = kreg;
            } else {
                half8_t *kd = reinterpret_cast<half8_t *>(k_lds + key * KP + 32 * c16);
                kd[0] = dec8<MODE>(kreg.x, kreg.y);
                kd[1] = dec8<MODE>(kreg.z, kreg.w);
            }
        }
        if (stages_v) {
            // V: 4 keys x 4 dims -> V^T[dd][slot]; keys 4 kg .. 4 kg + 3 are quarter q4 = kg % 4 of their group of
            // 16 and go to slots 8 (q4 & 1) + 4 (q4 >> 1) .. + 3 of it
            const int ddw = tid % DW, kg = tid / DW;
            const int q4 = kg & 3, pos = 16 * (kg >> 2) + 8 * (q4 & 1) + 4 * (q4 >> 1);
            uint32_t lo2[4], hi2[4];   // halfs (key 0, key 1) and (key 2, key 3) of dim 4 ddw + c
            if constexpr (BF8) {
#pragma unroll
                for (int c = 0; c < 4; c++) {   // byte c of each word, placed as the high byte of its half
                    const uint32_t sel = 0x000c000cu | ((uint32_t)c << 8) | ((uint32_t)(4 + c) << 24);
                    lo2[c] = perm(vreg[1], vreg[0], sel);
                    hi2[c] = perm(vreg[3], vreg[2], sel);
                }
            } else {
                uint32_t p01[4], p23[4];
#pragma unroll
                for (int r = 0; r < 4; r++) dec_word<MODE>(vreg[r], p01[r], p23[r]);
                lo2[0] = perm(p01[1], p01[0], 0x05040100u); hi2[0] = perm(p01[3], p01[2], 0x05040100u);
                lo2[1] = perm(p01[1], p01[0], 0x07060302u); hi2[1] = perm(p01[3], p01[2], 0x07060302u);
                lo2[2] = perm(p23[1], p23[0], 0x05040100u); hi2[2] = perm(p23[3], p23[2], 0x05040100u);
                lo2[3] = perm(p23[1], p23[0], 0x07060302u); hi2[3] = perm(p23[3], p23[2], 0x07060302u);
            }
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const int row = 4 * ddw + c;
                *reinterpret_cast<u32x2 *>(vt_lds + row * VS + (((pos >> 3) ^ swz(row)) << 3) + (pos & 4)) = u32x2{lo2[c], hi2[c]};
            }
        }
    };

    const int key_begin = ZS ? zchunk * kchunk_keys : 0;
    const int key_end = ZS ? min(keys_scored, key_begin + kchunk_keys) : keys_scored;
    prefetch(key_begin);
    stage(0);
    if (key_begin + BN < key_end) prefetch(key_begin + BN);
    __syncthreads();
    // One key tile; the buffer index is a compile-time constant (the loop below is unrolled by two), so every
    // LDS address is a loop-invariant per-lane register plus an immediate offset instead of vector adds per tile.
    auto tile_body = [&](const int key0, auto cur_c) {
        constexpr int cur = decltype(cur_c)::value;
        const unsigned char *k_lds = smem + cur * kBufBytes;
        const _Float16 *vt_lds = reinterpret_cast<const _Float16 *>(k_lds + BN * KP);
        const bool ragged = mask_tail && key0 + BN > L;   // only the last tile can hold masked keys
        bool diag = false, skip = false;
        if constexpr (VC) {
            diag = causal && key0 + BN - 1 > q0;          // some key of the tile lies past the wave's first query
            skip = causal && key0 > q0 + 63;              // every key lies past the wave's last query
        }
        if constexpr (VC) {   // a wave with nothing to score in this tile still stages: one copy of that code, up front
            if (key0 + BN < key_end) stage(cur ^ 1);
            if (key0 + 2 * BN < key_end) prefetch(key0 + 2 * BN);
        }
        if (!skip) {
            // ---- S^T = K Q^T, raw scores: [query block][key block]
            int8v_t kf[BF8 ? 2 : 1];
            if constexpr (BF8) {
#pragma unroll
                for (int c = 0; c < 2; c++) {
                    const u32x4 *src = reinterpret_cast<const u32x4 *>(k_lds + (32 * c + n) * KP + 32 * h);
                    const u32x4 w0 = src[0], w1 = src[1];
                    kf[c] = int8v_t{(int)w0.x, (int)w0.y, (int)w0.z, (int)w0.w, (int)w1.x, (int)w1.y, (int)w1.z, (int)w1.w};
                }
            }
            half8_t vf[4][2];   // [16-key step][32-dim block]
#pragma unroll
            for (int g = 0; g < 4; g++)
#pragma unroll
                for (int d = 0; d < 2; d++) {
                    const int row = 32 * d + n;
                    vf[g][d] = *reinterpret_cast<const half8_t *>(vt_lds + row * VS + (((2 * g + h) ^ swz(row)) << 3));
                }
            // the next tile goes to the other buffer while this tile's fragments are on their way from LDS
            if constexpr (!VC) if (key0 + BN < key_end) stage(cur ^ 1);
            float16_t sc[2][2];
            const float16_t zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            if constexpr (BF8) {
#pragma unroll
                for (int b = 0; b < 2; b++)
#pragma unroll
                    for (int c = 0; c < 2; c++)   // cbsz = blgp = 1: both operands are BF8 (E5M2); no block scales
                        sc[b][c] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(kf[c], qf[b], zero16, 1, 1, 0, 0, 0, 0);
            } else {
#pragma unroll
                for (int c = 0; c < 2; c++) {   // one key block at a time: four fp16 K fragments live
                    half8_t k16[4];
#pragma unroll
                    for (int st = 0; st < 4; st++)
                        k16[st] = *reinterpret_cast<const half8_t *>(k_lds + (32 * c + n) * KP + 32 * st + 16 * h);
#pragma unroll
                    for (int b = 0; b < 2; b++)
#pragma unroll
                        for (int st = 0; st < 4; st++)
                            sc[b][c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(k16[st], qh16[b][st], st == 0 ? zero16 : sc[b][c], 0, 0, 0);
                }
            }
            if constexpr (!VC) if (key0 + 2 * BN < key_end) prefetch(key0 + 2 * BN);   // the tile after that into registers
#pragma unroll
            for (int b = 0; b < 2; b++) {
                // ---- online softmax of one 32-query block; p = 2^(s * c - m * c) on the raw-score maximum
                if (ragged || diag) {
                    int last = diag ? min(L - 1, q0 + 32 * b + n) : L - 1;   // last visible key
                    asm volatile("" : "+v"(last));   // keeps the 32 compares inside this rarely taken branch
                    const int rel = last - key0 - 4 * h;   // key 32 c + 8 (r / 4) + 4 h + r % 4 is hidden if 32 c + 8 (r / 4) + r % 4 > rel
#pragma unroll
                    for (int c = 0; c < 2; c++)
#pragma unroll
                        for (int r = 0; r < 16; r++)
                            if (32 * c + 8 * (r >> 2) + (r & 3) > rel) sc[b][c][r] = -INFINITY;
                }
                // The reference point m of the exponentials (P = 2^((s - m) c)) is not tracked per tile: the block's P
                // is computed against the current one, and the lane's share of the row sum -- needed anyway -- tells
                // whether that was safe.  P >= 0, so a share below kGuard bounds every P of the lane below kGuard:
                // nothing overflowed fp16, whose relative precision is the same everywhere below that, and O / l
                // does not depend on m.  Only when some lane's share reaches kGuard (the first tile, where m is
                // -inf and P comes out inf or NaN; later a score more than 12 binary orders above m) the true
                // maximum of the block is taken, m raised to it, the accumulators rescaled and P computed again.
                // On random data that happens once or twice per query block and sequence, so the 16 maximum
                // instructions, the cross-lane exchange and the compare of the per-tile tracking are gone from
                // the loop (they were a sixth of its vector instructions).
                half8_t pb[4];
                auto exp_block = [&](const float mc) {
                    float lsum = 0.f;
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        uint32_t pw[4];
#pragma unroll
                        for (int i = 0; i < 4; i++) {   // P rounded to fp16 (nearest even), as P.to(fp16)
                            const float e0 = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[b][g >> 1][8 * (g & 1) + 2 * i], scale_log2e, -mc));
                            const float e1 = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[b][g >> 1][8 * (g & 1) + 2 * i + 1], scale_log2e, -mc));
                            pw[i] = as_u32(__builtin_convertvector(float2v_t{e0, e1}, half2_t));
                            lsum = dot2(pw[i], 0x3c003c00u, lsum);   // the row sum takes the rounded values that multiply V
                        }
                        pb[g] = __builtin_bit_cast(half8_t, u32x4{pw[0], pw[1], pw[2], pw[3]});
                    }
                    return lsum;
                };
                float lsum = exp_block(mc_run[b]);
                if (__builtin_expect(__builtin_amdgcn_ballot_w64(!(lsum < kGuard)) != 0, 0)) {   // wave-uniform, rare
                    float mx = max3_raw(sc[b][0][0], sc[b][0][1], sc[b][0][2]);
                    mx = max_raw(mx, sc[b][0][3]);
#pragma unroll
                    for (int i = 2; i < 16; i++) mx = max3_raw(mx, sc[b][i >> 3][(2 * i) & 15], sc[b][i >> 3][(2 * i + 1) & 15]);
                    mx = max_xor32(mx);   // the two lanes that share the query
                    const float m_old = m_run[b];
                    const float m_new = max_raw(m_old, mx);
                    const float alpha = __builtin_amdgcn_exp2f((m_old - m_new) * scale_log2e);
                    m_run[b] = m_new;
                    mc_run[b] = m_new * scale_log2e;
                    l_run[b] *= alpha;
#pragma unroll
                    for (int d = 0; d < 2; d++) o[b][d] *= alpha;
                    lsum = exp_block(mc_run[b]);
                }
                l_run[b] += lsum;
                // ---- O^T += V^T P^T
#pragma unroll
                for (int g = 0; g < 4; g++)
#pragma unroll
                    for (int d = 0; d < 2; d++)
                        o[b][d] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[g][d], pb[g], o[b][d], 0, 0, 0);
            }
        }
        __syncthreads();  // tile i+1 is visible; every wave is done reading tile i
    };
    for (int key0 = key_begin; key0 < key_end; key0 += 2 * BN) {
        tile_body(key0, std::integral_constant<int, 0>{});
        if (key0 + BN < key_end) tile_body(key0 + BN, std::integral_constant<int, 1>{});
    }

    // ---- epilogue: the two lanes of a query add their shares of the row sum; normalise, store [q][dd]
    // (a key range: unnormalised, with the reference point and the row sum beside it)
    const int64_t rows_total = (int64_t)n_heads * L;
    float *oh = ZS ? part + ((int64_t)zchunk * rows_total + q_row0) * D : out + q_row0 * D;
#pragma unroll
    for (int b = 0; b < 2; b++) {
        const float other = as_float((uint32_t)__builtin_amdgcn_ds_bpermute(4 * (lane ^ 32), (int)as_u32(l_run[b])));
        const float l = ZS ? 1.f : l_run[b] + other;
        const int row = q0 + 32 * b + n;
        if constexpr (ZS)
            if (row < L && h == 0)
                *reinterpret_cast<float2v_t *>(part + (int64_t)n_kchunks * rows_total * D +
                                               ((int64_t)zchunk * rows_total + q_row0 + row) * 2) = float2v_t{m_run[b], l_run[b] + other};
        if (row < L) {
#pragma unroll
            for (int d = 0; d < 2; d++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const float4_t x = {o[b][d][4 * g], o[b][d][4 * g + 1], o[b][d][4 * g + 2], o[b][d][4 * g + 3]};
                    *reinterpret_cast<float4_t *>(oh + (int64_t)row * D + 32 * d + 8 * g + 4 * h) = x / l;
                }
        }
    }
}

// Fixed-length heads (cu_seqlens == nullptr; L rows per head) or packed variable-length sequences
// (cu_seqlens given: n_seq sequences of at most max_seqlen rows inside total_rows rows per head).
struct AttnArgs {
    const void *q, *k, *v;
    void *out;
    int64_t n_heads, L, kv_group;
    float scale;
    int tail;
    const void *cu_seqlens;
    int64_t n_seq, max_seqlen, total_rows;
    int causal;
    void *ws;           // optional device workspace for key ranges over workgroups (fixed-length heads)
    int64_t ws_bytes;
};

// Bytes of workspace that n_kchunks key ranges of n_heads * L rows need: accumulators, then (m, l) pairs.
static int64_t key_chunk_ws_bytes(int64_t n_heads, int64_t L, int64_t d, int n_kchunks) {
    return n_kchunks * n_heads * L * (d + 2) * 4;
}

// Key ranges of whole BN-key tiles, every range starting below the last scored key: keys per range, and the number
// of ranges that leaves.
static void key_range_plan(int64_t keys_scored, int bn, int &n_kchunks, int64_t &kchunk_keys) {
    const int64_t n_tiles_k = keys_scored / bn;
    kchunk_keys = (n_tiles_k + n_kchunks - 1) / n_kchunks * bn;
    n_kchunks = (int)((keys_scored + kchunk_keys - 1) / kchunk_keys);
}

static int launch_key_range_merge(const AttnArgs &a, int d, int n_kchunks, hipStream_t s) {
    const int64_t rows_total = a.n_heads * a.L, quads = rows_total * (d / 4);
    const dim3 grid((unsigned)((quads + 255) / 256)), block(256);
    const float c = a.scale * 1.4426950408889634f;
    const float *part = (const float *)a.ws;
    float *out = (float *)a.out;
    switch (n_kchunks) {
        case 2: hipLaunchKernelGGL(flash_attn_merge_kernel<2>, grid, block, 0, s, part, out, rows_total, d / 4, c); break;
        case 3: hipLaunchKernelGGL(flash_attn_merge_kernel<3>, grid, block, 0, s, part, out, rows_total, d / 4, c); break;
        case 4: hipLaunchKernelGGL(flash_attn_merge_kernel<4>, grid, block, 0, s, part, out, rows_total, d / 4, c); break;
        case 5: hipLaunchKernelGGL(flash_attn_merge_kernel<5>, grid, block, 0, s, part, out, rows_total, d / 4, c); break;
        case 6: hipLaunchKernelGGL(flash_attn_merge_kernel<6>, grid, block, 0, s, part, out, rows_total, d / 4, c); break;
        case 7: hipLaunchKernelGGL(flash_attn_merge_kernel<7>, grid, block, 0, s, part, out, rows_total, d / 4, c); break;
        case 8: hipLaunchKernelGGL(flash_attn_merge_kernel<8>, grid, block, 0, s, part, out, rows_total, d / 4, c); break;
        default:
            set_error("feather_flash_attn_fp8: %d key ranges", n_kchunks);
            return FEATHER_EINVAL;
    }
    return check_launch("feather_flash_attn_fp8 (merge of the key ranges)");
}

template <int D, int MODE, int QB, int SB, int BN, int OCC, bool VC, int WAVES = 4, int KSPLIT = 1, bool ZS = false>
static int launch_attn(const AttnArgs &a, hipStream_t s, int n_kchunks = 1) {
    constexpr int QT = 16 * QB * WAVES / KSPLIT;
    constexpr int KS = MODE == FEATHER_E5M2 ? (D + 16) / 2 : D + 8;   // K row pitch in fp16 units, as in the kernel
    constexpr size_t lds = (size_t)(BN * KS + D * BN) * 2 * 2;        // two (K, V^T) buffers
    const int64_t L = VC ? a.max_seqlen : a.L;
    const int tiles_per_seq = (int)((L + QT - 1) / QT);
    const int64_t tiles = VC ? tiles_per_seq * a.n_seq : tiles_per_seq;
    const int64_t blocks = tiles * a.n_heads;
    FEATHER_CHECK(blocks < (1ll << 31), FEATHER_ESHAPE, "feather_flash_attn_fp8: grid too large");
    if (blocks == 0) return FEATHER_OK;
    // the reference scores whole 64-key tiles (zero rows past L); otherwise only tiles of BN up to L
    int64_t keys_scored = a.tail == FEATHER_TAIL_REFERENCE ? (L + 63) / 64 * 64 : (L + BN - 1) / BN * BN;
    auto kern = flash_attn_kernel<D, MODE, QB, SB, BN, OCC, VC, WAVES, KSPLIT, ZS>;
    int64_t kchunk_keys = keys_scored;
    if (ZS) key_range_plan(keys_scored, BN, n_kchunks, kchunk_keys);
    static unsigned long long lds_raised = 0;   // per instantiation, one bit per device
    hipError_t e = raise_lds_limit(reinterpret_cast<const void *>(kern), lds, lds_raised);
    FEATHER_CHECK(e == hipSuccess, FEATHER_ELAUNCH, "feather_flash_attn_fp8: cannot raise LDS limit: %s",
                  hipGetErrorString(e));
    const float log2e = 1.4426950408889634f;
    hipLaunchKernelGGL(kern, dim3((unsigned)(blocks * (ZS ? n_kchunks : 1))), dim3(64 * WAVES), lds, s,
                       (const uint32_t *)a.q, (const uint32_t *)a.k, (const uint32_t *)a.v, (float *)a.out, (int)L,
                       (int)a.n_heads, (int)a.kv_group, (int)tiles, a.scale * log2e, (int)keys_scored,
                       a.tail == FEATHER_TAIL_MASK ? 1 : 0, (const int32_t *)a.cu_seqlens, tiles_per_seq,
                       (int)a.total_rows, a.causal, (float *)a.ws, (int)kchunk_keys, n_kchunks);
    int rc = check_launch("feather_flash_attn_fp8");
    if (!ZS || rc != FEATHER_OK) return rc;
    return launch_key_range_merge(a, D, n_kchunks, s);
}

template <int MODE, bool VC, int WAVES, int OCC, bool ZS = false>
static int launch_attn64_wide(const AttnArgs &a, hipStream_t s, int n_kchunks = 1) {
    constexpr int QT = 64 * WAVES, BN = 64, D = 64;
    constexpr size_t lds = (size_t)(BN * ((MODE == FEATHER_E5M2 ? D : 2 * D) + 16) + D * BN * 2) * 2;   // two (K, V^T fp16) buffers
    const int64_t L = VC ? a.max_seqlen : a.L;
    const int tiles_per_seq = (int)((L + QT - 1) / QT);
    const int64_t tiles = VC ? tiles_per_seq * a.n_seq : tiles_per_seq;
    const int64_t blocks = tiles * a.n_heads;
    FEATHER_CHECK(blocks < (1ll << 31), FEATHER_ESHAPE, "feather_flash_attn_fp8: grid too large");
    if (blocks == 0) return FEATHER_OK;
    // both tail modes score whole 64-key tiles here (the reference scores zero rows past L, the mask hides them)
    const int64_t keys_scored = (L + BN - 1) / BN * BN;
    const float log2e = 1.4426950408889634f;
    int64_t kchunk_keys = keys_scored;
    if (ZS) key_range_plan(keys_scored, BN, n_kchunks, kchunk_keys);
    hipLaunchKernelGGL((flash_attn64_wide_kernel<MODE, VC, WAVES, OCC, ZS>), dim3((unsigned)(blocks * (ZS ? n_kchunks : 1))),
                       dim3(64 * WAVES), lds, s, (const uint32_t *)a.q, (const uint32_t *)a.k, (const uint32_t *)a.v,
                       (float *)a.out, (int)L, (int)a.n_heads, (int)a.kv_group, (int)tiles, a.scale * log2e,
                       (int)keys_scored, a.tail == FEATHER_TAIL_MASK ? 1 : 0, (const int32_t *)a.cu_seqlens, tiles_per_seq,
                       (int)a.total_rows, a.causal, (float *)a.ws, (int)kchunk_keys, n_kchunks);
    int rc = check_launch("feather_flash_attn_fp8");
    if (!ZS || rc != FEATHER_OK) return rc;
    return launch_key_range_merge(a, D, n_kchunks, s);
}

// Workgroup shapes.  A wave of the d = 64 kernel owns 64 queries.  Staging a K/V tile into LDS is
// shared by the workgroup's waves, and from d = 128 on it is a large share of the vector work, so
// eight waves (twice the queries per staged tile, two waves per SIMD from one workgroup to overlap
// the barrier-separated phases) are faster wherever the coarser grid still covers the chip's 256 CUs;
// d = 256 takes eight waves at every length.
// Key ranges over workgroups (fixed-length, non-causal heads of 64 dims and more): the number of ranges (1, 2, 4
// or 8; 1 = the plain kernel) the finest workgroup shape of head dim d is cut into.  A cost model in nanoseconds:
// the key loop of a workgroup at its measured time per tile, against the merge kernel (launch and one round trip,
// then the partial results written, read back and the output written at ~4 TB/s); the grid stays within one pass
// over the 256 CUs.
static int pick_key_chunks(int64_t d, int64_t n_heads, int64_t L) {
    int64_t queries, bn, tile_ns;
    switch (d) {
        case 64: queries = 256; bn = 64; tile_ns = 1250; break;
        case 128: queries = 128; bn = 64; tile_ns = 1900; break;
        case 256: queries = 64; bn = 64; tile_ns = 2200; break;
        case 512: queries = 64; bn = 32; tile_ns = 2800; break;
        default: return 1;
    }
    const int64_t wgs = (L + queries - 1) / queries * n_heads, tiles = (L + bn - 1) / bn;
    int best = 1;
    int64_t best_ns = tiles * tile_ns;
    for (int z = 2; z <= kMaxKeyChunks && wgs * z <= 256 && z <= tiles; z *= 2) {
        const int64_t ns = (tiles + z - 1) / z * tile_ns + 3500 + (2 * z + 1) * n_heads * L * d * 4 / 4000;
        if (ns + 500 < best_ns) {
            best = z;
            best_ns = ns;
        }
    }
    return best;
}

template <int MODE, bool VC>
static int dispatch_attn(const AttnArgs &a, int64_t d, hipStream_t s) {
    const int64_t rows = VC ? a.max_seqlen : a.L, seqs = VC ? a.n_seq : 1;
    int zs = 1;
    if (!VC && a.ws) {
        zs = pick_key_chunks(d, a.n_heads, a.L);
        while (zs > 1 && a.ws_bytes < key_chunk_ws_bytes(a.n_heads, a.L, d, zs)) zs /= 2;   // a smaller workspace: fewer ranges
    }
    auto fills_chip = [&](int64_t queries_per_group) {
        return (rows + queries_per_group - 1) / queries_per_group * seqs * a.n_heads >= 256;
    };
    auto rounds = [&](int64_t queries_per_group) {   // passes of the grid over the 256 CUs, one workgroup per CU
        return ((rows + queries_per_group - 1) / queries_per_group * seqs * a.n_heads + 255) / 256;
    };
    switch (d) {
        case 32:   // narrower than anything the reference's tl.dot accepts (d / 4 >= 16); one MFMA k-step per score
            return launch_attn<32, MODE, 4, 4, 64, 2, VC>(a, s);
        case 64:   // all four query blocks of a wave share every K fragment
            // eight waves halve the staging work per query (-2 % time); a causal tile of 512 queries
            // would idle its early waves through too many masked key tiles
            if constexpr (!VC)
                if (zs > 1) return launch_attn64_wide<MODE, false, 4, 2, true>(a, s, zs);
            if (!a.causal && fills_chip(512)) return launch_attn64_wide<MODE, VC, 8, 1>(a, s);
            return launch_attn64_wide<MODE, VC, 4, 2>(a, s);
        case 128:
            if constexpr (!VC)
                if (zs > 1) return launch_attn<128, MODE, 2, 2, 64, 2, false, 4, 1, true>(a, s, zs);
            if (fills_chip(256)) return launch_attn<128, MODE, 2, 2, 64, 1, VC, 8>(a, s);
            return launch_attn<128, MODE, 2, 2, 64, 2, VC>(a, s);
        case 256: {
            // Three shapes, from the finest work items to the cheapest per query (time per 64 keys of
            // a workgroup's loop at full occupancy, measured): A = 64 queries, two wave groups halve
            // every key tile (2.9 us); B = 128 queries, eight waves of 16 (3.2 us); C = 256 queries,
            // eight waves of 32 on 32-key tiles, which halves the LDS reads per query that bound this
            // head dim (4.6 us; L = 8192: 792 -> 640 us against B).  Pick by rounds over the 256 CUs x cost.
            if constexpr (!VC)
                if (zs > 1) return launch_attn<256, MODE, 1, 1, 64, 1, false, 8, 2, true>(a, s, zs);
            const int64_t ra = rounds(64), rb = rounds(128), rc = rounds(256);
            if (!a.causal && ra * 29 <= rb * 32 && ra * 29 <= rc * 46) return launch_attn<256, MODE, 1, 1, 64, 1, VC, 8, 2>(a, s);
            if (rc * 46 < rb * 32 || fills_chip(256)) return launch_attn<256, MODE, 2, 2, 32, 1, VC, 8>(a, s);
            return launch_attn<256, MODE, 1, 1, 64, 1, VC, 8>(a, s);
        }
        case 512: {
            // A = 64 queries, two wave groups of 16 keys per 32-key tile (3.1 us per tile of a
            // workgroup's loop); B = 128 queries, eight waves (3.5 us)
            if constexpr (!VC)
                if (zs > 1) return launch_attn<512, MODE, 1, 1, 32, 1, false, 8, 2, true>(a, s, zs);
            const int64_t ra = rounds(64), rb = rounds(128);
            if (!a.causal && ra * 31 <= rb * 35) return launch_attn<512, MODE, 1, 1, 32, 1, VC, 8, 2>(a, s);
            if (fills_chip(128) || !a.causal) return launch_attn<512, MODE, 1, 1, 32, 1, VC, 8>(a, s);
            return launch_attn<512, MODE, 1, 1, 32, 1, VC>(a, s);
        }
    }
    set_error("feather_flash_attn_fp8: head dim %lld not supported (32, 64, 128, 256, 512)", (long long)d);
    return FEATHER_ESHAPE;
}

}  // namespace feather

using namespace feather;

extern "C" int64_t feather_flash_attn_workspace_bytes(int64_t n_heads, int64_t L, int64_t d) {
    if (n_heads <= 0 || L <= 0 || L >= (1ll << 30)) return 0;
    const int z = pick_key_chunks(d, n_heads, L);
    return z > 1 ? key_chunk_ws_bytes(n_heads, L, d, z) : 0;
}

extern "C" int feather_flash_attn_fp8(const void *q, const void *k, const void *v, void *out_f32, int64_t n_heads,
                                      int64_t L, int64_t d, int64_t kv_group, int mode, float scale, int tail,
                                      void *stream) {
    return feather_flash_attn_fp8_ws(q, k, v, out_f32, nullptr, 0, n_heads, L, d, kv_group, mode, scale, tail, stream);
}

extern "C" int feather_flash_attn_fp8_ws(const void *q, const void *k, const void *v, void *out_f32, void *workspace,
                                         int64_t workspace_bytes, int64_t n_heads, int64_t L, int64_t d,
                                         int64_t kv_group, int mode, float scale, int tail, void *stream) {
    FEATHER_CHECK(mode == FEATHER_E5M2 || mode == FEATHER_E4M3, FEATHER_EMODE,
                  "feather_flash_attn_fp8: mode %d not supported", mode);
    FEATHER_CHECK(workspace_bytes >= 0 && (workspace || workspace_bytes == 0) && aligned(workspace, 16), FEATHER_EINVAL,
                  "feather_flash_attn_fp8_ws: workspace must be 16-byte aligned, its size not negative");
    FEATHER_CHECK(tail == FEATHER_TAIL_MASK || tail == FEATHER_TAIL_REFERENCE, FEATHER_EINVAL,
                  "feather_flash_attn_fp8: bad tail flag %d", tail);
    FEATHER_CHECK(n_heads >= 0 && L >= 0 && d > 0, FEATHER_EINVAL, "feather_flash_attn_fp8: negative shape");
    FEATHER_CHECK(scale > 0.f, FEATHER_EINVAL,
                  "feather_flash_attn_fp8: scale must be positive (the running maximum is kept on raw scores)");
    FEATHER_CHECK(kv_group >= 1 && n_heads % kv_group == 0, FEATHER_ESHAPE,
                  "feather_flash_attn_fp8: n_heads=%lld is not a multiple of kv_group=%lld", (long long)n_heads,
                  (long long)kv_group);
    FEATHER_CHECK(L < (1ll << 30), FEATHER_ESHAPE, "feather_flash_attn_fp8: sequence too long");
    if (n_heads == 0 || L == 0) return FEATHER_OK;
    FEATHER_CHECK(q && k && v && out_f32, FEATHER_EINVAL, "feather_flash_attn_fp8: null pointer");
    FEATHER_CHECK(aligned(q, 16) && aligned(k, 16) && aligned(v, 16) && aligned(out_f32, 16), FEATHER_EINVAL,
                  "feather_flash_attn_fp8: pointers must be 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    const AttnArgs a = {q, k, v, out_f32, n_heads, L, kv_group, scale, tail, nullptr, 0, 0, 0, 0, workspace,
                        workspace_bytes};
    if (mode == FEATHER_E5M2) return dispatch_attn<FEATHER_E5M2, false>(a, d, s);
    return dispatch_attn<FEATHER_E4M3, false>(a, d, s);
}

extern "C" int feather_flash_attn_fp8_varlen(const void *q, const void *k, const void *v, void *out_f32,
                                             const void *cu_seqlens, int64_t n_seq, int64_t max_seqlen,
                                             int64_t total_rows, int64_t n_heads, int64_t d, int64_t kv_group, int mode,
                                             float scale, int causal, void *stream) {
    const char *me = "feather_flash_attn_fp8_varlen";
    FEATHER_CHECK(mode == FEATHER_E5M2 || mode == FEATHER_E4M3, FEATHER_EMODE, "%s: mode %d not supported", me, mode);
    FEATHER_CHECK(n_heads >= 0 && n_seq >= 0 && max_seqlen >= 0 && total_rows >= 0 && d > 0, FEATHER_EINVAL,
                  "%s: negative shape", me);
    FEATHER_CHECK(causal == 0 || causal == 1, FEATHER_EINVAL, "%s: causal must be 0 or 1", me);
    FEATHER_CHECK(scale > 0.f, FEATHER_EINVAL, "%s: scale must be positive (the running maximum is kept on raw scores)", me);
    FEATHER_CHECK(kv_group >= 1 && n_heads % kv_group == 0, FEATHER_ESHAPE,
                  "%s: n_heads=%lld is not a multiple of kv_group=%lld", me, (long long)n_heads, (long long)kv_group);
    FEATHER_CHECK(max_seqlen <= total_rows && total_rows < (1ll << 30), FEATHER_ESHAPE,
                  "%s: max_seqlen=%lld must not exceed total_rows=%lld (< 2^30)", me, (long long)max_seqlen,
                  (long long)total_rows);
    FEATHER_CHECK(d == 32 || d == 64 || d == 128 || d == 256 || d == 512, FEATHER_ESHAPE,
                  "%s: head dim %lld not supported (32, 64, 128, 256, 512)", me, (long long)d);
    if (n_heads == 0 || n_seq == 0 || max_seqlen == 0) return FEATHER_OK;
    FEATHER_CHECK(q && k && v && out_f32 && cu_seqlens, FEATHER_EINVAL, "%s: null pointer", me);
    FEATHER_CHECK(aligned(q, 16) && aligned(k, 16) && aligned(v, 16) && aligned(out_f32, 16) && aligned(cu_seqlens, 4),
                  FEATHER_EINVAL, "%s: q/k/v/out must be 16-byte aligned", me);
    hipStream_t s = (hipStream_t)stream;
    const AttnArgs a = {q, k, v, out_f32, n_heads, 0, kv_group, scale, FEATHER_TAIL_MASK, cu_seqlens, n_seq,
                        max_seqlen, total_rows, causal, nullptr, 0};
    if (mode == FEATHER_E5M2) return dispatch_attn<FEATHER_E5M2, true>(a, d, s);
    return dispatch_attn<FEATHER_E4M3, true>(a, d, s);
}
