// Packed-FP8 GEMV: out[r] = sum_k dec(m[r,k]) * dec(v[k]), fp32 accumulate.
//
// The kernel is a pure HBM stream of the matrix (1 byte per element); the
// vector (K bytes) is decoded ONCE per workgroup into LDS as fp16 and re-used
// by every row the workgroup owns.
//
//   * one wave owns RPW rows at a time; a lane reads 16 consecutive codes
//     (one 128-bit non-temporal load) per row per step, so a wave-load covers
//     1 KiB of contiguous row bytes; U steps are issued back to back and
//     unconditionally, so RPW * U loads are in flight per lane;
//   * decode is register-only: E5M2 is byte placement (v_perm_b32), E4M3 is
//     byte-parallel integer arithmetic on four codes at a time;
//   * multiply-accumulate is v_dot2_f32_f16 (two exact fp16 x fp16 products
//     added into an fp32 accumulator);
//   * the RPW row sums are folded across the wave with DPP.
//
// Measured dead ends, kept here so they are not tried again.  (1) Feeding
// the codes to FP8 MFMAs (matrix bytes as A, vector bytes as B, dot product on
// the diagonal of the 16x16 result) removes the decode but ran 12 % SLOWER at
// 16384^2 (47.3 us against 41.6 us for E5M2).  (2) Issuing the loads of the
// next group before the arithmetic of the current one (software pipelining,
// twice the bytes in flight) also lost 6 %: at ~6.4 TB/s the memory system is
// saturated and deeper queues only add latency.  (3) The multiply-accumulate on
// v_mfma_f32_4x4x4f16 (one MFMA issue per packed word instead of two v_dot2c;
// the lane's dot product sits on the diagonal of its 4x4 block) is exact and
// changes nothing: E4M3 45.2 us either way.  (4) Plain instead of non-temporal
// loads: 48.8 us.  Buffer loads (any cache policy) instead of global loads: no
// gain once the row bases are wave-uniform.  (5) E4M3 through the hardware's
// FP8 -> fp16 conversion (v_cvt_scalef32_pk_f16_fp8: 9 instructions per word
// with the check below instead of 14) with the exact decode as a wave-uniform
// fallback for batches that hold a code on which the two differ (zero exponent
// with a non-zero mantissa: OCP subnormals against the reference's raw mantissa
// bits; 0x7F / 0xFF).  Correct, but the RNE packer emits those subnormal codes
// for every |x| < 2^-6, 1-2 % of N(0,1) data, so every batch of a wave (8192
// codes) falls back and pays for both decodes: 64 us.  (6) Per-wave time
// stamps (s_memrealtime; one workgroup of 64 rows per CU) show that the two waves of a SIMD do not advance
// together: the older one wins the vector ALU whenever both have data and ends
// 6-11 us before the younger one in E4M3 mode (3 us in E5M2), all workgroups
// ending within 3 us of each other.  Levelling the two through s_setprio (each
// wave publishes its step count in LDS, the one behind raises its priority)
// shrinks that spread to 3 us and leaves the time where it was (43.5 -> 42.8-44.1
// us): the memory system is as busy with four waves per CU in the last
// microseconds as with eight.  (7) With one workgroup of 64 rows per CU, fetching the vector with 128-bit
// loads and the first group of matrix loads before the vector is decoded into LDS
// gained 0.5 us for E5M2 at 16384^2 only and lost as much elsewhere; it pays since
// the workgroups are eight rows (see the kernel).
//
// A workgroup takes a contiguous range of rows and decodes the vector once for
// all of them.
#include "common.h"

namespace feather {

constexpr int kGemvThreads = 256;          // generic path
constexpr int kGemvWaves = kGemvThreads / kWave;
constexpr int kMaxChunk = 32768;  // codes of the vector held in LDS at once (64 KiB as fp16)

// 16 codes (one uint4) of a row against the matching 16 fp16 of the vector.
// Keeps a wave-uniform value in scalar registers, so that the compiler does not fold it into per-lane
// (vector) address arithmetic.
__device__ __forceinline__ uint32_t pin_scalar(uint32_t v) {
    asm volatile("" : "+s"(v));
    return v;
}
// Same for a per-lane 32-bit offset: pinned next to its use, its zero extension stays in the block of the load
// and the load takes the form "scalar 64-bit base + 32-bit vector offset".
__device__ __forceinline__ uint32_t pin_vector(uint32_t v) {
    asm volatile("" : "+v"(v));
    return v;
}
typedef const __attribute__((address_space(1))) uint8_t *global_u8_ptr;   // global address space kept through the asm
__device__ __forceinline__ global_u8_ptr pin_scalar(global_u8_ptr p) {
    asm volatile("" : "+s"(p));
    return p;
}
__device__ __forceinline__ u32x4 load_nt128_global(global_u8_ptr p) {
    return __builtin_nontemporal_load(reinterpret_cast<const __attribute__((address_space(1))) u32x4 *>(p));
}

template <int MODE>
__device__ __forceinline__ float mac16(const u32x4 &a, const u32x4 &x0, const u32x4 &x1, float acc) {
    uint32_t p, q;
    dec_word<MODE>(a.x, p, q);
    acc = dot2(p, x0.x, acc);
    acc = dot2(q, x0.y, acc);
    dec_word<MODE>(a.y, p, q);
    acc = dot2(p, x0.z, acc);
    acc = dot2(q, x0.w, acc);
    dec_word<MODE>(a.z, p, q);
    acc = dot2(p, x1.x, acc);
    acc = dot2(q, x1.y, acc);
    dec_word<MODE>(a.w, p, q);
    acc = dot2(p, x1.z, acc);
    acc = dot2(q, x1.w, acc);
    return acc;
}

// Fast path: rows are 16-byte aligned (K % 16 == 0, base aligned).
//   m        matrix, row stride K bytes
//   v        vector words for columns [k0, k0 + kc)
//   k0, kc   column chunk handled by this launch (kc <= kMaxChunk, kc % 16 == 0)
//   accumulate  add to out instead of overwriting (later chunks)
//   FULL     kc is a multiple of 1024: every wave-load is in range, no lane guards
//
// A row is walked in steps of 1 KiB (one 128-bit load per lane).  The step at
// which a wave STARTS is rotated with the row index (stride kStagger steps):
// without it all waves of the chip sweep the same column offsets in lock step,
// their addresses differ by multiples of the row pitch and pile onto a few HBM
// channels; the rotation spreads concurrent waves over the whole row and is
// worth ~15 % of bandwidth at 16384 x 16384.
constexpr int kStagger = 7;

template <int MODE, int RPW, int U, int WAVES, bool FULL, bool EARLY>
__global__ __launch_bounds__(WAVES * kWave) void gemv_fp8_kernel(const uint8_t *__restrict__ m,
                                                                const uint32_t *__restrict__ v,
                                                                float *__restrict__ out, int M, int64_t K, int k0,
                                                                int kc, int rows_per_wg, int accumulate) {
    extern __shared__ uint32_t lds32[];  // fp16 vector chunk, zero-padded to whole steps
    constexpr int kStep = kWave * 16;    // codes per wave-load
    constexpr int kThreads = WAVES * kWave;
    const int n_steps = (kc + kStep - 1) / kStep;
    const int lane = lane_id();
    const int wave = wave_id();
    const int row_begin = blockIdx.x * rows_per_wg;
    const int row_end = min(row_begin + rows_per_wg, M);

    // One group of wave-loads: U steps of RPW rows, starting at step `it` of the rotated walk.
    int col[U];
    u32x4 a[RPW][U];
    auto issue = [&](int r0, int it) {
        const int s0 = (int)(((unsigned)(r0 / RPW) * (unsigned)kStagger) % (unsigned)n_steps);
        const uint32_t lane_off = pin_vector((uint32_t)(lane * 16));
#pragma unroll
        for (int u = 0; u < U; u++) {
            int st = it + u + s0;
            if (st >= n_steps) st -= n_steps;
            col[u] = st * kStep;
#pragma unroll
            for (int r = 0; r < RPW; r++) {
                const int row = min(r0 + r, M - 1);  // surplus rows re-read the last row, result dropped
                // wave-uniform 64-bit base (scalar registers) + the lane's 32-bit offset: no vector address arithmetic
                global_u8_ptr base = pin_scalar((global_u8_ptr)(m + (int64_t)row * K + k0 + col[u]));
                if (FULL || col[u] + lane * 16 < kc) a[r][u] = load_nt128_global(base + lane_off);
                else a[r][u] = u32x4{0, 0, 0, 0};
            }
        }
    };

    // The kernel starts with a dependent chain: vector words -> decode -> LDS -> barrier -> first
    // matrix loads -> first arithmetic, two memory latencies before anything is computed.  With EARLY
    // a thread fetches its share of the vector (up to kMaxChunk / 16 / kThreads 128-bit loads) and
    // then at once its first group of matrix loads; loads return in order, so the vector is decoded
    // into LDS while the matrix data is still on its way.  With workgroups of eight rows, where every
    // workgroup pays that start for two to four groups of loads: 16384^2 E4M3 43.0 -> 41.15 us, E5M2
    // 40.9 -> 39.8 us; 8192^2 E5M2 12.14 -> 11.9 us.  (Issued the other way round the vector words
    // queue behind the matrix loads: slower than no overlap at all.)
    bool have = false;
    if (EARLY) {
        constexpr int kQuads = kMaxChunk / 16 / kThreads;
        u32x4 xv[kQuads];
#pragma unroll
        for (int j = 0; j < kQuads; j++) {
            const int q = threadIdx.x + j * kThreads;
            xv[j] = q < kc / 16 ? reinterpret_cast<const u32x4 *>(v)[q] : u32x4{0, 0, 0, 0};
        }
        if (n_steps >= U && row_begin + wave * RPW < row_end) {
            issue(row_begin + wave * RPW, 0);
            have = true;
        }
#pragma unroll
        for (int j = 0; j < kQuads; j++) {
            const int q = threadIdx.x + j * kThreads;
            if (q < n_steps * (kStep / 16)) {
                uint32_t o[8];
                dec_word<MODE>(xv[j].x, o[0], o[1]);
                dec_word<MODE>(xv[j].y, o[2], o[3]);
                dec_word<MODE>(xv[j].z, o[4], o[5]);
                dec_word<MODE>(xv[j].w, o[6], o[7]);
                u32x4 *dst = reinterpret_cast<u32x4 *>(lds32) + 2 * q;
                dst[0] = u32x4{o[0], o[1], o[2], o[3]};
                dst[1] = u32x4{o[4], o[5], o[6], o[7]};
            }
        }
    } else {
        for (int i = threadIdx.x; i < n_steps * (kStep / 4); i += kThreads) {
            uint32_t p01 = 0, p23 = 0;
            if (i < kc / 4) dec_word<MODE>(v[i], p01, p23);
            reinterpret_cast<u32x2 *>(lds32)[i] = u32x2{p01, p23};
        }
    }
    __syncthreads();

    const u32x4 *lds128 = reinterpret_cast<const u32x4 *>(lds32);
    for (int r0 = row_begin + wave * RPW; r0 < row_end; r0 += WAVES * RPW) {
        float acc[RPW];
#pragma unroll
        for (int r = 0; r < RPW; r++) acc[r] = 0.f;
        int it = 0;
        for (; it + U <= n_steps; it += U) {   // U wave-loads per row in flight
            if (!EARLY || !have) issue(r0, it);
            have = false;
#pragma unroll
            for (int u = 0; u < U; u++) {
                // fp16 vector: 2 bytes per column; scalar step offset + the lane's constant offset
                const u32x4 *xp = reinterpret_cast<const u32x4 *>(reinterpret_cast<const uint8_t *>(lds32) +
                                                                  pin_scalar(2u * (uint32_t)col[u]) + (uint32_t)(lane * 32));
                u32x4 x0 = xp[0], x1 = xp[1];
#pragma unroll
                for (int r = 0; r < RPW; r++) acc[r] = mac16<MODE>(a[r][u], x0, x1, acc[r]);
            }
        }
        if (it < n_steps) {
            const int s0 = (int)(((unsigned)(r0 / RPW) * (unsigned)kStagger) % (unsigned)n_steps);
            for (; it < n_steps; it++) {       // fewer than U steps left
                int st = it + s0;
                if (st >= n_steps) st -= n_steps;
                int c = st * kStep;
                u32x4 b[RPW];
#pragma unroll
                for (int r = 0; r < RPW; r++) {
                    const int row = min(r0 + r, M - 1);
                    if (FULL || c + lane * 16 < kc) b[r] = load_nt128(m + (int64_t)row * K + k0 + lane * 16 + c);
                    else b[r] = u32x4{0, 0, 0, 0};
                }
                int c8 = (c + lane * 16) / 8;
                u32x4 x0 = lds128[c8], x1 = lds128[c8 + 1];
#pragma unroll
                for (int r = 0; r < RPW; r++) acc[r] = mac16<MODE>(b[r], x0, x1, acc[r]);
            }
        }
#pragma unroll
        for (int r = 0; r < RPW; r++) {
            float s = wave_sum(acc[r]);
            if (lane == 0 && r0 + r < row_end) {
                if (accumulate) s += out[r0 + r];
                out[r0 + r] = s;
            }
        }
    }
}

// Generic path: any K % 4 == 0 and 4-byte aligned rows; one word per lane per
// step.  Used for shapes whose rows are not 16-byte aligned.
template <int MODE>
__global__ __launch_bounds__(kGemvThreads) void gemv_fp8_generic_kernel(const uint32_t *__restrict__ m,
                                                                       const uint32_t *__restrict__ v,
                                                                       float *__restrict__ out, int M, int64_t n_col) {
    const int lane = lane_id();
    const int wave = wave_id();
    for (int row = blockIdx.x * kGemvWaves + wave; row < M; row += gridDim.x * kGemvWaves) {
        const uint32_t *rp = m + (int64_t)row * n_col;
        float acc = 0.f;
        for (int64_t j = lane; j < n_col; j += kWave) {
            uint32_t p, q, x, y;
            dec_word<MODE>(rp[j], p, q);
            dec_word<MODE>(v[j], x, y);
            acc = dot2(p, x, acc);
            acc = dot2(q, y, acc);
        }
        float s = wave_sum(acc);
        if (lane == 0) out[row] = s;
    }
}

__global__ void fill_zero_kernel(float *p, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = 0.f;
}

template <int MODE, int RPW, int U, bool EARLY>
static int launch_gemv_fast(const void *m, const void *v, float *out, int64_t M, int64_t K, int64_t wgs, hipStream_t s) {
    constexpr int WAVES = 8;
    constexpr int kStep = kWave * 16;
    int64_t rows_per_wg = (M + wgs - 1) / wgs;
    rows_per_wg = (rows_per_wg + WAVES * RPW - 1) / (WAVES * RPW) * (WAVES * RPW);
    int64_t blocks = (M + rows_per_wg - 1) / rows_per_wg;
    for (int64_t k0 = 0; k0 < K; k0 += kMaxChunk) {
        int kc = (int)((K - k0) < kMaxChunk ? (K - k0) : kMaxChunk);
        int n_steps = (kc + kStep - 1) / kStep;
        size_t lds = (size_t)n_steps * kStep * 2;
        const void *vk = (const uint32_t *)v + k0 / 4;
        auto go = [&](auto kern) {
            hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(WAVES * kWave), lds, s, (const uint8_t *)m,
                               (const uint32_t *)vk, out, (int)M, K, (int)k0, kc, (int)rows_per_wg, k0 > 0 ? 1 : 0);
        };
        // E4M3 rows under 16 steps gain from it only on more workgroups than are resident at once, i.e. from 8192 rows
        // on (K = 4096: 16384 rows 14.6 -> 13.2 us, 8192 rows 8.6 -> 8.2 us; K = 8192: 8192 rows 13.7 -> 13.3 us, 16384
        // rows 24.0 -> 23.5 us) and lose below (4096 rows: K = 4096 5.3 -> 5.6 us, K = 8192 7.9 -> 8.2 us); the fetch
        // uses 128-bit loads
        const bool early = EARLY && aligned(vk, 16) && (MODE == FEATHER_E5M2 || kc >= 16 * kStep || M >= 8192);
        if (kc % kStep == 0) {
            if (early) go(gemv_fp8_kernel<MODE, RPW, U, WAVES, true, EARLY>);
            else go(gemv_fp8_kernel<MODE, RPW, U, WAVES, true, false>);
        } else {
            if (early) go(gemv_fp8_kernel<MODE, RPW, U, WAVES, false, EARLY>);
            else go(gemv_fp8_kernel<MODE, RPW, U, WAVES, false, false>);
        }
        int rc = check_launch("feather_gemv_fp8");
        if (rc != FEATHER_OK) return rc;
    }
    return FEATHER_OK;
}

template <int MODE>
static int launch_gemv(const void *m, const void *v, float *out, int64_t M, int64_t K, hipStream_t s) {
    if (K % 16 != 0 || !aligned(m, 16)) {
        int64_t blocks = (M + kGemvWaves - 1) / kGemvWaves;
        if (blocks > 256 * 8) blocks = 256 * 8;
        hipLaunchKernelGGL((gemv_fp8_generic_kernel<MODE>), dim3((unsigned)blocks), dim3(kGemvThreads), 0, s,
                           (const uint32_t *)m, (const uint32_t *)v, out, (int)M, K / 4);
        return check_launch("feather_gemv_fp8");
    }
    // Shape of the launch (measured on MI355X, rotating matrices of 1 GiB in total).  Rows of four
    // steps or more: one row per wave, four steps in flight, and workgroups of eight rows, as many as
    // the matrix has -- each decodes the vector for itself (1/8 of its matrix bytes, from L2), several
    // are resident per CU and a CU that finishes one picks up the next, which evens out what one
    // workgroup per CU with a fixed share of the rows left to the slowest CU.  16384^2: E5M2 41.8 ->
    // 40.9 us, E4M3 45.0 -> 43.0 us before the early fetch (with one workgroup per CU four rows
    // per wave that share every LDS read of the vector had been E4M3's best shape); 8192^2: 13.0 -> 12.2
    // and 15.7 -> 13.0 us; 4096 x 8192 E4M3 11.2 -> 8.3 us.  Four-wave or sixteen-wave workgroups, eight
    // steps in flight and other rotations than 7 steps per row are equal or slower.  Shorter rows keep
    // four rows per wave and two steps in flight, in twice as many workgroups as CUs.
    if (K >= 4 * kWave * 16) return launch_gemv_fast<MODE, 1, 4, true>(m, v, out, M, K, (M + 7) / 8, s);
    return launch_gemv_fast<MODE, 4, 2, false>(m, v, out, M, K, 512, s);
}

}  // namespace feather

using namespace feather;

extern "C" int feather_gemv_fp8(const void *m, const void *v, void *out_f32, int64_t M, int64_t K, int mode,
                                void *stream) {
    FEATHER_CHECK(mode == FEATHER_E5M2 || mode == FEATHER_E4M3, FEATHER_EMODE, "feather_gemv_fp8: mode %d not supported",
                  mode);
    FEATHER_CHECK(M >= 0 && K >= 0, FEATHER_EINVAL, "feather_gemv_fp8: negative shape");
    FEATHER_CHECK(K % 4 == 0, FEATHER_ESHAPE,
                  "feather_gemv_fp8: K=%lld is not a multiple of 4 (rows would straddle packed words)", (long long)K);
    FEATHER_CHECK(M < (1ll << 31) && K < (1ll << 31), FEATHER_ESHAPE, "feather_gemv_fp8: shape too large");
    if (M == 0) return FEATHER_OK;
    FEATHER_CHECK(out_f32, FEATHER_EINVAL, "feather_gemv_fp8: null out");
    FEATHER_CHECK(aligned(out_f32, 4), FEATHER_EINVAL, "feather_gemv_fp8: misaligned out");
    if (K == 0) {
        // empty rows sum to zero; a fill kernel (not a memset node) keeps the call graph-capturable
        int64_t blocks = (M + 255) / 256;
        hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)(blocks > 4096 ? 4096 : blocks)), dim3(256), 0,
                           (hipStream_t)stream, (float *)out_f32, M);
        return check_launch("feather_gemv_fp8");
    }
    FEATHER_CHECK(m && v, FEATHER_EINVAL, "feather_gemv_fp8: null pointer");
    FEATHER_CHECK(aligned(m, 4) && aligned(v, 4), FEATHER_EINVAL, "feather_gemv_fp8: misaligned pointer");
    hipStream_t s = (hipStream_t)stream;
    if (mode == FEATHER_E5M2) return launch_gemv<FEATHER_E5M2>(m, v, (float *)out_f32, M, K, s);
    return launch_gemv<FEATHER_E4M3>(m, v, (float *)out_f32, M, K, s);
}
