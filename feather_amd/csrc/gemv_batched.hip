// Batched packed-FP8 GEMV (skinny GEMM): out[b, r] = sum_k dec(w[r,k]) * dec(x[b,k])
// for up to 64 vectors, streaming the weight matrix once for the whole batch.
//
// With more than a couple of vectors the per-element multiply count rules out
// the VALU, so the product runs on the matrix cores: a 16-row slab of W is the
// A operand of v_mfma_f32_16x16x32_f16 and 16 vectors are the B columns.
// A workgroup of 4 waves owns 64 rows (16 per wave) and a slice of K, walked in
// chunks of 256 columns.  Per chunk every lane loads 4 x 16 consecutive codes
// of its row (128-bit loads) and decodes them in registers; the vectors' chunk
// is decoded ONCE per workgroup into LDS as fp16 (each thread 16 codes per 16
// vectors) and read from there as the B operand by all four waves, so the
// vector bytes pulled from L2 and their decode cost a quarter of the weight's
// instead of twice as much with one 16-row slab per workgroup.  The loads of
// chunk c + 1 are issued before the MFMAs of chunk c; LDS is double buffered,
// one barrier per chunk.
// A chunk step costs one memory latency (~1 us under load) whatever its size, so
// a workgroup that must walk all of K itself (the fused SwiGLU epilogue needs
// complete sums) runs KG = 2 such four-wave groups side by side: group g takes
// chunks g, g + 2, ..., each group stages its own vector chunks, and group 1
// hands its accumulators to group 0 through LDS at the end (a fixed order of
// additions).  Twice the bytes in flight per CU, half the steps.
// Small matrices do not have enough 64-row tiles to fill 256 CUs; the internal
// launcher therefore cuts K into slices that write separate partial results
// which the consumer adds in slice order (deterministic, no atomics).
// (Handing the vectors over as already-decoded fp16 instead of packed codes was
// measured and dropped: it doubles the vector bytes pulled from L2.)
#include "common.h"
#include "internal.h"

namespace feather {

constexpr int kBgThreads = 256;
constexpr int kBgChunk = 256;                  // columns per chunk
constexpr int kBgPitch = kBgChunk + 8;         // halfs per LDS row: +16 B keeps 8 lanes x 16 B on distinct banks
constexpr int kBgRows = 64;                    // rows per workgroup

template <int MODE>
__device__ __forceinline__ half8_t bg_dec8(uint32_t w0, uint32_t w1) {
    u32x4 r;
    uint32_t a, b;
    dec_word<MODE>(w0, a, b);
    r.x = a; r.y = b;
    dec_word<MODE>(w1, a, b);
    r.z = a; r.w = b;
    return __builtin_bit_cast(half8_t, r);
}

// K % 256 == 0, w and x 16-byte aligned.  NB = number of 16-vector column blocks.
// grid = (row tiles, K slices); slice s covers chunks [s * cps, min((s + 1) * cps, K / 256)).
// SWIGLU: W is [gate rows; up rows] (M = 2 * inter); a wave takes 8 gate rows and the 8 up rows
// of the same indices, and the epilogue writes pack(fp16(silu(gate) * up)) as FP8 words to
// `packed` ([nvec, inter / 4]) instead of fp32 sums to `out` (one K slice only).
// KG: K groups per workgroup (1 or 2); every slice must hold a multiple of KG chunks.
// ROT: rotated K walk (long walks only, see below).
template <int MODE, int NB, bool SWIGLU, int KG, bool ROT = false>
__global__ __launch_bounds__(kBgThreads * KG) void gemv_batched_kernel(const uint8_t *__restrict__ w,
                                                                 const uint8_t *__restrict__ x,
                                                                 float *__restrict__ out, int M, int K, int nvec,
                                                                 int cps, int64_t part_stride,
                                                                 uint32_t *__restrict__ packed,
                                                                 float *__restrict__ act_f32) {
    extern __shared__ __attribute__((aligned(16))) _Float16 xs_all[];   // [KG][2][16 * NB][kBgPitch]
    const int lane = threadIdx.x & 63;
    const int grp = KG == 1 ? 0 : wave_id() / 4, wave = KG == 1 ? wave_id() : wave_id() % 4;
    const int tig = threadIdx.x - kBgThreads * grp;              // thread index inside its K group
    _Float16 *const xs = xs_all + grp * (2 * 16 * NB * kBgPitch);
    const int j = lane & 15, kb = lane >> 4;
    const int row0 = blockIdx.x * kBgRows + 16 * wave;
    const int inter = M / 2;
    const int g0 = blockIdx.x * (kBgRows / 2) + 8 * wave;        // SWIGLU: first of this wave's 8 gate rows
    const int row = SWIGLU ? (j < 8 ? min(g0 + j, inter - 1) : inter + min(g0 + j - 8, inter - 1)) : min(row0 + j, M - 1);
    const int n_chunks = K / kBgChunk;
    const int c_begin = blockIdx.y * cps, c_end = min(c_begin + cps, n_chunks);
    const uint8_t *wp = w + (int64_t)row * K + 16 * kb;
    // this thread's share of the vectors' chunk: 16-byte piece (vec, col16) = (piece / 16, piece % 16)
    // (columns of vectors past nvec are filled from the last vector: their sums are never stored, and a column of
    // the MFMA result depends on its own vector only, so the loads need no lane mask)
    const uint8_t *xp[NB];
    int xdst[NB];
#pragma unroll
    for (int i = 0; i < NB; i++) {
        int piece = tig + kBgThreads * i;
        int vec = piece >> 4, col16 = piece & 15;
        xp[i] = x + (int64_t)min(vec, nvec - 1) * K + 16 * col16;
        xdst[i] = vec * kBgPitch + 16 * col16;
    }
    float4_t acc[NB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) acc[nb] = float4_t{0.f, 0.f, 0.f, 0.f};

    u32x4 wa[4], xa[NB];
    auto issue = [&](int c, u32x4 (&wr)[4], u32x4 (&xr)[NB]) {
        const int64_t col = (int64_t)c * kBgChunk;
#pragma unroll
        for (int u = 0; u < 4; u++) wr[u] = *reinterpret_cast<const u32x4 *>(wp + col + 64 * u);
#pragma unroll
        for (int i = 0; i < NB; i++) xr[i] = *reinterpret_cast<const u32x4 *>(xp[i] + col);
    };
    // One chunk: vectors' chunk -> LDS, (the caller's prefetch goes here), barrier, MFMAs.
    auto stage_x = [&](int it, const u32x4 (&xr)[NB]) {
        _Float16 *buf = xs + ((it / KG) & 1) * (16 * NB * kBgPitch);
#pragma unroll
        for (int i = 0; i < NB; i++) {
            *reinterpret_cast<half8_t *>(buf + xdst[i]) = bg_dec8<MODE>(xr[i].x, xr[i].y);
            *reinterpret_cast<half8_t *>(buf + xdst[i] + 8) = bg_dec8<MODE>(xr[i].z, xr[i].w);
        }
        return buf;
    };
    auto mac = [&](const _Float16 *buf, const u32x4 (&wr)[4]) {
#pragma unroll
        for (int u = 0; u < 4; u++) {
            half8_t a0 = bg_dec8<MODE>(wr[u].x, wr[u].y), a1 = bg_dec8<MODE>(wr[u].z, wr[u].w);
#pragma unroll
            for (int nb = 0; nb < NB; nb++) {
                const _Float16 *b = buf + (16 * nb + j) * kBgPitch + 64 * u + 16 * kb;
                acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, *reinterpret_cast<const half8_t *>(b), acc[nb], 0, 0, 0);
                acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, *reinterpret_cast<const half8_t *>(b + 8), acc[nb], 0, 0, 0);
            }
        }
    };
    if (c_begin >= c_end) return;                  // cannot happen: the launcher creates no empty slice
    // ROT: every row tile starts its K walk at another chunk and wraps around.  With a common start all
    // workgroups read the same column offsets at the same time, addresses that differ by multiples of
    // the row pitch and fall on few memory channels (16384 x 16384, 32 vectors, E5M2: 72 -> 56 us).
    // Walks of a few chunks gain nothing from it and keep the plain order.
    const int n_it = c_end - c_begin;              // a multiple of KG
    const int rot = ROT ? (int)((blockIdx.x * 7u) % (unsigned)(n_it / KG)) * KG : 0;
    auto chunk_of = [&](int it) {
        if constexpr (!ROT) return c_begin + it;
        int t = it + rot;
        return c_begin + (t >= n_it ? t - n_it : t);
    };
    issue(chunk_of(grp), wa, xa);
    // Every chunk but the last prefetches its successor unconditionally, so the number of loads
    // in flight is known at compile time and the wait for chunk c leaves chunk c + 1 outstanding
    // (a prefetch inside an `if` makes the compiler wait for everything).
    // The loop is unrolled by two so that the two register sets swap roles without copies.
    u32x4 wb[4], xb[NB];
    auto step = [&](int it, const u32x4 (&wc)[4], const u32x4 (&xc)[NB], u32x4 (&wn)[4], u32x4 (&xn)[NB]) {
        const _Float16 *buf = stage_x(it, xc);
        issue(chunk_of(it + KG), wn, xn);
        __syncthreads();
        mac(buf, wc);
    };
    auto last = [&](const u32x4 (&wc)[4], const u32x4 (&xc)[NB]) {
        const _Float16 *buf = stage_x(n_it - KG + grp, xc);
        __syncthreads();
        mac(buf, wc);
    };
    int it = grp;
    for (; it + KG < n_it - KG; it += 2 * KG) {
        step(it, wa, xa, wb, xb);
        step(it + KG, wb, xb, wa, xa);
    }
    if (it < n_it - KG) {
        step(it, wa, xa, wb, xb);
        last(wb, xb);
    } else {
        last(wa, xa);
    }
    if constexpr (KG > 1) {
        // groups 1.. -> group 0 through LDS (the vectors' buffers are free once every wave is past its MFMAs)
        float *red = reinterpret_cast<float *>(xs_all);
        __syncthreads();
        if (grp > 0) {
#pragma unroll
            for (int nb = 0; nb < NB; nb++)
#pragma unroll
                for (int i = 0; i < 4; i++) red[((grp - 1) * 4 * NB + 4 * nb + i) * kBgThreads + tig] = acc[nb][i];
        }
        __syncthreads();
        if (grp > 0) return;
#pragma unroll
        for (int g = 1; g < KG; g++)
#pragma unroll
            for (int nb = 0; nb < NB; nb++)
#pragma unroll
                for (int i = 0; i < 4; i++) acc[nb][i] += red[((g - 1) * 4 * NB + 4 * nb + i) * kBgThreads + tig];
    }
    if constexpr (SWIGLU) {
        // accumulator rows 4 kb + {0..3}: kb 0, 1 hold gate rows g0 + 4 kb + i, kb 2, 3 the up rows of
        // the same indices, 32 lanes further on
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
            float u[4];
#pragma unroll
            for (int i = 0; i < 4; i++) u[i] = __shfl_xor(acc[nb][i], 32, kWave);
            const int vec = 16 * nb + j, g = g0 + 4 * kb;
            if (kb < 2 && vec < nvec && g < inter) {
                // silu(a) * b with the hardware exponential and reciprocal (1-2 ulp from the library's
                // expf and IEEE division, which took most of this epilogue's 1.8 us)
                auto f = [](float a, float b) {
                    return a * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * a)) * b;
                };
                const float4_t a = float4_t{f(acc[nb][0], u[0]), f(acc[nb][1], u[1]), f(acc[nb][2], u[2]), f(acc[nb][3], u[3])};
                packed[(int64_t)vec * (inter / 4) + g / 4] = quant4<MODE>(a[0], a[1], a[2], a[3]);
                if (act_f32) *reinterpret_cast<float4_t *>(act_f32 + (int64_t)vec * inter + g) = a;   // the values the codes were rounded from
            }
        }
        return;
    }
    float *o_base = out + (int64_t)blockIdx.y * part_stride;
    const int r = row0 + 4 * kb;                   // accumulator rows 4 kb + {0..3}, column = vector
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
        int vec = 16 * nb + j;
        if (vec < nvec) {
            float *o = o_base + (int64_t)vec * M + r;
            if (r + 3 < M && (M & 3) == 0) {
                *reinterpret_cast<float4_t *>(o) = acc[nb];
            } else {
#pragma unroll
                for (int i = 0; i < 4; i++)
                    if (r + i < M) o[i] = acc[nb][i];
            }
        }
    }
}

template <int MODE, int NB, bool SWIGLU, int KG, bool ROT = false>
static void bg_launch_kg(const void *w, const void *x, float *out, int M, int K, int nvec, int splits, int cps,
                         int64_t part_stride, uint32_t *packed, float *act_f32, hipStream_t s) {
    const size_t lds = (size_t)KG * 2 * 16 * NB * kBgPitch * sizeof(_Float16);
    static unsigned long long lds_raised = 0;      // per instantiation, one bit per device
    (void)raise_lds_limit(reinterpret_cast<const void *>(&gemv_batched_kernel<MODE, NB, SWIGLU, KG, ROT>), lds, lds_raised);
    hipLaunchKernelGGL((gemv_batched_kernel<MODE, NB, SWIGLU, KG, ROT>),
                       dim3((unsigned)((M + kBgRows - 1) / kBgRows), (unsigned)splits), dim3(kBgThreads * KG), lds, s,
                       (const uint8_t *)w, (const uint8_t *)x, out, M, K, nvec, cps, part_stride, packed, act_f32);
}

// Two K groups per workgroup when every slice (the last one too) gives each group at least two chunks
// and either the grid does not fill the chip twice over or the K walk is long.  Measured at 32 vectors,
// E4M3: 16384 x 16384 90.7 -> 71.4 us, 11264 x 2048 11.1 -> 9.5 us, but 32000 x 2048 (500 workgroups of
// 8 chunks) 18.1 -> 18.7 us; four groups (1024 threads) were slower than two on every shape tried.
template <int MODE, int NB, bool SWIGLU>
static void bg_launch(const void *w, const void *x, float *out, int M, int K, int nvec, int splits, int cps,
                      int64_t part_stride, uint32_t *packed, float *act_f32, hipStream_t s) {
    const int last = K / kBgChunk - (splits - 1) * cps;   // chunks of the last slice
    const int64_t groups = (int64_t)((M + kBgRows - 1) / kBgRows) * splits;
    const bool two = cps >= 4 && cps % 2 == 0 && last % 2 == 0 && (groups <= 256 || cps >= 16);
    if constexpr (!SWIGLU) {
        if (cps >= 32 && last >= 32) {             // long K walk: rotated start per row tile
            if (two) bg_launch_kg<MODE, NB, false, 2, true>(w, x, out, M, K, nvec, splits, cps, part_stride, packed, act_f32, s);
            else bg_launch_kg<MODE, NB, false, 1, true>(w, x, out, M, K, nvec, splits, cps, part_stride, packed, act_f32, s);
            return;
        }
    }
    if (two)
        bg_launch_kg<MODE, NB, SWIGLU, 2>(w, x, out, M, K, nvec, splits, cps, part_stride, packed, act_f32, s);
    else
        bg_launch_kg<MODE, NB, SWIGLU, 1>(w, x, out, M, K, nvec, splits, cps, part_stride, packed, act_f32, s);
}

int gemv_batched_launch(const void *w, const void *x, float *out_f32, int64_t M, int64_t K, int64_t nvec, int mode,
                        int splits, int64_t part_stride, int *splits_out, hipStream_t stream) {
    const int n_chunks = (int)(K / kBgChunk);
    splits = splits < 1 ? 1 : (splits > n_chunks ? n_chunks : splits);
    const int cps = (n_chunks + splits - 1) / splits;
    splits = (n_chunks + cps - 1) / cps;           // no empty slice
    if (splits_out) *splits_out = splits;
    const int nb = (int)((nvec + 15) / 16);
#define FEATHER_BG(MM, NBB) bg_launch<MM, NBB, false>(w, x, out_f32, (int)M, (int)K, (int)nvec, splits, cps, part_stride, nullptr, nullptr, stream)
    if (mode == FEATHER_E5M2) {
        switch (nb) { case 1: FEATHER_BG(FEATHER_E5M2, 1); break; case 2: FEATHER_BG(FEATHER_E5M2, 2); break;
                      case 3: FEATHER_BG(FEATHER_E5M2, 3); break; default: FEATHER_BG(FEATHER_E5M2, 4); }
    } else {
        switch (nb) { case 1: FEATHER_BG(FEATHER_E4M3, 1); break; case 2: FEATHER_BG(FEATHER_E4M3, 2); break;
                      case 3: FEATHER_BG(FEATHER_E4M3, 3); break; default: FEATHER_BG(FEATHER_E4M3, 4); }
    }
#undef FEATHER_BG
    return check_launch("feather_gemv_fp8_batched");
}

// act = pack(fp16(silu(W_gate x) * (W_up x))) with w = [gate rows; up rows] ([2 * inter, K]); the
// GEMV and the activation in one kernel, no fp32 round trip.  Needs K % 256 == 0, inter % 4 == 0.
int gemv_batched_swiglu_launch(const void *w, const void *x, uint32_t *act_packed, float *act_f32, int64_t inter,
                               int64_t K, int64_t nvec, int mode, hipStream_t stream) {
    const int n_chunks = (int)(K / kBgChunk);
    const int nb = (int)((nvec + 15) / 16);
#define FEATHER_BG(MM, NBB) \
    bg_launch<MM, NBB, true>(w, x, nullptr, (int)(2 * inter), (int)K, (int)nvec, 1, n_chunks, 0, act_packed, act_f32, stream)
    if (mode == FEATHER_E5M2) {
        switch (nb) { case 1: FEATHER_BG(FEATHER_E5M2, 1); break; case 2: FEATHER_BG(FEATHER_E5M2, 2); break;
                      case 3: FEATHER_BG(FEATHER_E5M2, 3); break; default: FEATHER_BG(FEATHER_E5M2, 4); }
    } else {
        switch (nb) { case 1: FEATHER_BG(FEATHER_E4M3, 1); break; case 2: FEATHER_BG(FEATHER_E4M3, 2); break;
                      case 3: FEATHER_BG(FEATHER_E4M3, 3); break; default: FEATHER_BG(FEATHER_E4M3, 4); }
    }
#undef FEATHER_BG
    return check_launch("feather_decode_step (gate_up + swiglu)");
}

}  // namespace feather

using namespace feather;

extern "C" int feather_gemv_fp8_batched(const void *w, const void *x, void *out_f32, int64_t M, int64_t K,
                                        int64_t nvec, int mode, void *stream) {
    const char *me = "feather_gemv_fp8_batched";
    FEATHER_CHECK(mode == FEATHER_E5M2 || mode == FEATHER_E4M3, FEATHER_EMODE, "%s: mode %d not supported", me, mode);
    FEATHER_CHECK(M >= 0 && K >= 0, FEATHER_EINVAL, "%s: negative shape", me);
    FEATHER_CHECK(nvec >= 1 && nvec <= 64, FEATHER_ESHAPE, "%s: nvec=%lld outside [1, 64]", me, (long long)nvec);
    FEATHER_CHECK(K % 4 == 0, FEATHER_ESHAPE, "%s: K=%lld is not a multiple of 4", me, (long long)K);
    FEATHER_CHECK(M < (1ll << 31) && K < (1ll << 31), FEATHER_ESHAPE, "%s: shape too large", me);
    if (M == 0) return FEATHER_OK;
    FEATHER_CHECK(w && x && out_f32, FEATHER_EINVAL, "%s: null pointer", me);
    FEATHER_CHECK(aligned(w, 4) && aligned(x, 4) && aligned(out_f32, 16), FEATHER_EINVAL, "%s: misaligned pointer", me);
    if (K % kBgChunk != 0 || K == 0 || !aligned(w, 16) || !aligned(x, 16)) {
        // shapes the MFMA path does not cover: one streaming GEMV per vector
        for (int64_t b = 0; b < nvec; b++) {
            int rc = feather_gemv_fp8(w, (const uint8_t *)x + b * K, (float *)out_f32 + b * M, M, K, mode, stream);
            if (rc != FEATHER_OK) return rc;
        }
        return FEATHER_OK;
    }
    return gemv_batched_launch(w, x, (float *)out_f32, M, K, nvec, mode, 1, 0, nullptr, (hipStream_t)stream);
}

extern "C" int feather_gemv_fp8_batched_swiglu(const void *w_gate_up, const void *x, void *act_packed, void *act_f32,
                                               int64_t inter, int64_t K, int64_t nvec, int mode, void *stream) {
    const char *me = "feather_gemv_fp8_batched_swiglu";
    FEATHER_CHECK(mode == FEATHER_E5M2 || mode == FEATHER_E4M3, FEATHER_EMODE, "%s: mode %d not supported", me, mode);
    FEATHER_CHECK(inter >= 0 && K >= 0, FEATHER_EINVAL, "%s: negative shape", me);
    FEATHER_CHECK(nvec >= 1 && nvec <= 64, FEATHER_ESHAPE, "%s: nvec=%lld outside [1, 64]", me, (long long)nvec);
    FEATHER_CHECK(K > 0 && K % kBgChunk == 0, FEATHER_ESHAPE, "%s: K=%lld is not a positive multiple of %d", me, (long long)K,
                  kBgChunk);
    FEATHER_CHECK(inter % 4 == 0, FEATHER_ESHAPE, "%s: inter=%lld is not a multiple of 4", me, (long long)inter);
    FEATHER_CHECK(2 * inter < (1ll << 31) && K < (1ll << 31), FEATHER_ESHAPE, "%s: shape too large", me);
    if (inter == 0) return FEATHER_OK;
    FEATHER_CHECK(w_gate_up && x && act_packed, FEATHER_EINVAL, "%s: null pointer", me);
    FEATHER_CHECK(aligned(w_gate_up, 16) && aligned(x, 16) && aligned(act_packed, 4) && aligned(act_f32, 16), FEATHER_EINVAL,
                  "%s: misaligned pointer", me);
    return gemv_batched_swiglu_launch(w_gate_up, x, (uint32_t *)act_packed, (float *)act_f32, inter, K, nvec, mode,
                                      (hipStream_t)stream);
}
