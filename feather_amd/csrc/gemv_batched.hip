// Batched packed-FP8 GEMV (skinny GEMM): out[b, r] = sum_k dec(w[r,k]) * dec(x[b,k])
// for up to 64 vectors, streaming the weight matrix once for the whole batch.
//
// With more than a couple of vectors the per-element multiply count rules out
// the VALU, so the product runs on the matrix cores: a 16-row slab of W is the
// A operand of v_mfma_f32_16x16x32_f16 and 16 vectors are the B columns.  A
// lane loads 16 consecutive codes of one row (128-bit load, 64 B contiguous per
// row across the 4 lanes that share it) and decodes them in registers; the
// vectors (a few hundred KB at most, L2 resident) are read the same way.
// One workgroup owns 16 rows; its 4 waves split K and reduce through LDS in a
// fixed order, so results are deterministic.  (Handing the vectors over as
// already-decoded fp16 instead of packed codes was measured and dropped: it
// doubles the vector bytes every workgroup pulls from L2 and ran 10-40 % slower.)
#include "common.h"

namespace feather {

constexpr int kBgThreads = 256;

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

// K % 256 == 0 (64 columns per wave step, 4 waves), w and x 16-byte aligned.  NB = number of
// 16-vector column blocks.
template <int MODE, int NB>
__global__ __launch_bounds__(kBgThreads) void gemv_batched_kernel(const uint8_t *__restrict__ w,
                                                                 const uint8_t *__restrict__ x,
                                                                 float *__restrict__ out, int M, int K, int nvec) {
    __shared__ float4_t red[3][NB][kWave];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int j = lane & 15, kb = lane >> 4;
    const int row0 = blockIdx.x * 16;
    const int row = min(row0 + j, M - 1);
    const int kq = K / 4;                      // this wave's share of K
    const uint8_t *wp = w + (int64_t)row * K + wave * kq + 16 * kb;
    const uint8_t *xp[NB];
    bool xok[NB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
        int vec = 16 * nb + j;
        xok[nb] = vec < nvec;
        xp[nb] = x + (int64_t)min(vec, nvec - 1) * K + wave * kq + 16 * kb;
    }
    float4_t acc[NB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) acc[nb] = float4_t{0.f, 0.f, 0.f, 0.f};

    constexpr int UN = 4;                      // 64-column steps whose loads are issued together
    for (int c = 0; c < kq; c += 64 * UN) {
        u32x4 a[UN], b[UN][NB];
#pragma unroll
        for (int u = 0; u < UN; u++) {
            const bool in = c + 64 * u < kq;
            a[u] = in ? load_nt128(wp + c + 64 * u) : u32x4{0, 0, 0, 0};
#pragma unroll
            for (int nb = 0; nb < NB; nb++)
                b[u][nb] = in && xok[nb] ? *reinterpret_cast<const u32x4 *>(xp[nb] + c + 64 * u) : u32x4{0, 0, 0, 0};
        }
#pragma unroll
        for (int u = 0; u < UN; u++) {
            half8_t a0 = bg_dec8<MODE>(a[u].x, a[u].y), a1 = bg_dec8<MODE>(a[u].z, a[u].w);
#pragma unroll
            for (int nb = 0; nb < NB; nb++) {
                acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, bg_dec8<MODE>(b[u][nb].x, b[u][nb].y), acc[nb], 0, 0, 0);
                acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, bg_dec8<MODE>(b[u][nb].z, b[u][nb].w), acc[nb], 0, 0, 0);
            }
        }
    }
    if (wave > 0) {
#pragma unroll
        for (int nb = 0; nb < NB; nb++) red[wave - 1][nb][lane] = acc[nb];
    }
    __syncthreads();
    if (wave == 0) {
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
            float4_t s = acc[nb];
            s += red[0][nb][lane];
            s += red[1][nb][lane];
            s += red[2][nb][lane];
            int vec = 16 * nb + j;
            int r = row0 + 4 * kb;             // accumulator rows 4 kb + {0..3}, column = vector
            if (vec < nvec) {
                float *o = out + (int64_t)vec * M + r;
                if (r + 3 < M && (M & 3) == 0) {
                    *reinterpret_cast<float4_t *>(o) = s;
                } else {
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        if (r + i < M) o[i] = s[i];
                }
            }
        }
    }
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
    hipStream_t s = (hipStream_t)stream;
    if (K % 256 != 0 || K == 0 || !aligned(w, 16) || !aligned(x, 16)) {
        // shapes the MFMA path does not cover: one streaming GEMV per vector
        for (int64_t b = 0; b < nvec; b++) {
            int rc = feather_gemv_fp8(w, (const uint8_t *)x + b * K, (float *)out_f32 + b * M, M, K, mode, stream);
            if (rc != FEATHER_OK) return rc;
        }
        return FEATHER_OK;
    }
    unsigned blocks = (unsigned)((M + 15) / 16);
    int nb = (int)((nvec + 15) / 16);
#define FEATHER_BG(MM, NBB)                                                                                        \
    hipLaunchKernelGGL((gemv_batched_kernel<MM, NBB>), dim3(blocks), dim3(kBgThreads), 0, s, (const uint8_t *)w,  \
                       (const uint8_t *)x, (float *)out_f32, (int)M, (int)K, (int)nvec)
    if (mode == FEATHER_E5M2) {
        switch (nb) { case 1: FEATHER_BG(FEATHER_E5M2, 1); break; case 2: FEATHER_BG(FEATHER_E5M2, 2); break;
                      case 3: FEATHER_BG(FEATHER_E5M2, 3); break; default: FEATHER_BG(FEATHER_E5M2, 4); }
    } else {
        switch (nb) { case 1: FEATHER_BG(FEATHER_E4M3, 1); break; case 2: FEATHER_BG(FEATHER_E4M3, 2); break;
                      case 3: FEATHER_BG(FEATHER_E4M3, 3); break; default: FEATHER_BG(FEATHER_E4M3, 4); }
    }
#undef FEATHER_BG
    return check_launch(me);
}
