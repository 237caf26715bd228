// Packed dot products (FP8 E5M2 / E4M3 and FP16 containers), fp32 accumulate.
//
// Both operands stream from HBM once (2 x 4 bytes per word pair); each lane
// reads 128-bit chunks of both vectors, decodes in registers and accumulates
// with v_dot2_f32_f16.  The reduction is deterministic: every workgroup writes
// one partial to scratch and a second one-wave kernel adds the partials in
// index order; an input that a single workgroup covers (up to 4096 words) is
// finished by that workgroup and needs no second launch.  (A single-kernel "last workgroup finishes" scheme needs
// device-scope release/acquire around the arrival counter, which on this
// multi-XCD part costs an L2 write-back/invalidate per workgroup and measured
// ~45 us for 2^24 elements; the second launch costs a few us.  The same scheme
// with relaxed device-scope atomics only (partial published by an exchange,
// ticket drawn after it returned, partials read back with atomic loads) gives
// correct sums without fences, but the tickets serialise at the memory side:
// 22 us with 1024 workgroups, 11-14 us with 256, no better than two launches.)
#include "common.h"

namespace feather {

constexpr int kDotThreads = 256;
constexpr int kDotMaxBlocks = 4096;
constexpr int kDotUnroll = 1;
// scratch layout: [64 B ..) kDotMaxBlocks fp32 partials (the first 64 B are unused padding)
constexpr int64_t kDotScratchBytes = 64 + (int64_t)kDotMaxBlocks * 4;

enum DotKind { kDotE5M2 = 0, kDotE4M3 = 1, kDotF16 = 2, kDotF16Wide = 3 };

// fp16 container word pair: fp16(lo1*lo2) +fp16 fp16(hi1*hi2), widened to fp32
// (reference dot.py:134-141).  Contraction is off so the two products and the
// sum are each rounded to fp16, as separate Triton fp16 ops are.
__device__ __forceinline__ float f16_word_term(uint32_t a, uint32_t b) {
#pragma clang fp contract(off)
    half2_t p = as_half2(a) * as_half2(b);
    _Float16 s = p.x + p.y;
    return (float)s;
}

template <int KIND>
__device__ __forceinline__ float mac_word(uint32_t a, uint32_t b, float acc) {
    if constexpr (KIND == kDotF16) {
        return acc + f16_word_term(a, b);
    } else if constexpr (KIND == kDotF16Wide) {
        return dot2(a, b, acc);  // the container word already is an fp16 pair
    } else {
        uint32_t p, q, x, y;
        dec_word<KIND>(a, p, q);
        dec_word<KIND>(b, x, y);
        acc = dot2(p, x, acc);
        return dot2(q, y, acc);
    }
}

template <int KIND, bool VEC>
__global__ __launch_bounds__(kDotThreads) void dot_kernel(const uint32_t *__restrict__ x1,
                                                         const uint32_t *__restrict__ x2, float *__restrict__ out,
                                                         uint32_t *__restrict__ scratch, int64_t n_words) {
    __shared__ float wave_part[kDotThreads / kWave];
    float acc[kDotUnroll];
#pragma unroll
    for (int u = 0; u < kDotUnroll; u++) acc[u] = 0.f;

    const int64_t tid = (int64_t)blockIdx.x * kDotThreads + threadIdx.x;
    const int64_t nthreads = (int64_t)gridDim.x * kDotThreads;
    int64_t done = 0;
    if constexpr (VEC) {
        const int64_t n4 = n_words / 4;
        const u32x4 *a4 = reinterpret_cast<const u32x4 *>(x1);
        const u32x4 *b4 = reinterpret_cast<const u32x4 *>(x2);
        for (int64_t i = tid; i < n4; i += nthreads * kDotUnroll) {
            u32x4 a[kDotUnroll], b[kDotUnroll];
#pragma unroll
            for (int u = 0; u < kDotUnroll; u++) {
                int64_t j = i + u * nthreads;
                a[u] = u32x4{0, 0, 0, 0};
                b[u] = u32x4{0, 0, 0, 0};
                if (j < n4) {
                    a[u] = load_nt128(a4 + j);
                    b[u] = load_nt128(b4 + j);
                }
            }
#pragma unroll
            for (int u = 0; u < kDotUnroll; u++) {
                acc[u] = mac_word<KIND>(a[u].x, b[u].x, acc[u]);
                acc[u] = mac_word<KIND>(a[u].y, b[u].y, acc[u]);
                acc[u] = mac_word<KIND>(a[u].z, b[u].z, acc[u]);
                acc[u] = mac_word<KIND>(a[u].w, b[u].w, acc[u]);
            }
        }
        done = n4 * 4;
    }
    for (int64_t j = done + tid; j < n_words; j += nthreads) acc[0] = mac_word<KIND>(x1[j], x2[j], acc[0]);

    float tot = acc[0];                                     // fixed order of the per-thread sums
#pragma unroll
    for (int u = 1; u < kDotUnroll; u++) tot += acc[u];
    float s = wave_sum(tot);
    const int lane = lane_id(), wave = wave_id();
    if (lane == 0) wave_part[wave] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        float t = 0.f;
#pragma unroll
        for (int w = 0; w < kDotThreads / kWave; w++) t += wave_part[w];
        // a single workgroup holds the whole sum: no second kernel (the launch is half of a short dot's time)
        if (gridDim.x == 1) out[0] = t;
        else reinterpret_cast<float *>(scratch + 16)[blockIdx.x] = t;
    }
}

// One workgroup adds the partials in a fixed order: thread t takes t, t + 256, ... (every load is
// issued before the first add: a loop of dependent loads pays one memory round trip per turn and
// made this kernel take 5.7 us for 1024 partials), then the wave fold, then the waves in order.
constexpr int kFinishThreads = 256;
__global__ __launch_bounds__(kFinishThreads) void dot_finish_kernel(const uint32_t *__restrict__ scratch,
                                                                   float *__restrict__ out, int n_partials) {
    __shared__ float wave_part[kFinishThreads / kWave];
    const float *partials = reinterpret_cast<const float *>(scratch + 16);
    constexpr int kPer = kDotMaxBlocks / kFinishThreads;
    float v[kPer];
#pragma unroll
    for (int k = 0; k < kPer; k++) v[k] = partials[min((int)threadIdx.x + kFinishThreads * k, n_partials - 1)];
    float t = 0.f;
#pragma unroll
    for (int k = 0; k < kPer; k++)
        if ((int)threadIdx.x + kFinishThreads * k < n_partials) t += v[k];
    t = wave_sum(t);
    if (lane_id() == 0) wave_part[wave_id()] = t;
    __syncthreads();
    if (threadIdx.x == 0) {
        float r = 0.f;
#pragma unroll
        for (int w = 0; w < kFinishThreads / kWave; w++) r += wave_part[w];
        out[0] = r;
    }
}

template <int KIND>
static int launch_dot(const void *x1, const void *x2, void *out, void *scratch, int64_t n_words, hipStream_t s,
                      const char *what) {
    bool vec = aligned(x1, 16) && aligned(x2, 16) && n_words >= 4;
    int64_t per_block = (int64_t)kDotThreads * 4 * kDotUnroll;  // words per workgroup per sweep
    int64_t blocks = (n_words + per_block - 1) / per_block;
    if (blocks > kDotMaxBlocks) blocks = kDotMaxBlocks;
    if (blocks < 1) blocks = 1;
    if (vec)
        hipLaunchKernelGGL((dot_kernel<KIND, true>), dim3((unsigned)blocks), dim3(kDotThreads), 0, s,
                           (const uint32_t *)x1, (const uint32_t *)x2, (float *)out, (uint32_t *)scratch, n_words);
    else
        hipLaunchKernelGGL((dot_kernel<KIND, false>), dim3((unsigned)blocks), dim3(kDotThreads), 0, s,
                           (const uint32_t *)x1, (const uint32_t *)x2, (float *)out, (uint32_t *)scratch, n_words);
    int rc = check_launch(what);
    if (rc != FEATHER_OK || blocks == 1) return rc;
    hipLaunchKernelGGL(dot_finish_kernel, dim3(1), dim3(kFinishThreads), 0, s, (const uint32_t *)scratch, (float *)out,
                       (int)blocks);
    return check_launch(what);
}

static int check_dot_args(const void *x1, const void *x2, const void *out, const void *scratch, int64_t n_words,
                          const char *what) {
    FEATHER_CHECK(n_words >= 0, FEATHER_EINVAL, "%s: negative n_words", what);
    FEATHER_CHECK(out && scratch, FEATHER_EINVAL, "%s: null out/scratch", what);
    FEATHER_CHECK(n_words == 0 || (x1 && x2), FEATHER_EINVAL, "%s: null input", what);
    FEATHER_CHECK(aligned(x1, 4) && aligned(x2, 4) && aligned(out, 4) && aligned(scratch, 64), FEATHER_EINVAL,
                  "%s: misaligned pointer", what);
    return FEATHER_OK;
}

}  // namespace feather

using namespace feather;

extern "C" int64_t feather_dot_scratch_bytes(void) { return kDotScratchBytes; }

extern "C" int feather_dot_fp8(const void *x1, const void *x2, void *out_f32, void *scratch, int64_t n_words, int mode,
                               void *stream) {
    FEATHER_CHECK(mode == FEATHER_E5M2 || mode == FEATHER_E4M3, FEATHER_EMODE, "feather_dot_fp8: mode %d not supported",
                  mode);
    int rc = check_dot_args(x1, x2, out_f32, scratch, n_words, "feather_dot_fp8");
    if (rc != FEATHER_OK) return rc;
    hipStream_t s = (hipStream_t)stream;
    if (mode == FEATHER_E5M2) return launch_dot<kDotE5M2>(x1, x2, out_f32, scratch, n_words, s, "feather_dot_fp8");
    return launch_dot<kDotE4M3>(x1, x2, out_f32, scratch, n_words, s, "feather_dot_fp8");
}

extern "C" int feather_dot_fp16(const void *x1, const void *x2, void *out_f32, void *scratch, int64_t n_words,
                                int fp16_products, void *stream) {
    int rc = check_dot_args(x1, x2, out_f32, scratch, n_words, "feather_dot_fp16");
    if (rc != FEATHER_OK) return rc;
    if (fp16_products)
        return launch_dot<kDotF16>(x1, x2, out_f32, scratch, n_words, (hipStream_t)stream, "feather_dot_fp16");
    return launch_dot<kDotF16Wide>(x1, x2, out_f32, scratch, n_words, (hipStream_t)stream, "feather_dot_fp16");
}
