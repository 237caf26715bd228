// Pack / unpack kernels: fp16 -> four FP8 codes per 32-bit word and back, and
// the two-fp16-per-word container.  All are pure streaming kernels bound by HBM
// bandwidth (pack: 2 B in + 1 B out per element; unpack to fp32: 1 B in + 4 B
// out), so the work is laid out for full-width coalesced accesses: one lane
// converts 16 consecutive elements from two 128-bit loads into one 128-bit
// store.
#include <stdarg.h>
#include <stdio.h>

#include "common.h"

namespace feather {

// ---------------------------------------------------------------- error state

static thread_local char g_err[256] = "";

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

// two fp16 (one 32-bit register) -> two codes in bits [0,16)
template <int MODE, int ROUND>
__device__ __forceinline__ uint32_t enc_pair(uint32_t hh) {
    return enc<MODE, ROUND>(hh & 0xFFFFu) | (enc<MODE, ROUND>(hh >> 16) << 8);
}

// ---------------------------------------------------------------- pack fp8

// Vector body: thread t converts elements [16t, 16t+16) (n16 such groups).
// Scalar tail: the remaining n - 16*n16 elements, one word per thread with
// zero padding, handled by the first threads of the grid.
template <int MODE, int ROUND, bool ALIGNED>
__global__ __launch_bounds__(256) void pack_fp8_kernel(const uint16_t *__restrict__ src, uint32_t *__restrict__ dst,
                                                      int64_t n, int64_t n16) {
    int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t g = t; g < n16; g += stride) {
        uint32_t in[8];
        if constexpr (ALIGNED) {
            const u32x4 *p = reinterpret_cast<const u32x4 *>(src) + 2 * g;
            u32x4 a = load_nt128(p), b = load_nt128(p + 1);
            in[0] = a.x; in[1] = a.y; in[2] = a.z; in[3] = a.w;
            in[4] = b.x; in[5] = b.y; in[6] = b.z; in[7] = b.w;
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++)
                in[i] = (uint32_t)src[16 * g + 2 * i] | ((uint32_t)src[16 * g + 2 * i + 1] << 16);
        }
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            if constexpr (MODE == FEATHER_E4M3 && ROUND == FEATHER_ROUND_RNE)   // codes in bytes 0 and 2 of each register
                w[i] = perm(enc_e4m3_pair(in[2 * i + 1]), enc_e4m3_pair(in[2 * i]), 0x06040200u);
            else
                w[i] = enc_pair<MODE, ROUND>(in[2 * i]) | (enc_pair<MODE, ROUND>(in[2 * i + 1]) << 16);
        }
        if constexpr (ALIGNED) {
            store_nt128(reinterpret_cast<u32x4 *>(dst) + g, u32x4{w[0], w[1], w[2], w[3]});
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++) dst[4 * g + i] = w[i];
        }
    }
    // tail words
    int64_t first = 16 * n16;
    int64_t tail_words = (n - first + 3) / 4;
    if (t < tail_words) {
        uint32_t w = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int64_t idx = first + 4 * t + i;
            uint32_t h = idx < n ? src[idx] : 0u;
            w |= enc<MODE, ROUND>(h) << (8 * i);
        }
        dst[first / 4 + t] = w;
    }
}

template <int MODE, int ROUND>
static int launch_pack(const void *src, void *dst, int64_t n, hipStream_t s) {
    int64_t n16 = n / 16;
    bool al = aligned(src, 16) && aligned(dst, 16);
    // One 16-element group per thread and as many workgroups as that takes: a grid capped at 4096 workgroups that
    // strides over the input reached 5.2 TB/s on 134 M elements, one group per thread 6.1 TB/s (the loop in the kernel
    // only runs more than once beyond 2^31 workgroups).
    int64_t threads_needed = n16 > 4 ? n16 : 4;
    int64_t blocks = (threads_needed + 255) / 256;
    if (blocks > 0x7FFFFFFF) blocks = 0x7FFFFFFF;
    if (blocks < 1) blocks = 1;
    if (al)
        hipLaunchKernelGGL((pack_fp8_kernel<MODE, ROUND, true>), dim3((unsigned)blocks), dim3(256), 0, s,
                           (const uint16_t *)src, (uint32_t *)dst, n, n16);
    else
        hipLaunchKernelGGL((pack_fp8_kernel<MODE, ROUND, false>), dim3((unsigned)blocks), dim3(256), 0, s,
                           (const uint16_t *)src, (uint32_t *)dst, n, n16);
    return check_launch("feather_pack_fp8");
}

// ---------------------------------------------------------------- fp32 -> packed fp8

// The rounding chain of an fp32 producer that feeds a packed GEMV: fp32 -> fp16 (RNE) -> FP8 code
// (RNE), four codes per word (quant4).  One thread converts four elements from one 128-bit load to one
// word: loads and stores of a wave are contiguous (16 elements per thread from four loads, each a
// 64-byte stride apart across the lanes, ran at a third of the speed).  The last, partial word is padded with +0.
template <int MODE, bool ALIGNED>
__global__ __launch_bounds__(256) void quant_pack_f32_kernel(const float *__restrict__ src, uint32_t *__restrict__ dst,
                                                            int64_t n) {
    const int64_t n_words = (n + 3) / 4, stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < n_words; g += stride) {
        float4_t v;
        if (4 * g + 3 < n) {
            if constexpr (ALIGNED) v = __builtin_nontemporal_load(reinterpret_cast<const float4_t *>(src) + g);
            else v = float4_t{src[4 * g], src[4 * g + 1], src[4 * g + 2], src[4 * g + 3]};
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++) v[i] = 4 * g + i < n ? src[4 * g + i] : 0.f;
        }
        __builtin_nontemporal_store(quant4<MODE>(v[0], v[1], v[2], v[3]), dst + g);
    }
}

template <int MODE>
static int launch_quant_pack(const void *src, void *dst, int64_t n, hipStream_t s) {
    int64_t blocks = ((n + 3) / 4 + 255) / 256;
    if (blocks > 0x7FFFFFFF) blocks = 0x7FFFFFFF;
    if (aligned(src, 16))
        hipLaunchKernelGGL((quant_pack_f32_kernel<MODE, true>), dim3((unsigned)blocks), dim3(256), 0, s, (const float *)src,
                           (uint32_t *)dst, n);
    else
        hipLaunchKernelGGL((quant_pack_f32_kernel<MODE, false>), dim3((unsigned)blocks), dim3(256), 0, s, (const float *)src,
                           (uint32_t *)dst, n);
    return check_launch("feather_quant_pack_f32");
}

// ---------------------------------------------------------------- unpack fp8

template <int MODE, int SEM>
__device__ __forceinline__ void dec_word_sem(uint32_t w, uint32_t &p01, uint32_t &p23) {
    if constexpr (MODE == FEATHER_E4M3 && SEM == FEATHER_SEM_IEEE) {
        p01 = dec_e4m3_ieee_bits(w & 0xFFu) | (dec_e4m3_ieee_bits((w >> 8) & 0xFFu) << 16);
        p23 = dec_e4m3_ieee_bits((w >> 16) & 0xFFu) | (dec_e4m3_ieee_bits(w >> 24) << 16);
    } else {
        dec_word<MODE>(w, p01, p23);
    }
}

// One word per lane per step: 4-byte loads and 16-byte (fp32) or 8-byte (fp16)
// stores are both contiguous across the wave.
template <int MODE, int SEM, int OUT, bool RELU>
__global__ __launch_bounds__(256) void unpack_fp8_kernel(const uint32_t *__restrict__ src, void *__restrict__ dst,
                                                        int64_t n_words) {
    int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t j = t; j < n_words; j += stride) {
        uint32_t w = __builtin_nontemporal_load(src + j);
        half2_t a, b;
        if constexpr (MODE == FEATHER_E4M3 && SEM == FEATHER_SEM_IEEE) {
            // the matrix core's FP8 format is the OCP E4M3fn of the CPU API's decode (subnormals m * 2^-9, 0x7F / 0xFF
            // NaN): the hardware conversion does the whole word in two instructions; every value is exact in fp16
            typedef float float2_t __attribute__((ext_vector_type(2)));
            const float2_t lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, false), hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, true);
            a = half2_t{(_Float16)lo[0], (_Float16)lo[1]};
            b = half2_t{(_Float16)hi[0], (_Float16)hi[1]};
        } else {
            uint32_t p01, p23;
            dec_word_sem<MODE, SEM>(w, p01, p23);
            a = as_half2(p01);
            b = as_half2(p23);
        }
        if constexpr (RELU) {
            // max(0, x) as in tl.maximum(0.0, x): a negative or NaN-free compare
            a.x = a.x > (_Float16)0 ? a.x : (_Float16)0;
            a.y = a.y > (_Float16)0 ? a.y : (_Float16)0;
            b.x = b.x > (_Float16)0 ? b.x : (_Float16)0;
            b.y = b.y > (_Float16)0 ? b.y : (_Float16)0;
        }
        if constexpr (OUT == FEATHER_OUT_F32) {
            store_nt128(reinterpret_cast<u32x4 *>(dst) + j,
                        u32x4{as_u32((float)a.x), as_u32((float)a.y), as_u32((float)b.x), as_u32((float)b.y)});
        } else {
            store_nt64(reinterpret_cast<u32x2 *>(dst) + j, u32x2{as_u32(a), as_u32(b)});
        }
    }
}

template <int MODE, int SEM, int OUT, bool RELU>
static int launch_unpack(const void *src, void *dst, int64_t n_words, hipStream_t s) {
    // four words per thread (grid-stride): 6.0 TB/s on 134 M elements against 5.6 TB/s with a grid capped at 8192
    // workgroups and 5.7 TB/s with one word per thread
    int64_t blocks = (n_words + 1023) / 1024;
    if (blocks > 0x7FFFFFFF) blocks = 0x7FFFFFFF;
    if (blocks < 1) blocks = 1;
    hipLaunchKernelGGL((unpack_fp8_kernel<MODE, SEM, OUT, RELU>), dim3((unsigned)blocks), dim3(256), 0, s,
                       (const uint32_t *)src, dst, n_words);
    return check_launch("feather_unpack_fp8");
}

template <int MODE, int SEM>
static int dispatch_unpack(const void *src, void *dst, int64_t n_words, int out_dtype, int relu, hipStream_t s) {
    if (out_dtype == FEATHER_OUT_F32)
        return relu ? launch_unpack<MODE, SEM, FEATHER_OUT_F32, true>(src, dst, n_words, s)
                    : launch_unpack<MODE, SEM, FEATHER_OUT_F32, false>(src, dst, n_words, s);
    return relu ? launch_unpack<MODE, SEM, FEATHER_OUT_F16, true>(src, dst, n_words, s)
                : launch_unpack<MODE, SEM, FEATHER_OUT_F16, false>(src, dst, n_words, s);
}

// ---------------------------------------------------------------- fp16 container

// word j = src[2j] | src[2j+1] << 16, odd tail padded with +0.  On a
// little-endian device this is a copy with a zeroed last half-word.
__global__ __launch_bounds__(256) void pack_fp16_kernel(const uint16_t *__restrict__ src, uint32_t *__restrict__ dst,
                                                       int64_t n) {
    int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    int64_t nw = (n + 1) / 2;
    for (int64_t j = t; j < nw; j += stride) {
        uint32_t lo = src[2 * j];
        uint32_t hi = 2 * j + 1 < n ? src[2 * j + 1] : 0u;
        dst[j] = lo | (hi << 16);
    }
}

__global__ __launch_bounds__(256) void unpack_fp16_kernel(const uint32_t *__restrict__ src, uint16_t *__restrict__ dst,
                                                         int64_t n_words) {
    int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t j = t; j < n_words; j += stride) {
        uint32_t w = src[j];
        dst[2 * j] = (uint16_t)(w & 0xFFFFu);
        dst[2 * j + 1] = (uint16_t)(w >> 16);
    }
}

// Bulk of the fp16 container when both sides are 16-byte aligned: the container is a plain copy
// on a little-endian device, moved 4 x 128 bits per lane and round with streaming accesses.
__global__ __launch_bounds__(256) void copy128_kernel(const u32x4 *__restrict__ src, u32x4 *__restrict__ dst, int64_t n16) {
    constexpr int U = 4;
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += U * stride) {
        u32x4 v[U];
#pragma unroll
        for (int u = 0; u < U; u++)
            if (i + u * stride < n16) v[u] = load_nt128(src + i + u * stride);
#pragma unroll
        for (int u = 0; u < U; u++)
            if (i + u * stride < n16) store_nt128(dst + i + u * stride, v[u]);
    }
}

// copies the first n16 16-byte units; returns how many it took (0 if the pointers are not aligned)
static int64_t launch_copy128(const void *src, void *dst, int64_t n16, hipStream_t s) {
    if (n16 <= 0 || !aligned(src, 16) || !aligned(dst, 16)) return 0;
    // one 16-byte unit per thread: 6.4 TB/s on 268 MB against 4.7 TB/s with four units per thread on a capped grid
    int64_t blocks = (n16 + 255) / 256;
    if (blocks > 0x7FFFFFFF) blocks = 0x7FFFFFFF;
    hipLaunchKernelGGL(copy128_kernel, dim3((unsigned)blocks), dim3(256), 0, s, (const u32x4 *)src, (u32x4 *)dst, n16);
    return n16;
}

}  // namespace feather

using namespace feather;

extern "C" int feather_version(void) { return FEATHER_HIP_VERSION; }

extern "C" const char *feather_last_error(void) { return g_err; }

extern "C" int feather_pack_fp8(const void *src_f16, void *dst_u32, int64_t n, int mode, int rounding, void *stream) {
    FEATHER_CHECK(n >= 0, FEATHER_EINVAL, "feather_pack_fp8: negative n");
    FEATHER_CHECK(mode == FEATHER_E5M2 || mode == FEATHER_E4M3, FEATHER_EMODE, "feather_pack_fp8: mode %d not supported",
                  mode);
    FEATHER_CHECK(rounding == FEATHER_ROUND_RNE || rounding == FEATHER_ROUND_TRUNC, FEATHER_EINVAL,
                  "feather_pack_fp8: bad rounding %d", rounding);
    FEATHER_CHECK(!(rounding == FEATHER_ROUND_TRUNC && mode != FEATHER_E5M2), FEATHER_EMODE,
                  "feather_pack_fp8: truncating pack supports E5M2 only");
    if (n == 0) return FEATHER_OK;
    FEATHER_CHECK(src_f16 && dst_u32, FEATHER_EINVAL, "feather_pack_fp8: null pointer");
    FEATHER_CHECK(aligned(src_f16, 2) && aligned(dst_u32, 4), FEATHER_EINVAL, "feather_pack_fp8: misaligned pointer");
    hipStream_t s = (hipStream_t)stream;
    if (rounding == FEATHER_ROUND_TRUNC) return launch_pack<FEATHER_E5M2, FEATHER_ROUND_TRUNC>(src_f16, dst_u32, n, s);
    if (mode == FEATHER_E5M2) return launch_pack<FEATHER_E5M2, FEATHER_ROUND_RNE>(src_f16, dst_u32, n, s);
    return launch_pack<FEATHER_E4M3, FEATHER_ROUND_RNE>(src_f16, dst_u32, n, s);
}

extern "C" int feather_quant_pack_f32(const void *src_f32, void *dst_u32, int64_t n, int mode, void *stream) {
    FEATHER_CHECK(n >= 0, FEATHER_EINVAL, "feather_quant_pack_f32: negative n");
    FEATHER_CHECK(mode == FEATHER_E5M2 || mode == FEATHER_E4M3, FEATHER_EMODE,
                  "feather_quant_pack_f32: mode %d not supported", mode);
    if (n == 0) return FEATHER_OK;
    FEATHER_CHECK(src_f32 && dst_u32, FEATHER_EINVAL, "feather_quant_pack_f32: null pointer");
    FEATHER_CHECK(aligned(src_f32, 4) && aligned(dst_u32, 4), FEATHER_EINVAL, "feather_quant_pack_f32: misaligned pointer");
    if (mode == FEATHER_E5M2) return launch_quant_pack<FEATHER_E5M2>(src_f32, dst_u32, n, (hipStream_t)stream);
    return launch_quant_pack<FEATHER_E4M3>(src_f32, dst_u32, n, (hipStream_t)stream);
}

extern "C" int feather_unpack_fp8(const void *src_u32, void *dst, int64_t n_words, int mode, int semantics,
                                  int out_dtype, int relu, void *stream) {
    FEATHER_CHECK(n_words >= 0, FEATHER_EINVAL, "feather_unpack_fp8: negative n_words");
    FEATHER_CHECK(mode == FEATHER_E5M2 || mode == FEATHER_E4M3, FEATHER_EMODE,
                  "feather_unpack_fp8: mode %d not supported", mode);
    FEATHER_CHECK(semantics == FEATHER_SEM_KERNEL || semantics == FEATHER_SEM_IEEE, FEATHER_EINVAL,
                  "feather_unpack_fp8: bad semantics %d", semantics);
    FEATHER_CHECK(out_dtype == FEATHER_OUT_F32 || out_dtype == FEATHER_OUT_F16, FEATHER_EINVAL,
                  "feather_unpack_fp8: bad out_dtype %d", out_dtype);
    if (n_words == 0) return FEATHER_OK;
    FEATHER_CHECK(src_u32 && dst, FEATHER_EINVAL, "feather_unpack_fp8: null pointer");
    FEATHER_CHECK(aligned(src_u32, 4) && aligned(dst, out_dtype == FEATHER_OUT_F32 ? 16 : 8), FEATHER_EINVAL,
                  "feather_unpack_fp8: misaligned pointer");
    hipStream_t s = (hipStream_t)stream;
    if (mode == FEATHER_E5M2) return dispatch_unpack<FEATHER_E5M2, FEATHER_SEM_KERNEL>(src_u32, dst, n_words, out_dtype, relu, s);
    if (semantics == FEATHER_SEM_IEEE)
        return dispatch_unpack<FEATHER_E4M3, FEATHER_SEM_IEEE>(src_u32, dst, n_words, out_dtype, relu, s);
    return dispatch_unpack<FEATHER_E4M3, FEATHER_SEM_KERNEL>(src_u32, dst, n_words, out_dtype, relu, s);
}

extern "C" int feather_pack_fp16(const void *src_f16, void *dst_u32, int64_t n, void *stream) {
    FEATHER_CHECK(n >= 0, FEATHER_EINVAL, "feather_pack_fp16: negative n");
    if (n == 0) return FEATHER_OK;
    FEATHER_CHECK(src_f16 && dst_u32, FEATHER_EINVAL, "feather_pack_fp16: null pointer");
    FEATHER_CHECK(aligned(src_f16, 2) && aligned(dst_u32, 4), FEATHER_EINVAL, "feather_pack_fp16: misaligned pointer");
    const int64_t done = launch_copy128(src_f16, dst_u32, n / 8, (hipStream_t)stream) * 8;   // halfs moved in bulk
    n -= done;
    if (n > 0) {
        int64_t nw = (n + 1) / 2;
        int64_t blocks = (nw + 255) / 256;
        if (blocks > 256 * 32) blocks = 256 * 32;
        hipLaunchKernelGGL(pack_fp16_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                           (const uint16_t *)src_f16 + done, (uint32_t *)dst_u32 + done / 2, n);
    }
    return check_launch("feather_pack_fp16");
}

extern "C" int feather_unpack_fp16(const void *src_u32, void *dst_f16, int64_t n_words, void *stream) {
    FEATHER_CHECK(n_words >= 0, FEATHER_EINVAL, "feather_unpack_fp16: negative n_words");
    if (n_words == 0) return FEATHER_OK;
    FEATHER_CHECK(src_u32 && dst_f16, FEATHER_EINVAL, "feather_unpack_fp16: null pointer");
    FEATHER_CHECK(aligned(src_u32, 4) && aligned(dst_f16, 2), FEATHER_EINVAL, "feather_unpack_fp16: misaligned pointer");
    const int64_t done = launch_copy128(src_u32, dst_f16, n_words / 4, (hipStream_t)stream) * 4;   // words moved in bulk
    n_words -= done;
    if (n_words > 0) {
        int64_t blocks = (n_words + 255) / 256;
        if (blocks > 256 * 32) blocks = 256 * 32;
        hipLaunchKernelGGL(unpack_fp16_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                           (const uint32_t *)src_u32 + done, (uint16_t *)dst_f16 + 2 * done, n_words);
    }
    return check_launch("feather_unpack_fp16");
}
