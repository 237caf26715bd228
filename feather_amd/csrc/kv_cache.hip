// Prefill -> paged KV cache: scatter the K and V rows of packed variable-length
// sequences into the blocks their block tables name.  The source is either
// already packed (the operands of the prefill attention) or fp16, encoded on
// the way (fp16 -> FP8, round to nearest even, as pack_fp8_tensor).  The
// reference has no KV cache; the cache layout is the one the paged-attention
// kernel reads: [n_blocks, n_kv_heads, block_size, d / 4] words.
// One lane moves 16 codes (one 128-bit store); a copy, bound by HBM.
#include "common.h"

namespace feather {

template <int MODE, bool F16>
__global__ __launch_bounds__(256) void paged_cache_write_kernel(
    const void *__restrict__ k_src, const void *__restrict__ v_src, uint32_t *__restrict__ k_cache,
    uint32_t *__restrict__ v_cache, const int32_t *__restrict__ block_tables, const int32_t *__restrict__ cu_seqlens,
    const int32_t *__restrict__ start_pos, int n_seq, int total_rows, int n_kv_heads, int units, int block_size,
    int max_blocks, int n_blocks) {
    const int64_t u = (int64_t)blockIdx.x * 256 + threadIdx.x;      // 16-code unit
    if (u >= (int64_t)n_kv_heads * total_rows * units) return;
    const int c = (int)(u % units);
    const int t = (int)((u / units) % total_rows);
    const int h = (int)(u / ((int64_t)units * total_rows));
    if (t < cu_seqlens[0] || t >= cu_seqlens[n_seq]) return;        // a row outside every sequence
    int lo = 0, hi = n_seq;                                         // largest s with cu[s] <= t
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (cu_seqlens[mid] <= t) lo = mid; else hi = mid;
    }
    const int pos = (start_pos ? start_pos[lo] : 0) + t - cu_seqlens[lo];
    if (pos < 0 || pos >= max_blocks * block_size) return;          // no entry in the block table: dropped
    const int blk = block_tables[(int64_t)lo * max_blocks + pos / block_size];
    if ((unsigned)blk >= (unsigned)n_blocks) return;                // padding or a bad entry: dropped, never written
    const int64_t dst = ((((int64_t)blk * n_kv_heads + h) * block_size + pos % block_size) * units + c) * 4;
    const int64_t src = ((int64_t)h * total_rows + t) * units + c;  // in 16-code units
#pragma unroll
    for (int which = 0; which < 2; which++) {
        const void *sp = which ? v_src : k_src;
        uint32_t *cache = which ? v_cache : k_cache;
        u32x4 w;
        if constexpr (F16) {
            const u32x4 a = reinterpret_cast<const u32x4 *>(sp)[2 * src], b = reinterpret_cast<const u32x4 *>(sp)[2 * src + 1];
            auto enc4 = [](uint32_t p01, uint32_t p23) {            // two words of fp16 pairs -> one packed word
                if constexpr (MODE == FEATHER_E4M3) return perm(enc_e4m3_pair(p23), enc_e4m3_pair(p01), 0x06040200u);
                return enc<MODE, FEATHER_ROUND_RNE>(p01 & 0xFFFFu) | (enc<MODE, FEATHER_ROUND_RNE>(p01 >> 16) << 8) |
                       (enc<MODE, FEATHER_ROUND_RNE>(p23 & 0xFFFFu) << 16) | (enc<MODE, FEATHER_ROUND_RNE>(p23 >> 16) << 24);
            };
            w = u32x4{enc4(a.x, a.y), enc4(a.z, a.w), enc4(b.x, b.y), enc4(b.z, b.w)};
        } else {
            w = reinterpret_cast<const u32x4 *>(sp)[src];
        }
        *reinterpret_cast<u32x4 *>(cache + dst) = w;
    }
}

}  // namespace feather

using namespace feather;

extern "C" int feather_paged_cache_write(const void *k_src, const void *v_src, int src_f16, void *k_cache, void *v_cache,
                                         const void *block_tables, const void *cu_seqlens, const void *start_pos,
                                         int64_t n_seq, int64_t total_rows, int64_t n_kv_heads, int64_t d,
                                         int64_t block_size, int64_t max_blocks, int64_t n_blocks, int mode,
                                         void *stream) {
    const char *me = "feather_paged_cache_write";
    FEATHER_CHECK(mode == FEATHER_E5M2 || mode == FEATHER_E4M3, FEATHER_EMODE, "%s: mode %d not supported", me, mode);
    FEATHER_CHECK(src_f16 == 0 || src_f16 == 1, FEATHER_EINVAL, "%s: src_f16 must be 0 or 1", me);
    FEATHER_CHECK(n_seq >= 0 && total_rows >= 0 && n_kv_heads >= 0 && block_size > 0 && max_blocks >= 0 && n_blocks >= 0,
                  FEATHER_EINVAL, "%s: bad shape", me);
    FEATHER_CHECK(n_blocks < (1ll << 31), FEATHER_ESHAPE, "%s: n_blocks too large", me);
    FEATHER_CHECK(d > 0 && d % 16 == 0, FEATHER_ESHAPE, "%s: head dim %lld is not a multiple of 16", me, (long long)d);
    FEATHER_CHECK(total_rows < (1ll << 31) && max_blocks * block_size < (1ll << 31), FEATHER_ESHAPE, "%s: shape too large", me);
    if (n_seq == 0 || total_rows == 0 || n_kv_heads == 0) return FEATHER_OK;
    FEATHER_CHECK(k_src && v_src && k_cache && v_cache && block_tables && cu_seqlens, FEATHER_EINVAL, "%s: null pointer", me);
    FEATHER_CHECK(aligned(k_src, 16) && aligned(v_src, 16) && aligned(k_cache, 16) && aligned(v_cache, 16) &&
                      aligned(block_tables, 4) && aligned(cu_seqlens, 4) && aligned(start_pos, 4),
                  FEATHER_EINVAL, "%s: misaligned pointer", me);
    const int64_t units = n_kv_heads * total_rows * (d / 16);
    FEATHER_CHECK((units + 255) / 256 < (1ll << 31), FEATHER_ESHAPE, "%s: grid too large", me);
#define FEATHER_CW(MM, FF)                                                                                            \
    hipLaunchKernelGGL((paged_cache_write_kernel<MM, FF>), dim3((unsigned)((units + 255) / 256)), dim3(256), 0,       \
                       (hipStream_t)stream, k_src, v_src, (uint32_t *)k_cache, (uint32_t *)v_cache,                   \
                       (const int32_t *)block_tables, (const int32_t *)cu_seqlens, (const int32_t *)start_pos,        \
                       (int)n_seq, (int)total_rows, (int)n_kv_heads, (int)(d / 16), (int)block_size, (int)max_blocks,    \
                       (int)n_blocks)
    if (mode == FEATHER_E5M2) { if (src_f16) FEATHER_CW(FEATHER_E5M2, true); else FEATHER_CW(FEATHER_E5M2, false); }
    else { if (src_f16) FEATHER_CW(FEATHER_E4M3, true); else FEATHER_CW(FEATHER_E4M3, false); }
#undef FEATHER_CW
    return check_launch(me);
}
