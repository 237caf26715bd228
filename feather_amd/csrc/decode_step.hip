// One decode step of a Llama-shaped model whose linear layers are FP8-packed
// GEMVs and whose KV cache is a paged FP8 cache.  The reference has no model
// code; this driver strings the routines of this library together for a whole
// batch with one host call: per layer
//     (h += delta) -> RMSNorm -> pack            add_rmsnorm_pack_kernel
//     qkv = W_qkv x                              feather_gemv_fp8_batched
//     RoPE(q, k), pack q, append k/v to cache    rope_append_kernel
//     paged attention                            feather_paged_attn_fp8
//     o = W_o attn (attention emits packed FP8)  batched GEMV
//     (h += o) -> RMSNorm -> pack                add_rmsnorm_pack_kernel
//     act = pack(silu(W_gate x) * (W_up x))      batched GEMV with the SwiGLU epilogue
//                                                (or GEMV + swiglu_pack_kernel for odd shapes)
//     down = W_down act                          batched GEMV (added to h by the next norm)
// and a final norm + lm_head GEMV.  Every activation that feeds a GEMV is
// rounded fp32 -> fp16 -> FP8 (RNE, as pack_fp8_tensor does) and packed four
// codes per word in the producing kernel, so no separate quantisation pass
// touches memory.  All launches go to one stream; nothing allocates or syncs.
#include "internal.h"
#include "common.h"

namespace feather {

constexpr int kDsThreads = 256;

template <int THREADS = kDsThreads>
__device__ __forceinline__ float block_sum(float x, float *red) {
    x = wave_sum(x);
    const int lane = lane_id(), wave = wave_id();
    if (lane == 0) red[wave] = x;
    __syncthreads();
    float t = 0.f;
#pragma unroll
    for (int w = 0; w < THREADS / kWave; w++) t += red[w];
    __syncthreads();
    return t;
}

// h[b, :] = embed[token[b], :] (fp16 table -> fp32 residual stream)
__global__ __launch_bounds__(kDsThreads) void embed_kernel(const _Float16 *__restrict__ embed,
                                                          const int32_t *__restrict__ tokens,
                                                          float *__restrict__ h, int hidden) {
    const int b = blockIdx.x;
    const _Float16 *row = embed + (int64_t)tokens[b] * hidden;
    for (int i = threadIdx.x; i < hidden; i += kDsThreads) h[(int64_t)b * hidden + i] = (float)row[i];
}

// A GEMV result may arrive as n_part partial sums (slices of K), part_stride floats apart; they
// are added in slice order.
__device__ __forceinline__ float4 load_parts(const float *p, int n_part, int64_t part_stride) {
    constexpr int G = 8;                       // loads in flight: clamped address, unused ones dropped below
    float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int s = 0; s < n_part; s += G) {
        float4 b[G];
#pragma unroll
        for (int u = 0; u < G; u++)
            b[u] = *reinterpret_cast<const float4 *>(p + (int64_t)min(s + u, n_part - 1) * part_stride);
        if (s == 0) a = b[0];
#pragma unroll
        for (int u = 0; u < G; u++) {
            if (s + u > 0 && s + u < n_part) { a.x += b[u].x; a.y += b[u].y; a.z += b[u].z; a.w += b[u].w; }
        }
    }
    return a;
}

// h += delta (if given); xq = pack(fp16(h * rsqrt(mean(h^2) + eps) * w)).  One workgroup per row.
// The kernel is a chain of memory round trips and little else, so every load of a row's first
// 4096 elements (h, the norm weights and up to eight partial sums per element) is issued before
// the first value is used, and the second pass works from registers: two round trips (loads,
// stores) instead of one per 1024 elements and pass.
template <int MODE, int KEEP, int THREADS>
__global__ __launch_bounds__(THREADS) void add_rmsnorm_pack_kernel(float *__restrict__ h,
                                                                     const float *__restrict__ delta, int n_part,
                                                                     int64_t part_stride,
                                                                     const float *__restrict__ w,
                                                                     uint32_t *__restrict__ xq, int hidden,
                                                                     float eps, float *__restrict__ y_f32) {
    __shared__ float red[THREADS / kWave];
    const int b = blockIdx.x;
    float4 *hr = reinterpret_cast<float4 *>(h + (int64_t)b * hidden);
    const float *dr = delta ? delta + (int64_t)b * hidden : nullptr;
    const float4 *wr = reinterpret_cast<const float4 *>(w);
    const int n4 = hidden / 4;
    constexpr int kKeep = KEEP, G = 8;
    float4 x[kKeep], g[kKeep], part[kKeep][G];
    // ---- all loads (inactive slots read element 0 and are dropped)
#pragma unroll
    for (int it = 0; it < kKeep; it++) {
        const int i = threadIdx.x + it * THREADS, ii = i < n4 ? i : 0;
        x[it] = hr[ii];
        g[it] = wr[ii];
        if (dr) {
#pragma unroll
            for (int u = 0; u < G; u++)
                part[it][u] = *reinterpret_cast<const float4 *>(dr + 4 * ii + (int64_t)min(u, n_part - 1) * part_stride);
        }
    }
    float ss = 0.f;
#pragma unroll
    for (int it = 0; it < kKeep; it++) {
        const int i = threadIdx.x + it * THREADS;
        if (i < n4) {
            if (dr) {
                float4 d = part[it][0];                      // slices are added in index order
#pragma unroll
                for (int u = 1; u < G; u++)
                    if (u < n_part) { d.x += part[it][u].x; d.y += part[it][u].y; d.z += part[it][u].z; d.w += part[it][u].w; }
                for (int s0 = G; s0 < n_part; s0 += G) {     // more than G slices: further rounds
                    float4 q[G];
#pragma unroll
                    for (int u = 0; u < G; u++)
                        q[u] = *reinterpret_cast<const float4 *>(dr + 4 * i + (int64_t)min(s0 + u, n_part - 1) * part_stride);
#pragma unroll
                    for (int u = 0; u < G; u++)
                        if (s0 + u < n_part) { d.x += q[u].x; d.y += q[u].y; d.z += q[u].z; d.w += q[u].w; }
                }
                x[it].x += d.x; x[it].y += d.y; x[it].z += d.z; x[it].w += d.w;
                hr[i] = x[it];
            }
            ss += (x[it].x * x[it].x + x[it].y * x[it].y) + (x[it].z * x[it].z + x[it].w * x[it].w);
        }
    }
    for (int i = threadIdx.x + kKeep * THREADS; i < n4; i += THREADS) {   // rows longer than 4096
        float4 y = hr[i];
        if (dr) {
            float4 d = load_parts(dr + 4 * i, n_part, part_stride);
            y.x += d.x; y.y += d.y; y.z += d.z; y.w += d.w;
            hr[i] = y;
        }
        ss += (y.x * y.x + y.y * y.y) + (y.z * y.z + y.w * y.w);
    }
    const float r = 1.0f / sqrtf(block_sum<THREADS>(ss, red) / (float)hidden + eps);
#pragma unroll
    for (int it = 0; it < kKeep; it++) {
        const int i = threadIdx.x + it * THREADS;
        if (i < n4) {
            const float4 y = make_float4(x[it].x * r * g[it].x, x[it].y * r * g[it].y, x[it].z * r * g[it].z, x[it].w * r * g[it].w);
            xq[(int64_t)b * n4 + i] = quant4<MODE>(y.x, y.y, y.z, y.w);
            if (y_f32) reinterpret_cast<float4 *>(y_f32)[(int64_t)b * n4 + i] = y;   // the values the codes were rounded from
        }
    }
    for (int i = threadIdx.x + kKeep * THREADS; i < n4; i += THREADS) {
        float4 y = hr[i], gg = wr[i];
        y = make_float4(y.x * r * gg.x, y.y * r * gg.y, y.z * r * gg.z, y.w * r * gg.w);
        xq[(int64_t)b * n4 + i] = quant4<MODE>(y.x, y.y, y.z, y.w);
        if (y_f32) reinterpret_cast<float4 *>(y_f32)[(int64_t)b * n4 + i] = y;
    }
}

// gu [B, 2 * inter] (gate rows then up rows) -> pack(fp16(silu(gate) * up)) [B, inter / 4]
// One workgroup per vector; the row is spread over as many threads as it has groups of four elements (up to
// 512), so a thread issues the loads of one group -- residual, gain, eight partial sums -- instead of
// several: the kernel is one memory round trip plus a block reduction, and its length is the time the
// workgroup's loads take to drain through one CU (TinyLlama width, 256 threads with two groups each
// and two idle slots: 2.1 us from entry to the sums; see the launcher of the decode step).
template <int MODE>
static void launch_norm(int batch, hipStream_t s, float *h, const float *delta, int n_part, int64_t part_stride,
                        const void *w, uint32_t *xq, int hidden, float eps, float *y_f32 = nullptr) {
    const int n4 = hidden / 4;
    auto go = [&](auto kern, int threads) {
        hipLaunchKernelGGL(kern, dim3(batch), dim3(threads), 0, s, h, delta, n_part, part_stride, (const float *)w, xq,
                           hidden, eps, y_f32);
    };
    if (n4 <= 256) go(add_rmsnorm_pack_kernel<MODE, 1, 256>, 256);
    else if (n4 <= 512) go(add_rmsnorm_pack_kernel<MODE, 1, 512>, 512);
    else if (n4 <= 1024) go(add_rmsnorm_pack_kernel<MODE, 2, 512>, 512);
    else go(add_rmsnorm_pack_kernel<MODE, 4, 512>, 512);
}

template <int MODE>
__global__ __launch_bounds__(kDsThreads) void swiglu_pack_kernel(const float *__restrict__ gu, int n_part,
                                                                int64_t part_stride,
                                                                uint32_t *__restrict__ out, int inter, int batch) {
    const int per_row = inter / 4;
    for (int64_t i = (int64_t)blockIdx.x * kDsThreads + threadIdx.x; i < (int64_t)batch * per_row;
         i += (int64_t)gridDim.x * kDsThreads) {
        int b = (int)(i / per_row), c = (int)(i % per_row);
        float4 g = load_parts(gu + (int64_t)b * 2 * inter + 4 * c, n_part, part_stride);
        float4 u = load_parts(gu + (int64_t)b * 2 * inter + inter + 4 * c, n_part, part_stride);
        // the same arithmetic as the fused epilogue of the gate/up GEMV
        auto f = [](float a, float bb) {
            return a * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * a)) * bb;
        };
        out[i] = quant4<MODE>(f(g.x, u.x), f(g.y, u.y), f(g.z, u.z), f(g.w, u.w));
    }
}

// qkv [B, (n_q + 2 n_kv) * d] fp32 -> RoPE on q and k (rotate-half convention: element j pairs
// with j + d/2, angle pos * theta^(-2j/d)), q packed to qp [B, n_q, d/4], k and v encoded and
// written into the paged cache at position pos = ctx_lens[b]; ctx_after[b] = pos + 1.
// A position outside [0, max_blocks * block_size) or a block id outside [0, n_blocks) is never
// written: the token is dropped, ctx_after[b] is the old length (clamped into the table) and
// status[b] says why (1: no room / bad position, 2: bad block id; 0: appended).  pos_limit is the number of
// positions the caller's context bound allows (at most the table's max_blocks * block_size).
constexpr int kRopeThreads = 64;
// sin and cos of a non-negative angle below ~1e5 rad to ~1e-7 absolute: three-constant Cody-Waite reduction
// by pi/2 with fused multiply-adds, then the single-precision minimax polynomials on [-pi/4, pi/4].  The
// library's sincosf (full range reduction) was the longest phase of the RoPE kernel: 1.3 of its 2.2 us.
__device__ __forceinline__ void sincos_small(float x, float &s, float &c) {
    const float k = rintf(x * 0.636619772f);
    float r = fmaf(k, -1.57079625e+00f, x);
    r = fmaf(k, -7.54978942e-08f, r);
    r = fmaf(k, -5.39030295e-15f, r);
    const float r2 = r * r;
    const float sp = fmaf(r * r2, fmaf(r2, fmaf(r2, -1.9515295891e-4f, 8.3321608736e-3f), -1.6666654611e-1f), r);
    const float cp = fmaf(r2, fmaf(r2, fmaf(r2, fmaf(r2, 2.443315711809948e-5f, -1.388731625493765e-3f), 4.166664568298827e-2f), -0.5f), 1.0f);
    const int q = (int)k;
    const float ss = (q & 1) ? cp : sp, cc = (q & 1) ? sp : cp;
    s = (q & 2) ? -ss : ss;
    c = ((q + 1) & 2) ? -cc : cc;
}

// (parameter order: everything needed before the first loads sits in the 16 preloaded dwords)
template <int MODE>
__global__ __launch_bounds__(kRopeThreads) void rope_append_kernel(const float *__restrict__ qkv,
                                                                const int32_t *__restrict__ ctx_lens,
                                                                const int32_t *__restrict__ block_tables,
                                                                int64_t part_stride, int n_part, int n_q, int n_kv,
                                                                int d, int block_size, int max_blocks,
                                                                float log2_theta, uint32_t *__restrict__ qp,
                                                                uint32_t *__restrict__ k_cache,
                                                                uint32_t *__restrict__ v_cache,
                                                                int32_t *__restrict__ ctx_after, int n_blocks,
                                                                int32_t *__restrict__ status,
                                                                float *__restrict__ rot_f32, int pos_limit) {
    const int b = blockIdx.x;
    const int dw = d / 4, half_w = d / 8;            // words per head, words per rotation half
    const int heads = n_q + 2 * n_kv;
    const int item = blockIdx.y * kRopeThreads + threadIdx.x;
    const bool live = item < heads * half_w;
    const int head = live ? item / half_w : 0, t = live ? item % half_w : 0;
    // Two chains of loads: position -> block id, and the GEMV partials of the two elements this
    // thread rotates.  The position goes out first, then every partial (up to 8 slices per element),
    // then the block id as soon as the position is back: the chains overlap instead of queueing.
    const int pos_raw = ctx_lens[b];
    const float *x = qkv + ((int64_t)b * heads + head) * d;
    constexpr int G = 8;
    float4 pl[G], ph[G];
#pragma unroll
    for (int u = 0; u < G; u++) {
        const int64_t off = (int64_t)min(u, n_part - 1) * part_stride;
        pl[u] = *reinterpret_cast<const float4 *>(x + 4 * t + off);            // elements 4t .. 4t+3
        ph[u] = *reinterpret_cast<const float4 *>(x + d / 2 + 4 * t + off);    // their partners
    }
    const int cap = pos_limit;                       // at most max_blocks * block_size
    const bool pos_ok = pos_raw >= 0 && pos_raw < cap;
    const int pos = pos_ok ? pos_raw : 0;            // in range for the table lookup; nothing is written if !pos_ok
    const int blk = block_tables[(int64_t)b * max_blocks + pos / block_size];
    const bool blk_ok = (unsigned)blk < (unsigned)n_blocks;
    const bool append = pos_ok && blk_ok;
    if (threadIdx.x == 0 && blockIdx.y == 0) {
        ctx_after[b] = append ? pos + 1 : min(max(pos_raw, 0), cap);
        if (status) status[b] = pos_ok ? (blk_ok ? 0 : 2) : 1;
    }
    const int64_t slot = ((int64_t)(blk_ok ? blk : 0) * n_kv) * block_size;
    float4 lo = pl[0], hi = ph[0];                   // slices are added in index order
#pragma unroll
    for (int u = 1; u < G; u++)
        if (u < n_part) {
            lo.x += pl[u].x; lo.y += pl[u].y; lo.z += pl[u].z; lo.w += pl[u].w;
            hi.x += ph[u].x; hi.y += ph[u].y; hi.z += ph[u].z; hi.w += ph[u].w;
        }
    for (int s0 = G; s0 < n_part; s0 += G) {          // more than G slices: further rounds
#pragma unroll
        for (int u = 0; u < G; u++) {
            const int64_t off = (int64_t)min(s0 + u, n_part - 1) * part_stride;
            pl[u] = *reinterpret_cast<const float4 *>(x + 4 * t + off);
            ph[u] = *reinterpret_cast<const float4 *>(x + d / 2 + 4 * t + off);
        }
#pragma unroll
        for (int u = 0; u < G; u++)
            if (s0 + u < n_part) {
                lo.x += pl[u].x; lo.y += pl[u].y; lo.z += pl[u].z; lo.w += pl[u].w;
                hi.x += ph[u].x; hi.y += ph[u].y; hi.z += ph[u].z; hi.w += ph[u].w;
            }
    }
    if (!live) return;
    {
        if (head < n_q + n_kv) {
            float lo4[4] = {lo.x, lo.y, lo.z, lo.w}, hi4[4] = {hi.x, hi.y, hi.z, hi.w};
#pragma unroll
            for (int i = 0; i < 4; i++) {
                float inv_freq = exp2f(-(2.0f * (float)(4 * t + i) / (float)d) * log2_theta);
                float s, c;
                sincos_small((float)pos * inv_freq, s, c);
                float a = lo4[i], bb = hi4[i];
                lo4[i] = a * c - bb * s;
                hi4[i] = bb * c + a * s;
            }
            lo = make_float4(lo4[0], lo4[1], lo4[2], lo4[3]);
            hi = make_float4(hi4[0], hi4[1], hi4[2], hi4[3]);
        }
        const uint32_t wlo = quant4<MODE>(lo.x, lo.y, lo.z, lo.w), whi = quant4<MODE>(hi.x, hi.y, hi.z, hi.w);
        if (rot_f32) {                               // the values the codes were rounded from
            float *r = rot_f32 + ((int64_t)b * heads + head) * d;
            *reinterpret_cast<float4 *>(r + 4 * t) = lo;
            *reinterpret_cast<float4 *>(r + d / 2 + 4 * t) = hi;
        }
        uint32_t *dst;
        if (head < n_q) {
            dst = qp + ((int64_t)b * n_q + head) * dw;
        } else {
            if (!append) return;
            const int kvh = head < n_q + n_kv ? head - n_q : head - n_q - n_kv;
            uint32_t *cache = head < n_q + n_kv ? k_cache : v_cache;
            dst = cache + ((slot + (int64_t)kvh * block_size) + pos % block_size) * dw;
        }
        dst[t] = wlo;
        dst[t + half_w] = whi;
    }
}

// First kernel of a step when the attention runs with the fused prologue (paged_attn_split_kernel, FUSED):
// everything that depends only on the step's inputs and is the same for all layers, computed once.
//   blocks [0, batch)          embedding row of the sequence; the cos / sin pairs of its position (the table the
//                              rotary embedding of every layer reads); ctx_after and status of the sequence
//   blocks [batch, batch + n)  one entry of the attention work plan each: the (sequence, split) items in the order
//                              the attention workgroups take them -- all full 512-token splits in sequence order, then
//                              the partial last splits by size, largest first -- with the block ids of the split, so
//                              that an attention workgroup needs one memory round trip to know its work and its blocks
// A sequence's new token is appended iff its position ctx_lens[b] lies in [0, max_ctx) and the table entry of that
// position is a block of the cache; otherwise the sequence attends over the tokens it has and status says why.
constexpr int kPlanSplit = 512;                  // tokens per attention split (paged_attention.hip: kSplit)
__global__ __launch_bounds__(kDsThreads) void step_prologue_kernel(
    const _Float16 *__restrict__ embed, const int32_t *__restrict__ tokens, float *__restrict__ h, int hidden,
    const int32_t *__restrict__ ctx_lens, const int32_t *__restrict__ block_tables, int batch, int d, int block_size,
    int max_blocks, int n_blocks, int max_ctx, int n_splits, float log2_theta, float *__restrict__ cs,
    int32_t *__restrict__ plan, int32_t *__restrict__ ctx_after, int32_t *__restrict__ status) {
    // tokens the sequence holds after the step, whether the new one is appended, and why not
    auto seq_state = [&](int b, int &total, bool &append, int &why) {
        const int pos_raw = ctx_lens[b];
        const bool pos_ok = pos_raw >= 0 && pos_raw < max_ctx;
        const int blk = block_tables[(int64_t)b * max_blocks + (pos_ok ? pos_raw / block_size : 0)];
        const bool blk_ok = (unsigned)blk < (unsigned)n_blocks;
        append = pos_ok && blk_ok;
        total = append ? pos_raw + 1 : min(max(pos_raw, 0), max_ctx);
        why = pos_ok ? (blk_ok ? 0 : 2) : 1;
    };
    if ((int)blockIdx.x < batch) {
        const int b = blockIdx.x;
        int total, why;
        bool append;
        seq_state(b, total, append, why);
        const _Float16 *row = embed + (int64_t)tokens[b] * hidden;
        for (int i = threadIdx.x; i < hidden; i += kDsThreads) h[(int64_t)b * hidden + i] = (float)row[i];
        const int pos = append || why == 2 ? ctx_lens[b] : 0;          // a valid position even if the block id is not
        for (int jj = threadIdx.x; jj < d / 2; jj += kDsThreads) {
            const float inv_freq = exp2f(-(2.0f * (float)jj / (float)d) * log2_theta);   // as rope_append_kernel
            float sn, c;
            sincos_small((float)pos * inv_freq, sn, c);
            cs[((int64_t)b * (d / 2) + jj) * 2] = c;
            cs[((int64_t)b * (d / 2) + jj) * 2 + 1] = sn;
        }
        if (threadIdx.x == 0) {
            ctx_after[b] = total;
            if (status) status[b] = why;
        }
        return;
    }
    const int item = blockIdx.x - batch, lane = threadIdx.x & 63;
    const int ids_per = kPlanSplit / block_size;
    int32_t *entry = plan + (int64_t)item * (4 + ids_per);
    int total = 0, why = 0;
    bool append = false;
    if (lane < batch) seq_state(lane, total, append, why);
    int seq = -1, split = 0;
    if (n_splits == 1) {
        if (item < batch) seq = item;
    } else {
        const int nf = total / kPlanSplit, ps = total % kPlanSplit;   // full splits, tokens of the partial one
        int inc = nf;                                                 // inclusive prefix sum over the lanes
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
            int rank = 0;                                             // partial splits larger than this lane's (ties: lower sequence first)
            for (int t = 0; t < batch; t++) {
                const int pt = __builtin_amdgcn_readlane(ps, t);
                rank += (pt > ps || (pt == ps && t < lane)) ? 1 : 0;
            }
            hit = __builtin_amdgcn_ballot_w64(ps > 0 && rank == item - n_full);
            if (hit) split = __builtin_amdgcn_readlane(nf, __builtin_ctzll(hit));
        }
        if (hit) seq = __builtin_ctzll(hit);
    }
    if (seq < 0) {
        if (threadIdx.x == 0) entry[0] = -1;
        return;
    }
    const int seq_total = __builtin_amdgcn_readlane(total, seq);
    const bool seq_append = __builtin_amdgcn_readlane((int)append, seq) != 0;
    if (threadIdx.x == 0) {
        entry[0] = seq;
        entry[1] = split;
        entry[2] = seq_total;
        entry[3] = seq_append && split == (seq_total - 1) / kPlanSplit ? 1 : 0;   // the new token sits at seq_total - 1
    }
    for (int i = threadIdx.x; i < ids_per; i += kDsThreads) {
        const int bi = split * ids_per + i;
        entry[4 + i] = bi < max_blocks ? block_tables[(int64_t)seq * max_blocks + bi] : 0;
    }
}

// Per-sequence status of a step whose layers do not write it (the generic path writes it from the first layer's
// rotary kernel; a model without layers has none): the same rule as rope_append_kernel.
__global__ void seq_status_kernel(const int32_t *__restrict__ ctx_lens, const int32_t *__restrict__ block_tables, int batch,
                                  int block_size, int max_blocks, int n_blocks, int pos_limit, int32_t *__restrict__ status) {
    const int b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= batch) return;
    const int pos_raw = ctx_lens[b];
    const bool pos_ok = pos_raw >= 0 && pos_raw < pos_limit;
    const int blk = block_tables[(int64_t)b * max_blocks + (pos_ok ? pos_raw : 0) / block_size];
    status[b] = pos_ok ? ((unsigned)blk < (unsigned)n_blocks ? 0 : 2) : 1;
}

// K slices per GEMV: enough 64-row tiles x slices to cover the 256 CUs, at most one slice per
// 256-column chunk (the launcher's own clamp, repeated here to size the partial buffers)
static int plan_splits(int64_t M, int64_t K) {
    if (K % 256 != 0 || K == 0) return 1;          // the per-vector fallback writes complete sums
    const int64_t tiles = (M + 63) / 64, n_chunks = K / 256;
    int64_t s = (256 + tiles - 1) / tiles;       // measured: 128 or 512 workgroups per GEMV are both slower
    s = s < 1 ? 1 : (s > 16 ? 16 : s);
    s = s > n_chunks ? n_chunks : s;
    const int64_t cps = (n_chunks + s - 1) / s;
    return (int)((n_chunks + cps - 1) / cps);
}

struct StepPlan {
    int s_qkv, s_o, s_gu, s_down;
    int64_t qkv_rows;
    bool fused_mlp;                              // gate/up GEMV with the SwiGLU epilogue (no fp32 gate/up buffer)
    size_t b_h, b_delta, b_xq, b_act, b_qkv, b_qp, b_gu, b_ctx, b_plan, b_cs;
    bool fused_attn;                             // rotary embedding / query packing / K-V append inside the attention kernel
};

static StepPlan plan_step(const feather_decoder_t *dec, int64_t batch, int64_t max_ctx) {
    const int64_t H = dec->hidden, nq = dec->n_q_heads, nkv = dec->n_kv_heads, d = dec->head_dim, I = dec->inter;
    StepPlan P;
    P.qkv_rows = (nq + 2 * nkv) * d;
    P.s_qkv = plan_splits(P.qkv_rows, H);
    P.s_o = plan_splits(H, nq * d);
    P.fused_mlp = H % 256 == 0 && I % 4 == 0;
    P.s_gu = P.fused_mlp ? 1 : plan_splits(2 * I, H);
    P.s_down = plan_splits(H, I);
    auto up = [](int64_t b) { return (size_t)((b + 255) / 256 * 256); };
    P.b_h = up(batch * H * 4);
    P.b_delta = up((int64_t)(P.s_o > P.s_down ? P.s_o : P.s_down) * batch * H * 4);
    P.b_xq = up(batch * (H > I ? H : I));
    P.b_act = up(batch * I);
    P.b_qkv = up((int64_t)P.s_qkv * batch * P.qkv_rows * 4);
    P.b_qp = up(batch * nq * d);
    P.b_gu = P.fused_mlp ? 0 : up((int64_t)P.s_gu * batch * 2 * I * 4);
    P.b_ctx = up(batch * 4);
    P.fused_attn = paged_attn_fused_supported(batch, nq, nkv, d, dec->block_size, P.s_qkv);
    P.b_plan = P.fused_attn ? up(paged_attn_plan_ints(batch, dec->block_size, max_ctx) * 4) : 0;
    P.b_cs = P.fused_attn ? up(batch * (d / 2) * 8) : 0;
    return P;
}

template <int MODE>
static int run_step(const feather_decoder_t *dec, const int32_t *tokens, const int32_t *block_tables,
                    const int32_t *ctx_lens, int batch, int max_ctx, void *scratch, float *logits, int32_t *status,
                    hipStream_t s) {
    const int H = dec->hidden, nq = dec->n_q_heads, nkv = dec->n_kv_heads, d = dec->head_dim, I = dec->inter;
    const StepPlan P = plan_step(dec, batch, max_ctx);
    const int qkv_rows = (int)P.qkv_rows;
    // scratch carve-up (all offsets multiples of 256 bytes)
    char *p = (char *)scratch;
    auto take = [&](size_t bytes) { char *q = p; p += bytes; return q; };
    float *h = (float *)take(P.b_h);
    float *delta = (float *)take(P.b_delta);
    uint32_t *xq = (uint32_t *)take(P.b_xq);
    uint32_t *act = (uint32_t *)take(P.b_act);
    float *qkv = (float *)take(P.b_qkv);
    uint32_t *qp = (uint32_t *)take(P.b_qp);
    float *gu = (float *)take(P.b_gu);
    int32_t *ctx_after = (int32_t *)take(P.b_ctx);
    int32_t *plan = (int32_t *)take(P.b_plan);
    float *cs = (float *)take(P.b_cs);
    void *pa_scratch = p;
    const float scale = 1.0f / sqrtf((float)d);
    const float log2_theta = log2f(dec->rope_theta);
    void *st = (void *)s;
    int rc;
    // out receives `splits` partial results of [batch, M], batch * M floats apart
    auto gemv_x = [&](const void *w, const uint32_t *x, float *out, int M, int K, int splits) {
        if (K % 256 != 0) return feather_gemv_fp8_batched(w, x, out, M, K, batch, MODE, st);
        int got = 0;
        int r = gemv_batched_launch(w, x, out, M, K, batch, MODE, splits, (int64_t)batch * M, &got, s);
        if (r == FEATHER_OK && got != splits) {
            set_error("feather_decode_step: GEMV slice plan mismatch (%d vs %d)", got, splits);
            return (int)FEATHER_EINVAL;
        }
        return r;
    };
    auto gemv = [&](const void *w, float *out, int M, int K, int splits) { return gemv_x(w, xq, out, M, K, splits); };
#define DS_CHECK(call)            \
    do {                          \
        rc = (call);              \
        if (rc != FEATHER_OK) return rc; \
    } while (0)

    if (P.fused_attn) {
        const int n_splits = max((max_ctx + kPlanSplit - 1) / kPlanSplit, 1);
        hipLaunchKernelGGL(step_prologue_kernel, dim3(batch + batch * n_splits), dim3(kDsThreads), 0, s,
                           (const _Float16 *)dec->embed_f16, tokens, h, H, ctx_lens, block_tables, batch, d, dec->block_size,
                           dec->max_blocks, dec->n_blocks, max_ctx, n_splits, log2_theta, cs, plan, ctx_after, status);
    } else {
        hipLaunchKernelGGL(embed_kernel, dim3(batch), dim3(kDsThreads), 0, s, (const _Float16 *)dec->embed_f16, tokens, h, H);
        if (dec->n_layers == 0 && status)     // no rotary kernel will write it
            hipLaunchKernelGGL(seq_status_kernel, dim3(1), dim3(64), 0, s, ctx_lens, block_tables, batch, dec->block_size,
                               dec->max_blocks, dec->n_blocks, max_ctx, status);
    }
    DS_CHECK(check_launch("feather_decode_step (embed)"));
    const float *pending = nullptr;                       // output of the previous down projection, not yet added
    const int64_t hs = (int64_t)batch * H;
    for (int l = 0; l < dec->n_layers; l++) {
        const feather_decoder_layer_t &L = dec->layers[l];
        launch_norm<MODE>(batch, s, h, pending, P.s_down, hs, L.norm_attn, xq, H, dec->rms_eps);
        DS_CHECK(check_launch("feather_decode_step (norm)"));
        DS_CHECK(gemv(L.w_qkv, qkv, qkv_rows, H, P.s_qkv));
        if (P.fused_attn) {
            // rotary embedding, query packing and the append of the new K / V rows happen in the attention
            // kernel's prologue; it writes its output already rounded to FP8 and packed (the operand of W_o)
            DS_CHECK(paged_attn_fused_launch(plan, ctx_after, L.k_cache, L.v_cache, qkv, P.s_qkv, (int64_t)batch * qkv_rows, cs,
                                             xq, pa_scratch, batch, nq, nkv, dec->block_size, dec->max_blocks, dec->n_blocks,
                                             max_ctx, MODE, scale, s));
        } else {
            hipLaunchKernelGGL((rope_append_kernel<MODE>),
                               dim3(batch, ((nq + 2 * nkv) * (d / 8) + kRopeThreads - 1) / kRopeThreads), dim3(kRopeThreads), 0, s, qkv, ctx_lens,
                               block_tables, (int64_t)batch * qkv_rows, P.s_qkv, nq, nkv, d, dec->block_size, dec->max_blocks,
                               log2_theta, qp, (uint32_t *)L.k_cache, (uint32_t *)L.v_cache, ctx_after, dec->n_blocks,
                               l == 0 ? status : nullptr, (float *)nullptr, max_ctx);
            DS_CHECK(check_launch("feather_decode_step (rope)"));
            // attention writes its output already rounded to FP8 and packed (the operand of W_o)
            DS_CHECK(paged_attn_launch(qp, L.k_cache, L.v_cache, block_tables, ctx_after, nullptr, xq, nullptr, pa_scratch, batch, nq,
                                       nkv, d, dec->block_size, dec->max_blocks, dec->n_blocks, max_ctx, MODE, scale, s));
        }
        DS_CHECK(gemv(L.w_o, delta, H, nq * d, P.s_o));
        launch_norm<MODE>(batch, s, h, delta, P.s_o, hs, L.norm_mlp, xq, H, dec->rms_eps);
        DS_CHECK(check_launch("feather_decode_step (norm)"));
        if (P.fused_mlp) {
            DS_CHECK(gemv_batched_swiglu_launch(L.w_gate_up, xq, act, nullptr, I, H, batch, MODE, s));
        } else {
            DS_CHECK(gemv(L.w_gate_up, gu, 2 * I, H, P.s_gu));
            int64_t items = (int64_t)batch * I / 4;
            hipLaunchKernelGGL((swiglu_pack_kernel<MODE>), dim3((unsigned)((items + kDsThreads - 1) / kDsThreads)),
                               dim3(kDsThreads), 0, s, gu, P.s_gu, (int64_t)batch * 2 * I, act, I, batch);
            DS_CHECK(check_launch("feather_decode_step (swiglu)"));
        }
        DS_CHECK(gemv_x(L.w_down, act, delta, H, I, P.s_down));
        pending = delta;
    }
    launch_norm<MODE>(batch, s, h, pending, P.s_down, hs, dec->norm_final, xq, H, dec->rms_eps);
    DS_CHECK(check_launch("feather_decode_step (final norm)"));
    DS_CHECK(feather_gemv_fp8_batched(dec->w_lm_head, xq, logits, dec->vocab, H, batch, MODE, st));
#undef DS_CHECK
    return FEATHER_OK;
}

static int64_t step_scratch_bytes(const feather_decoder_t *dec, int64_t batch, int64_t max_ctx) {
    const StepPlan P = plan_step(dec, batch, max_ctx);
    auto up = [](int64_t b) { return (b + 255) / 256 * 256; };
    return (int64_t)(P.b_h + P.b_delta + P.b_xq + P.b_act + P.b_qkv + P.b_qp + P.b_gu + P.b_ctx + P.b_plan + P.b_cs) +
           up(feather_paged_attn_scratch_bytes(batch, dec->n_q_heads, dec->head_dim, max_ctx));
}

}  // namespace feather

using namespace feather;

static int check_decoder(const feather_decoder_t *dec, int64_t batch, int64_t max_ctx, const char *me) {
    FEATHER_CHECK(dec, FEATHER_EINVAL, "%s: null decoder", me);
    FEATHER_CHECK(dec->mode == FEATHER_E5M2 || dec->mode == FEATHER_E4M3, FEATHER_EMODE, "%s: mode %d not supported", me,
                  dec->mode);
    FEATHER_CHECK(dec->n_layers >= 0 && dec->hidden > 0 && dec->n_q_heads > 0 && dec->n_kv_heads > 0 &&
                      dec->head_dim > 0 && dec->inter > 0 && dec->vocab > 0 && dec->block_size > 0 && dec->max_blocks > 0 &&
                      dec->n_blocks > 0,
                  FEATHER_EINVAL, "%s: bad configuration", me);
    FEATHER_CHECK(dec->hidden == dec->n_q_heads * dec->head_dim, FEATHER_ESHAPE, "%s: hidden != n_q_heads * head_dim", me);
    FEATHER_CHECK(dec->head_dim == 64 || dec->head_dim == 128 || dec->head_dim == 256, FEATHER_ESHAPE,
                  "%s: head dim %d not supported", me, dec->head_dim);
    FEATHER_CHECK(dec->n_q_heads % dec->n_kv_heads == 0 && dec->n_q_heads / dec->n_kv_heads <= 16, FEATHER_ESHAPE,
                  "%s: unsupported head grouping", me);
    FEATHER_CHECK(dec->hidden % 16 == 0 && dec->inter % 16 == 0, FEATHER_ESHAPE,
                  "%s: hidden and inter must be multiples of 16", me);
    FEATHER_CHECK(batch >= 1 && batch <= 64, FEATHER_ESHAPE, "%s: batch %lld outside [1, 64]", me, (long long)batch);
    FEATHER_CHECK(max_ctx >= 1 && max_ctx <= (int64_t)dec->max_blocks * dec->block_size, FEATHER_ESHAPE,
                  "%s: max_ctx exceeds the block table", me);
    return FEATHER_OK;
}

extern "C" int feather_decode_step_attention_path(const feather_decoder_t *dec, int64_t batch, int64_t max_ctx) {
    if (check_decoder(dec, batch, max_ctx, "feather_decode_step_attention_path") != FEATHER_OK) return -1;
    return plan_step(dec, batch, max_ctx).fused_attn ? 1 : 0;
}

extern "C" int64_t feather_decode_step_scratch_bytes(const feather_decoder_t *dec, int64_t batch, int64_t max_ctx) {
    if (check_decoder(dec, batch, max_ctx, "feather_decode_step_scratch_bytes") != FEATHER_OK) return -1;
    return step_scratch_bytes(dec, batch, max_ctx);
}

extern "C" int feather_decode_step(const feather_decoder_t *dec, const void *token_ids, const void *block_tables,
                                   const void *ctx_lens, int64_t batch, int64_t max_ctx, void *scratch,
                                   void *logits_f32, void *seq_status, void *stream) {
    const char *me = "feather_decode_step";
    int rc = check_decoder(dec, batch, max_ctx, me);
    if (rc != FEATHER_OK) return rc;
    FEATHER_CHECK(token_ids && block_tables && ctx_lens && scratch && logits_f32, FEATHER_EINVAL, "%s: null pointer", me);
    FEATHER_CHECK(dec->embed_f16 && dec->norm_final && dec->w_lm_head && (dec->n_layers == 0 || dec->layers), FEATHER_EINVAL,
                  "%s: null weight pointer", me);
    for (int l = 0; l < dec->n_layers; l++) {
        const feather_decoder_layer_t &L = dec->layers[l];
        FEATHER_CHECK(L.w_qkv && L.w_o && L.w_gate_up && L.w_down && L.norm_attn && L.norm_mlp && L.k_cache && L.v_cache,
                      FEATHER_EINVAL, "%s: null pointer in layer %d", me, l);
    }
    FEATHER_CHECK(aligned(scratch, 256) && aligned(logits_f32, 16) && aligned(seq_status, 4), FEATHER_EINVAL,
                  "%s: misaligned scratch/logits/status", me);
    hipStream_t s = (hipStream_t)stream;
    if (dec->mode == FEATHER_E5M2)
        return run_step<FEATHER_E5M2>(dec, (const int32_t *)token_ids, (const int32_t *)block_tables,
                                      (const int32_t *)ctx_lens, (int)batch, (int)max_ctx, scratch, (float *)logits_f32,
                                      (int32_t *)seq_status, s);
    return run_step<FEATHER_E4M3>(dec, (const int32_t *)token_ids, (const int32_t *)block_tables,
                                  (const int32_t *)ctx_lens, (int)batch, (int)max_ctx, scratch, (float *)logits_f32,
                                      (int32_t *)seq_status, s);
}

// ---- the fused producers of the step as entry points of their own -------------------------------

extern "C" int feather_add_rmsnorm_pack(void *h_f32, const void *delta_f32, int64_t n_part, int64_t part_stride,
                                        const void *gain_f32, void *xq_u32, void *y_f32, int64_t batch, int64_t hidden,
                                        float eps, int mode, void *stream) {
    const char *me = "feather_add_rmsnorm_pack";
    FEATHER_CHECK(mode == FEATHER_E5M2 || mode == FEATHER_E4M3, FEATHER_EMODE, "%s: mode %d not supported", me, mode);
    FEATHER_CHECK(batch >= 0 && batch < (1ll << 31) && hidden > 0 && hidden < (1ll << 31), FEATHER_EINVAL, "%s: bad shape", me);
    FEATHER_CHECK(hidden % 4 == 0, FEATHER_ESHAPE, "%s: hidden=%lld is not a multiple of 4", me, (long long)hidden);
    FEATHER_CHECK(!delta_f32 || (n_part >= 1 && n_part <= 64 && part_stride >= 0 && part_stride % 4 == 0), FEATHER_EINVAL,
                  "%s: n_part must be in [1, 64] and part_stride a non-negative multiple of 4", me);
    FEATHER_CHECK(eps >= 0.f, FEATHER_EINVAL, "%s: negative eps", me);
    if (batch == 0) return FEATHER_OK;
    FEATHER_CHECK(h_f32 && gain_f32 && xq_u32, FEATHER_EINVAL, "%s: null pointer", me);
    FEATHER_CHECK(aligned(h_f32, 16) && aligned(delta_f32, 16) && aligned(gain_f32, 16) && aligned(xq_u32, 4) && aligned(y_f32, 16),
                  FEATHER_EINVAL, "%s: misaligned pointer", me);
    hipStream_t s = (hipStream_t)stream;
    if (mode == FEATHER_E5M2)
        launch_norm<FEATHER_E5M2>((int)batch, s, (float *)h_f32, (const float *)delta_f32, (int)n_part, part_stride, gain_f32,
                                  (uint32_t *)xq_u32, (int)hidden, eps, (float *)y_f32);
    else
        launch_norm<FEATHER_E4M3>((int)batch, s, (float *)h_f32, (const float *)delta_f32, (int)n_part, part_stride, gain_f32,
                                  (uint32_t *)xq_u32, (int)hidden, eps, (float *)y_f32);
    return check_launch(me);
}

extern "C" int feather_rope_append(const void *qkv_f32, int64_t n_part, int64_t part_stride, const void *ctx_lens,
                                   const void *block_tables, void *q_packed, void *k_cache, void *v_cache, void *ctx_after,
                                   void *seq_status, void *rot_f32, int64_t batch, int64_t n_q_heads, int64_t n_kv_heads,
                                   int64_t d, int64_t block_size, int64_t max_blocks, int64_t n_blocks, float rope_theta,
                                   int mode, void *stream) {
    const char *me = "feather_rope_append";
    FEATHER_CHECK(mode == FEATHER_E5M2 || mode == FEATHER_E4M3, FEATHER_EMODE, "%s: mode %d not supported", me, mode);
    FEATHER_CHECK(batch >= 0 && batch < 65536 && n_q_heads > 0 && n_kv_heads > 0 && block_size > 0 && max_blocks > 0 &&
                      n_blocks > 0 && n_blocks < (1ll << 31) && max_blocks * block_size < (1ll << 31),
                  FEATHER_EINVAL, "%s: bad shape", me);
    FEATHER_CHECK(d > 0 && d % 8 == 0 && d <= 1024, FEATHER_ESHAPE, "%s: head dim %lld is not a multiple of 8", me, (long long)d);
    FEATHER_CHECK(n_q_heads < (1ll << 31) && n_kv_heads < (1ll << 31) && (n_q_heads + 2 * n_kv_heads) * (d / 8) <= 65535ll * kRopeThreads, FEATHER_ESHAPE,
                  "%s: (n_q_heads + 2 n_kv_heads) * d / 8 = %lld exceeds the grid (%lld)", me,
                  (long long)((n_q_heads + 2 * n_kv_heads) * (d / 8)), 65535ll * kRopeThreads);
    FEATHER_CHECK(n_part >= 1 && n_part <= 64 && part_stride >= 0 && part_stride % 4 == 0, FEATHER_EINVAL,
                  "%s: n_part must be in [1, 64] and part_stride a non-negative multiple of 4", me);
    FEATHER_CHECK(rope_theta > 0.f, FEATHER_EINVAL, "%s: rope_theta must be positive", me);
    if (batch == 0) return FEATHER_OK;
    FEATHER_CHECK(qkv_f32 && ctx_lens && block_tables && q_packed && k_cache && v_cache && ctx_after, FEATHER_EINVAL,
                  "%s: null pointer", me);
    FEATHER_CHECK(aligned(qkv_f32, 16) && aligned(ctx_lens, 4) && aligned(block_tables, 4) && aligned(q_packed, 4) &&
                      aligned(k_cache, 4) && aligned(v_cache, 4) && aligned(ctx_after, 4) && aligned(seq_status, 4) &&
                      aligned(rot_f32, 16),
                  FEATHER_EINVAL, "%s: misaligned pointer", me);
    const int heads = (int)(n_q_heads + 2 * n_kv_heads);
    const dim3 grid((unsigned)batch, (unsigned)((heads * (d / 8) + kRopeThreads - 1) / kRopeThreads));
#define FEATHER_ROPE(MM)                                                                                                \
    hipLaunchKernelGGL((rope_append_kernel<MM>), grid, dim3(kRopeThreads), 0, (hipStream_t)stream, (const float *)qkv_f32, \
                       (const int32_t *)ctx_lens, (const int32_t *)block_tables, part_stride, (int)n_part, (int)n_q_heads, \
                       (int)n_kv_heads, (int)d, (int)block_size, (int)max_blocks, log2f(rope_theta), (uint32_t *)q_packed, \
                       (uint32_t *)k_cache, (uint32_t *)v_cache, (int32_t *)ctx_after, (int)n_blocks, (int32_t *)seq_status, \
                       (float *)rot_f32, (int)(max_blocks * block_size))
    if (mode == FEATHER_E5M2) FEATHER_ROPE(FEATHER_E5M2); else FEATHER_ROPE(FEATHER_E4M3);
#undef FEATHER_ROPE
    return check_launch(me);
}
