// Shared device/host helpers for the gfx950 kernels: FP8 decode in registers,
// wave64 reductions, error reporting.  Wave size is 64 everywhere.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/feather_hip.h"

namespace feather {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;

// ---------------------------------------------------------------- host side

void set_error(const char *fmt, ...);

#define FEATHER_CHECK(cond, code, ...)      \
    do {                                    \
        if (!(cond)) {                      \
            feather::set_error(__VA_ARGS__); \
            return (code);                  \
        }                                   \
    } while (0)

inline int check_launch(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("%s: launch failed: %s", what, hipGetErrorString(e));
        return FEATHER_ELAUNCH;
    }
    return FEATHER_OK;
}

inline bool aligned(const void *p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

// Kernels that ask for more than 64 KB of dynamic LDS need the limit raised once per device (the
// attribute belongs to the device's copy of the code).  `done` is one bit mask per kernel
// instantiation, kept by the caller in a function-local static.
inline hipError_t raise_lds_limit(const void *kernel, size_t bytes, unsigned long long &done) {
    if (bytes <= 64 * 1024) return hipSuccess;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    const unsigned long long bit = 1ull << (dev & 63);
    if (done & bit) return hipSuccess;
    e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e == hipSuccess) done |= bit;
    return e;
}

// ---------------------------------------------------------------- bit casts

__device__ __forceinline__ half2_t as_half2(uint32_t x) { return __builtin_bit_cast(half2_t, x); }
__device__ __forceinline__ uint32_t as_u32(half2_t x) { return __builtin_bit_cast(uint32_t, x); }
__device__ __forceinline__ float as_float(uint32_t x) { return __builtin_bit_cast(float, x); }
__device__ __forceinline__ uint32_t as_u32(float x) { return __builtin_bit_cast(uint32_t, x); }

// v_perm_b32: result byte i = byte sel[i] of the 8-byte value {hi, lo}
// (0..3 = lo bytes, 4..7 = hi bytes, 0x0c = constant 0x00).
__device__ __forceinline__ uint32_t perm(uint32_t hi, uint32_t lo, uint32_t sel) {
    return __builtin_amdgcn_perm(hi, lo, sel);
}

// Streaming (non-temporal) 128-bit accesses: data touched once should not
// displace the re-used vector / K/V tiles from L2.
__device__ __forceinline__ u32x4 load_nt128(const void *p) {
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
}
__device__ __forceinline__ void store_nt128(void *p, u32x4 v) {
    __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(p));
}
__device__ __forceinline__ void store_nt64(void *p, u32x2 v) {
    __builtin_nontemporal_store(v, reinterpret_cast<u32x2 *>(p));
}

// ---------------------------------------------------------------- FP8 -> fp16 pairs

// E5M2 code c is the fp16 with bits c << 8 (reference gemv.py:31-58): decoding a
// word is byte placement.  p01 = (c0, c1), p23 = (c2, c3) as packed fp16.
__device__ __forceinline__ void dec_e5m2_word(uint32_t w, uint32_t &p01, uint32_t &p23) {
    p01 = perm(w, w, 0x010c000cu);
    p23 = perm(w, w, 0x030c020cu);
}

// E4M3 code -> fp16 bits sign | (e ? e + 8 : 0) << 10 | m << 7 (reference
// gemv.py:83-88), four codes at a time with byte-parallel integer arithmetic:
//   high byte  H = sign | (a + (e > 0 ? 0x40 : 0)) >> 1,  a = c & 0x7F = e << 3 | m
//   low byte   L = (c & 1) << 7
// (e > 0) is (a >= 8), bit 7 of a + 0x78.  v_lerp_u8 computes (x + y + (z & 1)) >> 1 on each byte with a 9-bit
// intermediate, i.e. an add and a shift in one instruction and no carry between bytes.
__device__ __forceinline__ void dec_e4m3_word(uint32_t w, uint32_t &p01, uint32_t &p23) {
    uint32_t a = w & 0x7F7F7F7Fu;
    uint32_t bias = __builtin_amdgcn_lerp(a, 0x78787878u, 0u) & 0x40404040u;
    uint32_t hi = (w & 0x80808080u) | __builtin_amdgcn_lerp(a, bias, 0u);
    uint32_t lo = (w << 7) & 0x80808080u;
    p01 = perm(hi, lo, 0x05010400u);
    p23 = perm(hi, lo, 0x07030602u);
}

template <int MODE>
__device__ __forceinline__ void dec_word(uint32_t w, uint32_t &p01, uint32_t &p23) {
    if constexpr (MODE == FEATHER_E5M2) dec_e5m2_word(w, p01, p23);
    else dec_e4m3_word(w, p01, p23);
}

// E4M3fn code -> fp16 bits with the exact (OCP) value; used by the unpack
// kernel for the CPU-API semantics (reference fp8.py:381-391).
__device__ __forceinline__ uint32_t dec_e4m3_ieee_bits(uint32_t c) {
    uint32_t sign = (c & 0x80u) << 8;
    uint32_t e = (c >> 3) & 0xFu, m = c & 7u;
    if ((c & 0x7Fu) == 0x7Fu) return sign | 0x7E00u;
    if (e) return sign | ((e + 8u) << 10) | (m << 7);
    if (!m) return sign;
    uint32_t lead = m >= 4 ? 2u : (m >= 2 ? 1u : 0u);
    return sign | ((6u + lead) << 10) | ((m << (10u - lead)) & 0x3FFu);
}

// acc += a.x * b.x + a.y * b.y with fp32 accumulation (v_dot2_f32_f16); the
// fp16 x fp16 products are exact in fp32.
__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float acc) {
    return __builtin_amdgcn_fdot2(as_half2(a), as_half2(b), acc, false);
}

// ---------------------------------------------------------------- encoders

// fp16 bits -> E5M2, round to nearest even: E5M2 is the high byte of fp16, so
// rounding is an integer add on the bit pattern (a carry bumps the exponent,
// values >= 61440 reach 0x7C = inf).  NaN -> 0x7F | sign.
__device__ __forceinline__ uint32_t enc_e5m2(uint32_t h) {
    uint32_t a = h & 0x7FFFu;
    uint32_t sign = (h >> 8) & 0x80u;
    uint32_t r = (a + 0x7Fu + ((a >> 8) & 1u)) >> 8;
    return sign | (a > 0x7C00u ? 0x7Fu : r);
}

// fp16 bits -> E4M3fn (bias 7, subnormal unit 2^-9, max 448, 0x7F = NaN), RNE.
// Anything that rounds above 448 (|x| > 464), inf and NaN give 0x7F.
__device__ __forceinline__ uint32_t enc_e4m3(uint32_t h) {
    uint32_t a = h & 0x7FFFu;
    uint32_t sign = (h >> 8) & 0x80u;
    uint32_t exp = a >> 10;
    uint32_t code;
    if (exp >= 9u) {                                  // |x| >= 2^-6: normal in E4M3
        uint32_t t = a - (8u << 10);                  // rebias 15 -> 7
        t += 0x3Fu + ((t >> 7) & 1u);                 // RNE on the 7 dropped bits
        code = min(t >> 7, 0x7Fu);
    } else {                                          // subnormal target: units of 2^-9
        uint32_t full = (a & 0x3FFu) | 0x400u;
        uint32_t sh = 16u - max(exp, 1u);             // 8..15
        uint32_t q = full >> sh;
        uint32_t rem = full & ((1u << sh) - 1u);
        uint32_t half = 1u << (sh - 1u);
        q += (rem > half || (rem == half && (q & 1u))) ? 1u : 0u;
        code = exp == 0u ? 0u : q;                    // fp16 subnormals are < 2^-10 -> 0
    }
    return sign | code;
}

// Two fp16 values (one 32-bit register) -> their two E4M3fn codes in the low bytes of the two halves
// (bits [0, 8) and [16, 24)), round to nearest even: enc_e4m3 on 16-bit lanes with packed instructions, both
// paths computed and merged bit-wise instead of a branch per element (random data takes both branches in every
// wave: the scalar encoder made the E4M3 pack kernel VALU bound, 5.0 TB/s against 6.1 TB/s for E5M2).
//   |x| >= 2^-6 (bits >= 0x2400): rebias, add 0x3F + lsb, shift: a carry moves into the exponent; capped at 0x7F
//   |x| <  2^-6: the code is round-to-nearest-even(|x| * 2^9), read from the low bits of |x| * 512 + 1024 in
//                fp16 arithmetic (the product is exact, and the ulp at 1024 is 1)
typedef uint16_t u16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t enc_e4m3_pair(uint32_t hh) {
    const uint32_t a32 = hh & 0x7FFF7FFFu;
    const u16x2_t a = __builtin_bit_cast(u16x2_t, a32);
    u16x2_t t = a - (uint16_t)0x2000;
    t = t + (uint16_t)0x3F + ((t >> (uint16_t)7) & (uint16_t)1);
    const u16x2_t norm = __builtin_elementwise_min((u16x2_t)(t >> (uint16_t)7), (u16x2_t)(uint16_t)0x7F);
    const half2_t scaled = __builtin_elementwise_fma(as_half2(a32), (half2_t)(_Float16)512.0f, (half2_t)(_Float16)1024.0f);
    const uint32_t sub = as_u32(scaled) & 0x000F000Fu;
    // all-ones halves where |x| >= 2^-6: a + 0x5C00 has bit 15 set exactly then (a <= 0x7FFF: no wrap)
    const u16x2_t big = (u16x2_t)((a + (uint16_t)0x5C00) >> (uint16_t)15) * (uint16_t)0xFFFF;
    const uint32_t m = __builtin_bit_cast(uint32_t, big);
    const uint32_t mag = (__builtin_bit_cast(uint32_t, norm) & m) | (sub & ~m);
    return mag | ((hh >> 8) & 0x00800080u);
}

template <int MODE, int ROUND>
__device__ __forceinline__ uint32_t enc(uint32_t h) {
    if constexpr (ROUND == FEATHER_ROUND_TRUNC) return (h >> 8) & 0xFFu;
    else if constexpr (MODE == FEATHER_E5M2) return enc_e5m2(h);
    else return enc_e4m3(h);
}

// four fp32 values -> one packed word: fp32 -> fp16 (RNE) -> FP8 code (RNE), the rounding chain of
// pack_fp8_tensor applied to an fp32 producer
template <int MODE>
__device__ __forceinline__ uint32_t quant4(float a, float b, float c, float d) {
    // fp32 -> fp16 (round to nearest even) -> FP8 code (round to nearest even).
    // The values are pinned in registers first: when an argument is a product, the compiler otherwise
    // folds multiply and conversion into v_fma_mixlo_f16 x, y, +0, and (-0) + (+0) = +0 loses the sign of
    // a zero product (code 0x00 instead of 0x80).
    asm volatile("" : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
    uint32_t h0 = __builtin_bit_cast(uint16_t, (_Float16)a), h1 = __builtin_bit_cast(uint16_t, (_Float16)b);
    uint32_t h2 = __builtin_bit_cast(uint16_t, (_Float16)c), h3 = __builtin_bit_cast(uint16_t, (_Float16)d);
    if constexpr (MODE == FEATHER_E5M2)
        return enc_e5m2(h0) | (enc_e5m2(h1) << 8) | (enc_e5m2(h2) << 16) | (enc_e5m2(h3) << 24);
    else   // two elements per instruction; the codes come back in bytes 0 and 2 of each pair
        return perm(enc_e4m3_pair(h2 | (h3 << 16)), enc_e4m3_pair(h0 | (h1 << 16)), 0x06040200u);
}

// the four fp16 values that a packed word decodes to (kernel decode), as two fp16 pairs
template <int MODE>
__device__ __forceinline__ u32x2 dequant4(uint32_t word) {
    uint32_t p01, p23;
    dec_word<MODE>(word, p01, p23);
    return u32x2{p01, p23};
}

// ---------------------------------------------------------------- wave64 reductions

template <int CTRL>
__device__ __forceinline__ float dpp_mov(float x) {
    return as_float((uint32_t)__builtin_amdgcn_update_dpp(0, (int)as_u32(x), CTRL, 0xF, 0xF, true));
}

// Sum over the 64 lanes of a wave; every lane of row 0 (lanes 0..15) gets the
// total.  quad_perm / row_half_mirror / row_mirror fold each 16-lane row, then
// the four row sums are read with v_readlane.
__device__ __forceinline__ float wave_sum(float x) {
    x += dpp_mov<0xB1>(x);   // quad_perm [1,0,3,2]
    x += dpp_mov<0x4E>(x);   // quad_perm [2,3,0,1]
    x += dpp_mov<0x141>(x);  // row_half_mirror
    x += dpp_mov<0x140>(x);  // row_mirror
    float r0 = as_float((uint32_t)__builtin_amdgcn_readlane((int)as_u32(x), 0));
    float r1 = as_float((uint32_t)__builtin_amdgcn_readlane((int)as_u32(x), 16));
    float r2 = as_float((uint32_t)__builtin_amdgcn_readlane((int)as_u32(x), 32));
    float r3 = as_float((uint32_t)__builtin_amdgcn_readlane((int)as_u32(x), 48));
    return (r0 + r1) + (r2 + r3);
}

// max(x, x of lane ^ 16) and max(x, x of lane ^ 32) with the gfx950 row / half-wave swaps: one
// VALU instruction each instead of an LDS permute with six instructions of index arithmetic.
// v_permlane16_swap exchanges the odd 16-lane rows of its first operand with the even rows of the
// second, v_permlane32_swap the upper half of the first with the lower half of the second; with
// both operands holding x, every lane then finds x and its partner's x in the two registers.
// (Inline assembly: the compiler folds the two results of the corresponding builtins into one when
// both inputs are the same value.  The copy and the final v_max_f32 are part of the statement so that
// exactly one copy is made and the compiler adds no canonicalising max(x, x) on values it cannot see
// through; s_nop 1 covers the VALU-write -> permlane-read wait states.)
__device__ __forceinline__ float max_xor16(float x) {
    float a = x, b;
    asm volatile("v_mov_b32 %1, %0\n\ts_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\tv_max_f32 %0, %0, %1" : "+v"(a), "=&v"(b));
    return a;
}
__device__ __forceinline__ float max_xor32(float x) {
    float a = x, b;
    asm volatile("v_mov_b32 %1, %0\n\ts_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\tv_max_f32 %0, %0, %1" : "+v"(a), "=&v"(b));
    return a;
}

// Results of the matrix core are not interlocked against the vector ALU: a vector instruction that reads an MFMA
// result needs 7 / 11 / 19 cycles of distance from a 4- / 8- / 16-pass MFMA.  The compiler counts these wait states
// for the instructions it emits itself, but it does not look into asm statements, so an asm statement must never be
// the first reader of an MFMA result: max3_raw on fresh scores now and then took the maximum over accumulators that
// the last MFMA of the chain had not updated yet -- harmless for the result (the reference point of the softmax may
// be any value), but different from run to run.  mfma_settle takes the N accumulators at `acc` as operands, which
// places it after the MFMAs that write them and before every later reader, and lets 12 cycles pass (MFMAs retire in
// order, so the distance to the last one covers all).  For 4- and 8-pass MFMAs.
#define FEATHER_SETTLE_NOPS "s_nop 7\n\ts_nop 3"
template <int N>
__device__ __forceinline__ void mfma_settle(float4_t *a) {
    static_assert(N == 1 || N == 2 || N == 4 || N == 8 || N == 16, "accumulator count");
    if constexpr (N == 1) asm volatile(FEATHER_SETTLE_NOPS : "+v"(a[0]));
    if constexpr (N == 2) asm volatile(FEATHER_SETTLE_NOPS : "+v"(a[0]), "+v"(a[1]));
    if constexpr (N == 4) asm volatile(FEATHER_SETTLE_NOPS : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]));
    if constexpr (N == 8)
        asm volatile(FEATHER_SETTLE_NOPS : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(a[4]), "+v"(a[5]), "+v"(a[6]), "+v"(a[7]));
    if constexpr (N == 16)
        asm volatile(FEATHER_SETTLE_NOPS : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(a[4]), "+v"(a[5]), "+v"(a[6]), "+v"(a[7]),
                     "+v"(a[8]), "+v"(a[9]), "+v"(a[10]), "+v"(a[11]), "+v"(a[12]), "+v"(a[13]), "+v"(a[14]), "+v"(a[15]));
}

// max of two / three floats as single instructions.  In front of fmaxf the compiler puts a canonicalising
// max(x, x) on every value whose NaN quietness it cannot prove (MFMA results, values that came out of
// inline asm): 4 of the ~80 vector instructions of a softmax block.  Scores are never signalling
// NaNs, and for quiet NaNs v_max returns the other operand, as fmaxf does.
__device__ __forceinline__ float max_raw(float a, float b) {
    float r;
    asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
__device__ __forceinline__ float max3_raw(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

__device__ __forceinline__ int lane_id() { return (int)(threadIdx.x & (kWave - 1)); }

// Index of the wave inside its workgroup, marked as wave-uniform: everything derived from it (row
// bases, query offsets, step indices) then lives in SGPRs and is computed on the scalar unit
// instead of once per lane (the compiler cannot see that threadIdx.x / 64 is uniform).
__device__ __forceinline__ int wave_id() { return __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWave)); }

}  // namespace feather
