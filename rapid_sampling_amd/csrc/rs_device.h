// Device-side building blocks of the MI355X token sampler: canonical
// element-wise arithmetic, wave64 reductions and scans on the DPP data path,
// Philox.
//
// Arithmetic contract (shared with the CPU oracle used by the tests): every
// floating-point step is a single IEEE fp32 operation (compile with
// -ffp-contract=off; fused multiply-adds are explicit), and everything summed
// across tokens is an integer, so no result depends on how tokens are spread
// over lanes, waves or workgroups.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace rs {

constexpr int kWave = 64;

// ---------------------------------------------------------------- scalars --

// NaN -> 0, +-Inf -> +-FLT_MAX            (reference: sampling.cu:131-134)
__device__ __forceinline__ float sf(float x)
{
    float y = (x != x) ? 0.0f : x;
    return fminf(fmaxf(y, -3.402823466e+38f), 3.402823466e+38f);
}

typedef unsigned __int128 u128;

constexpr uint32_t kEMinBits = 0x2B800000u;               // bit pattern of 2^-40, the smallest live e
constexpr uint32_t kDeadBits = 0x2B000000u;               // 2^-41: where the registers keep what lies below

// A token whose e falls below 2^-40 is DEAD: its probability is exactly 0 (the reference's
// exp2f(x - max) underflows to 0 likewise, 149 octaves down, sampling.cu:235), it takes no part
// in the selection and can never be returned -- a logit masked with -inf must not come back
// however large top_k and top_p are.  In registers and histograms a dead token is any bit
// pattern below kEMinBits (kept at or above kDeadBits so that it still has a histogram bin,
// one octave below the live ones, where counts can be checked for completeness); everything
// that weighs or selects tokens looks at patterns >= kEMinBits only.

// Bit pattern of e = 2^(x - M), M = floor(max x) of the row (reference:
// exp2f(x - max) at sampling.cu:235; the common factor 2^(max - M) cancels in
// every probability).  n = floor(x) and f = x - n are exact; 2^f is a degree-5
// Horner polynomial with positive coefficients (monotone, poly(1) < 2); the
// result is scaled by 2^(n - M), n - M <= 0; what falls below 2^-40 is dead
// (kept here as something in [2^-41, 2^-40), see above).
// The significand depends on x alone, so a slice can use its own M and be
// re-based later by an exponent shift.
//
// This is the inner loop of every kernel, and the vector ALU is what bounds
// the streaming pass once the logits arrive fast enough, so the instruction
// count is kept down by hand: the Horner steps with a literal addend are
// written as v_fmaak_f32 (the compiler otherwise spends a move per step on
// some of them), and the scaling is v_cvt_i32_f32 (which saturates) +
// v_ldexp_f32 (exact; anything below 2^-41, zero included, ends at the clamp).
__device__ __forceinline__ uint32_t e_bits_of(float x, float M)
{
    const float n = __builtin_floorf(x);
    const float f = x - n;
    float p = __builtin_fmaf(0x1.e974fap-10f, f, 0x1.277856p-7f);
    asm("v_fmaak_f32 %0, %1, %2, 0x3d648e73" : "=v"(p) : "v"(p), "v"(f));      // p * f + 0x1.c91ce6p-5
    asm("v_fmaak_f32 %0, %1, %2, 0x3e75edab" : "=v"(p) : "v"(p), "v"(f));      // p * f + 0x1.ebdb56p-3
    asm("v_fmaak_f32 %0, %1, %2, 0x3f31725d" : "=v"(p) : "v"(p), "v"(f));      // p * f + 0x1.62e4bap-1
    p = __builtin_fmaf(p, f, 1.0f);
    int k;
    asm("v_cvt_i32_f32 %0, %1" : "=v"(k) : "v"(n - M));
    return __float_as_uint(fmaxf(__builtin_ldexpf(p, k), 0x1p-41f));
}

// The same without the clamp: whatever lies below 2^-40 (zero included) is dead.  For
// code that can tell such tokens by their bin and saves the instruction.
__device__ __forceinline__ uint32_t e_bits_raw(float x, float M)
{
    const float n = __builtin_floorf(x);
    const float f = x - n;
    float p = __builtin_fmaf(0x1.e974fap-10f, f, 0x1.277856p-7f);
    asm("v_fmaak_f32 %0, %1, %2, 0x3d648e73" : "=v"(p) : "v"(p), "v"(f));
    asm("v_fmaak_f32 %0, %1, %2, 0x3e75edab" : "=v"(p) : "v"(p), "v"(f));
    asm("v_fmaak_f32 %0, %1, %2, 0x3f31725d" : "=v"(p) : "v"(p), "v"(f));
    p = __builtin_fmaf(p, f, 1.0f);
    int k;
    asm("v_cvt_i32_f32 %0, %1" : "=v"(k) : "v"(n - M));
    return __float_as_uint(__builtin_ldexpf(p, k));
}

// Exact weight of a live token from the bit pattern of e (2^-40 <= e < 2):
// W = e * 2^63 = significand24 << (exponent - 87), in [2^23, 2^64).
__device__ __forceinline__ uint64_t w_of_bits(uint32_t b)
{
    return (uint64_t)((b & 0x7FFFFFu) | 0x800000u) << ((b >> 23) - 87u);
}

// ceil(f * s) for a float 0 < f <= 1 and s < 2^100, exact, clamped to [1, s].
__device__ inline u128 ceil_mul(float f, u128 s)
{
    if (!(f > 0.0f)) return 1;
    if (f >= 1.0f) return s;
    const uint32_t b = __float_as_uint(f);
    int ex = (int)(b >> 23);
    uint64_t m = b & 0x7FFFFFu;
    if (ex == 0) ex = 1; else m |= 0x800000u;
    const int sh = 150 - ex;                                // f = m * 2^-sh, sh >= 24
    u128 r;
    if (sh >= 126) r = 1;                                   // 0 < m*s < 2^124 < 2^sh
    else r = ((u128)m * s + (((u128)1 << sh) - 1)) >> sh;
    if (r < 1) r = 1;
    if (r > s) r = s;
    return r;
}

// 64 random bits -> r in [1, S]: floor(u64 * S / 2^64) + 1
__device__ __forceinline__ u128 r_from_bits(uint64_t u64, u128 S)
{
    const uint64_t s_lo = (uint64_t)S, s_hi = (uint64_t)(S >> 64);
    return (u128)u64 * s_hi + __umul64hi(u64, s_lo) + 1;
}

// floor(a / d) for a < 2^96 and a 32-bit divisor, by 32-bit long division
__device__ inline u128 div_u32(u128 a, uint32_t d)
{
    uint64_t rem = 0;
    u128 q = 0;
#pragma unroll
    for (int i = 2; i >= 0; --i) {
        const uint64_t cur = (rem << 32) | (uint32_t)(a >> (32 * i));
        const uint64_t qi = cur / d;
        rem = cur - qi * d;
        q |= (u128)qi << (32 * i);
    }
    return q;
}

// order-preserving map float -> uint32 (for atomicMax on floats)
__device__ __forceinline__ uint32_t fkey(float x)
{
    const uint32_t b = __float_as_uint(x);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
__device__ __forceinline__ float fkey_inv(uint32_t k)
{
    return __uint_as_float((k & 0x80000000u) ? (k & 0x7FFFFFFFu) : ~k);
}

// ---------------------------------------------------------- Philox4x32-10 --
// Counter-based generator of Salmon et al.; same stream layout as the
// reference's curand_init(seed, row, 0) (sampling.cu:137): key = seed,
// counter = (draw_lo, draw_hi, row_lo, row_hi).
__device__ inline void philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3,
                                     uint32_t k0, uint32_t k1, uint32_t out[4])
{
#pragma unroll
    for (int i = 0; i < 10; ++i) {
        const uint64_t p0 = (uint64_t)0xD2511F53u * c0;
        const uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
        const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
        const uint32_t n1 = (uint32_t)p1;
        const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
        const uint32_t n3 = (uint32_t)p0;
        c0 = n0; c1 = n1; c2 = n2; c3 = n3;
        k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
    }
    out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

// ------------------------------------------------------ wave64 primitives --
// All cross-lane traffic uses DPP (data-parallel primitives on the VALU
// operand path): row_shr:1,2,4,8 scan inside each row of 16 lanes, then
// row_bcast:15 carries lane 15 of a row into the next row (rows 1 and 3),
// row_bcast:31 carries lane 31 into rows 2 and 3.  Six steps, no LDS.  Lanes
// with no source read 0 (the identity of + and of max on unsigned).

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t dpp0_u32(uint32_t v)
{
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, ROW_MASK, 0xf, false);
}
template <int CTRL, int ROW_MASK, typename T>
__device__ __forceinline__ T dpp0(T v)
{
    static_assert(sizeof(T) == 4 || sizeof(T) == 8 || sizeof(T) == 16, "32-, 64- or 128-bit integers");
    if constexpr (sizeof(T) == 4) return (T)dpp0_u32<CTRL, ROW_MASK>((uint32_t)v);
    else if constexpr (sizeof(T) == 8) {
        const uint32_t lo = dpp0_u32<CTRL, ROW_MASK>((uint32_t)v), hi = dpp0_u32<CTRL, ROW_MASK>((uint32_t)((uint64_t)v >> 32));
        return (T)(((uint64_t)hi << 32) | lo);
    } else {
        const uint64_t lo = dpp0<CTRL, ROW_MASK>((uint64_t)v), hi = dpp0<CTRL, ROW_MASK>((uint64_t)((u128)v >> 64));
        return (T)(((u128)hi << 64) | lo);
    }
}

// Inclusive scan (sum) over the 64 lanes; lane 63 ends with the wave total.
// The reference's float ladder has to run 16,8,4,2,1 to stay monotone
// (sampling.cu:48-58); these are integers, exact in any order.
template <typename T>
__device__ __forceinline__ T wave_inclusive_scan(T v)
{
    v += dpp0<0x111, 0xf>(v);     // row_shr:1
    v += dpp0<0x112, 0xf>(v);     // row_shr:2
    v += dpp0<0x114, 0xf>(v);     // row_shr:4
    v += dpp0<0x118, 0xf>(v);     // row_shr:8
    v += dpp0<0x142, 0xa>(v);     // row_bcast:15 -> rows 1,3
    v += dpp0<0x143, 0xc>(v);     // row_bcast:31 -> rows 2,3
    return v;
}

__device__ __forceinline__ uint32_t lane63_u32(uint32_t v) { return (uint32_t)__builtin_amdgcn_readlane((int)v, 63); }
template <typename T>
__device__ __forceinline__ T lane63(T v)
{
    if constexpr (sizeof(T) == 4) return (T)lane63_u32((uint32_t)v);
    else if constexpr (sizeof(T) == 8) return (T)(((uint64_t)lane63_u32((uint32_t)((uint64_t)v >> 32)) << 32) | lane63_u32((uint32_t)v));
    else return (T)(((u128)lane63((uint64_t)((u128)v >> 64)) << 64) | lane63((uint64_t)v));
}

// Sum over the wave, returned to every lane (wave-uniform).
template <typename T>
__device__ __forceinline__ T wave_sum(T v) { return lane63(wave_inclusive_scan(v)); }

__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v)
{
    v = max(v, dpp0_u32<0x111, 0xf>(v));
    v = max(v, dpp0_u32<0x112, 0xf>(v));
    v = max(v, dpp0_u32<0x114, 0xf>(v));
    v = max(v, dpp0_u32<0x118, 0xf>(v));
    v = max(v, dpp0_u32<0x142, 0xa>(v));
    v = max(v, dpp0_u32<0x143, 0xc>(v));
    return lane63_u32(v);
}

}  // namespace rs
