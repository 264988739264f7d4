// The quantising encoders of the pools, shared by the append kernels and by the attention kernels
// that take a new row in flight: both must store the very same codes.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "f16_rule.hpp"

namespace bkv {

// binary16 code -> f32 under the cache's load rule (f16_storage.glsl:58-69):
// exponent field 0 reads as a signed zero.
__device__ __forceinline__ float f16_load(uint32_t h) {
    const uint32_t sign = (h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1fu;
    const uint32_t m = h & 0x3ffu;
    if (e == 0) return __uint_as_float(sign);
    if (e == 31) return __uint_as_float(sign | 0x7f800000u | (m << 13));
    return __uint_as_float(sign | ((e + 112u) << 23) | (m << 13));
}

// ---- the encoders' primitives, on 8 consecutive values of a 32-value block ----------------
// The append kernels give a block to four neighbouring lanes (8 values each, so that a wave's
// loads are contiguous); the attention kernels that take a new row in flight give it to one lane.
// Both go through these functions, so both store the very same codes.

__device__ __forceinline__ float amax8(const float (&x)[8], float amax = 0.0f) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float a = fabsf(x[i]);
        amax = a > amax ? a : amax;  // a NaN is never taken
    }
    return amax;
}

// max over the four lanes of a quad (DPP quad_perm [1,0,3,2], then [2,3,0,1]); every lane of the
// quad must be active.  Exact and independent of the order: no operand is a NaN.
__device__ __forceinline__ float quad_max(float a) {
    const float b = __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, a), 0xB1, 0xf, 0xf, false));
    a = b > a ? b : a;
    const float c = __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, a), 0x4E, 0xf, 0xf, false));
    return c > a ? c : a;
}

// q8_0 rule (shaders/qsa_kv_append.comp:113-132, qsa/cpu.rs:65-82): scale = amax/127 (1 if amax
// == 0), q = round-half-away(clamp(x/scale, +-127)); 8 codes = 2 words, element j in byte j % 4.
__device__ __forceinline__ float q8v_scale(float amax) { return amax > 0.0f ? amax / 127.0f : 1.0f; }

__device__ __forceinline__ void q8_codes8(const float (&x)[8], float scale, uint32_t& w0, uint32_t& w1) {
    uint32_t w[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        uint32_t packed = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float t = x[j * 4 + i] / scale;
            t = t < -127.0f ? -127.0f : t;
            t = t > 127.0f ? 127.0f : t;
            const int q = (int)roundf(t);
            packed |= ((uint32_t)q & 0xffu) << (8 * i);
        }
        w[j] = packed;
    }
    w0 = w[0];
    w1 = w[1];
}

// The int8 layout with f16 scales: the q8_0 rule with the scale stored through the cache's f16
// encoding; a scale the f16 rule would flush is raised to 2^-14.  (No reference counterpart.)
__device__ __forceinline__ uint32_t i8h_scale_bits(float amax) {
    if (!(amax > 0.0f)) return 0x3c00u;
    const uint32_t hb = f16_store_bits(amax / 127.0f);
    return (hb & 0x7fffu) == 0 ? 0x0400u : hb;
}

__device__ __forceinline__ void i8h_codes8(const float (&x)[8], float sh, uint32_t& w0, uint32_t& w1) {
    uint32_t w[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        uint32_t packed = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float t = x[j * 4 + i] / sh;
            t = !(t >= -127.0f) ? -127.0f : t;
            t = t > 127.0f ? 127.0f : t;
            const int q = (int)roundf(t);
            packed |= ((uint32_t)q & 0xffu) << (8 * i);
        }
        w[j] = packed;
    }
    w0 = w[0];
    w1 = w[1];
}

// The codes of 8 values on a reciprocal of the scale, r = v_rcp_f32(scale), good to one ulp:
// fma(x, r, 1.5 * 2^23) rounds the exact product x * r to the nearest integer n (ties to even) and
// leaves n's two's-complement low byte in the low byte of its bit pattern; d = fma(x, r, -n) is
// the product's distance from n.  The exact product is within 127 * 2^-23 of the quotient x /
// scale and the rule's correctly rounded quotient within 2^-18 of that, together less than 2^-15:
// where |d| < 1/2 - 2^-15 all three lie between the same two half-integers, so n is the rule's
// round-half-away(clamp(x / scale)) (|x| <= amax keeps the quotient inside the clamp).  `doubt`
// collects the largest d * d as an unsigned bit pattern -- a NaN's is larger than any number's --
// and the caller takes the exact path (q8_codes8 / i8h_codes8) where codes_in_doubt() says so:
// for the whole wave, so that the branch is uniform; one wave in 16 of N(0,1) rows does.
__device__ __forceinline__ void codes8_on_reciprocal(const float (&x)[8], float scale, uint32_t& w0, uint32_t& w1,
                                                     uint32_t& doubt) {
    const float r = __builtin_amdgcn_rcpf(scale);
    // a scale whose reciprocal or products could leave the normal range is always in doubt
    if (!(scale >= 0x1p-64f && scale <= 0x1p64f)) doubt = 0x7fc00000u;
    uint32_t y[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float yi = __builtin_fmaf(x[i], r, 12582912.0f);
        const float d = __builtin_fmaf(x[i], r, -(yi - 12582912.0f));
        const uint32_t d2 = __float_as_uint(d * d);
        doubt = d2 > doubt ? d2 : doubt;
        y[i] = __float_as_uint(yi);
    }
    // low bytes of four words into one
    w0 = __builtin_amdgcn_perm(__builtin_amdgcn_perm(y[3], y[2], 0x0c0c0400u),
                               __builtin_amdgcn_perm(y[1], y[0], 0x0c0c0400u), 0x05040100u);
    w1 = __builtin_amdgcn_perm(__builtin_amdgcn_perm(y[7], y[6], 0x0c0c0400u),
                               __builtin_amdgcn_perm(y[5], y[4], 0x0c0c0400u), 0x05040100u);
}
__device__ __forceinline__ bool codes_in_doubt(uint32_t doubt) {
    // rounding is monotonic: |d| >= 1/2 - 2^-15 implies rounded d * d >= this rounded square
    constexpr float kSure = (0.5f - 0x1p-15f) * (0.5f - 0x1p-15f);
    return doubt >= __builtin_bit_cast(uint32_t, kSure);
}

// The same for values that are binary16 numbers against a scale that is one (the int8 layout
// fed with f16 rows): the quotient of two 11-bit significands is either exactly a half-integer --
// which happens once in some 2000 values, too often for the exact path -- or at least 2^-13 away
// from every one of them.  With the reciprocal raised by 2^-21 (four times its error bound) the
// exact product lies strictly beyond an exact tie, on the side away from zero, and stays on its
// side of every half-integer otherwise (127 * 2^-21 + 2^-15 < 2^-13), so the rounding of the fma
// alone gives the rule's code: no distance, no doubt.  tests/cpp/i8h_f16_codes_exhaustive.c walks
// every (amax, x) pair of binary16 numbers with reciprocals one ulp off either way.  The caller
// keeps NaN, infinities and blocks whose amax is at most 2^-6 away from this path.
constexpr float kTieBias = 1.0f + 0x1p-21f;
__device__ __forceinline__ void codes8_f16_on_biased_reciprocal(const float (&x)[8], float r_biased, uint32_t& w0,
                                                               uint32_t& w1) {
    uint32_t y[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) y[i] = __float_as_uint(__builtin_fmaf(x[i], r_biased, 12582912.0f));
    w0 = __builtin_amdgcn_perm(__builtin_amdgcn_perm(y[3], y[2], 0x0c0c0400u),
                               __builtin_amdgcn_perm(y[1], y[0], 0x0c0c0400u), 0x05040100u);
    w1 = __builtin_amdgcn_perm(__builtin_amdgcn_perm(y[7], y[6], 0x0c0c0400u),
                               __builtin_amdgcn_perm(y[5], y[4], 0x0c0c0400u), 0x05040100u);
}

// the value of a binary16 code that is not a subnormal (scales never are): the hardware convert
__device__ __forceinline__ float f16_normal_value(uint32_t h) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
}

// ---- a whole block in one lane -------------------------------------------------------------
__device__ __forceinline__ float amax32(const float (&x)[32]) {
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 32; ++i) {
        const float a = fabsf(x[i]);
        amax = a > amax ? a : amax;
    }
    return amax;
}

__device__ __forceinline__ void q8_block(const float (&x)[32], float scale, uint32_t (&w)[8]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float y[8] = {x[8 * j], x[8 * j + 1], x[8 * j + 2], x[8 * j + 3],
                            x[8 * j + 4], x[8 * j + 5], x[8 * j + 6], x[8 * j + 7]};
        q8_codes8(y, scale, w[2 * j], w[2 * j + 1]);
    }
}

// One q8_0 block as the V pool holds it: w[0] = f32 scale, w[1..8] = 32 x i8.
__device__ __forceinline__ void q8v_block_words(const float (&x)[32], uint32_t (&w)[9]) {
    const float scale = q8v_scale(amax32(x));
    uint32_t c[8];
    q8_block(x, scale, c);
    w[0] = __float_as_uint(scale);
#pragma unroll
    for (int j = 0; j < 8; ++j) w[1 + j] = c[j];
}

// One block of the int8 layout: w = 32 x i8, scale_bits = the binary16 code of the scale.
__device__ __forceinline__ void i8h_block_words(const float (&x)[32], uint32_t (&w)[8], uint32_t& scale_bits) {
    const uint32_t hb = i8h_scale_bits(amax32(x));
    const float sh = f16_load(hb);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float y[8] = {x[8 * j], x[8 * j + 1], x[8 * j + 2], x[8 * j + 3],
                            x[8 * j + 4], x[8 * j + 5], x[8 * j + 6], x[8 * j + 7]};
        i8h_codes8(y, sh, w[2 * j], w[2 * j + 1]);
    }
    scale_bits = hb;
}

}  // namespace bkv
