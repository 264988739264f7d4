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

// q8_0 codes of 32 values (shaders/qsa_kv_append.comp:113-132, qsa/cpu.rs:65-82):
// scale = amax/127 (1 if amax == 0), q = round-half-away(clamp(x/scale, +-127)).
__device__ __forceinline__ void q8_block(const float (&x)[32], float scale, uint32_t (&w)[8]) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
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
}

__device__ __forceinline__ float amax32(const float (&x)[32]) {
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 32; ++i) {
        const float a = fabsf(x[i]);
        amax = a > amax ? a : amax;
    }
    return amax;
}

// One q8_0 block as the V pool holds it: w[0] = f32 scale, w[1..8] = 32 x i8.
__device__ __forceinline__ void q8v_block_words(const float (&x)[32], uint32_t (&w)[9]) {
    const float amax = amax32(x);
    const float scale = amax > 0.0f ? amax / 127.0f : 1.0f;
    uint32_t c[8];
    q8_block(x, scale, c);
    w[0] = __float_as_uint(scale);
#pragma unroll
    for (int j = 0; j < 8; ++j) w[1 + j] = c[j];
}

// One block of the int8 layout with f16 scales: the q8_0 rule with the scale stored through the
// cache's f16 encoding; a scale the f16 rule would flush is raised to 2^-14.  w = 32 x i8,
// scale_bits = the binary16 code of the scale.  (No reference counterpart.)
__device__ __forceinline__ void i8h_block_words(const float (&x)[32], uint32_t (&w)[8], uint32_t& scale_bits) {
    const float amax = amax32(x);
    uint32_t hb;
    if (amax > 0.0f) {
        hb = f16_store_bits(amax / 127.0f);
        if ((hb & 0x7fffu) == 0) hb = 0x0400u;
    } else {
        hb = 0x3c00u;
    }
    const float sh = f16_load(hb);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
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
    scale_bits = hb;
}

}  // namespace bkv
