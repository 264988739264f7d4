// The cache's f32 -> binary16 storage rule as a device function, shared by the append kernels
// and the fused decode step (crates/breccia-kernels/shaders/f16_storage.glsl:26-55,
// crates/breccia-kernels/src/qsa/cpu.rs:23-53): round-to-nearest-even like the hardware
// convert, except that every |x| < 2^-14 becomes a signed zero (no subnormals, even where
// rounding would reach 2^-14) and NaN becomes a signed infinity.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace bkv {

__device__ __forceinline__ uint32_t f16_store_bits(float x) {
    const uint32_t b = __float_as_uint(x);
    const uint32_t sign = (b >> 16) & 0x8000u;
    const uint32_t mag = b & 0x7fffffffu;
    const _Float16 h = static_cast<_Float16>(x);  // v_cvt_f16_f32, RNE, overflow -> inf
    uint32_t code = static_cast<uint32_t>(__builtin_bit_cast(uint16_t, h));
    if (mag < 0x38800000u) code = sign;
    if (mag > 0x7f800000u) code = sign | 0x7c00u;
    return code;
}

__device__ __forceinline__ uint32_t f16_store_pair(float lo, float hi) {
    return f16_store_bits(lo) | (f16_store_bits(hi) << 16);
}

}  // namespace bkv
