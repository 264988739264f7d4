/*
 * f16c_ref.c -- TEST INFRASTRUCTURE.  An independent f32 -> binary16 conversion
 * (the x86 F16C instruction, round-to-nearest-even, IEEE subnormals and NaN kept)
 * used only to pin bkvo_f32_to_f16_bits over the whole 2^32 input space.
 * Built with -mf16c; callers must check the CPU flag before calling.
 */
#include <immintrin.h>
#include <stdint.h>
#include <string.h>

/* out[i] = F16C(bits = first + i), for i in [0, count); count a multiple of 8. */
void f16c_convert_range(uint32_t first, uint64_t count, uint16_t *out) {
    for (uint64_t i = 0; i < count; i += 8) {
        uint32_t b[8];
        for (int j = 0; j < 8; ++j) b[j] = first + (uint32_t)(i + j);
        __m256 x;
        memcpy(&x, b, 32);
        __m128i h = _mm256_cvtps_ph(x, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC);
        memcpy(out + i, &h, 16);
    }
}

int f16c_cpu_supported(void) { return __builtin_cpu_supports("f16c") && __builtin_cpu_supports("avx"); }
