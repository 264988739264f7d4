// Register-level decoding of int8 codes for the kernels that feed them to the matrix cores.
#pragma once

#include <hip/hip_runtime.h>

namespace bkv {

typedef _Float16 h2m __attribute__((ext_vector_type(2)));

// four int8 codes (one dword) -> four exact f16 values: 0x6400 | (code ^ 0x80) is 1024 + (code + 128)
__device__ __forceinline__ void codes_to_f16(unsigned w, h2m& lo, h2m& hi) {
    const unsigned u = w ^ 0x80808080u;
    const h2m bias = h2m{(_Float16)1152.0f, (_Float16)1152.0f};
    lo = __builtin_bit_cast(h2m, __builtin_amdgcn_perm(0x64646464u, u, 0x04010400u)) - bias;
    hi = __builtin_bit_cast(h2m, __builtin_amdgcn_perm(0x64646464u, u, 0x04030402u)) - bias;
}
// the same for codes that already carry the ^ 0x80 bias
__device__ __forceinline__ void biased_to_f16(unsigned u, h2m& lo, h2m& hi) {
    const h2m bias = h2m{(_Float16)1152.0f, (_Float16)1152.0f};
    lo = __builtin_bit_cast(h2m, __builtin_amdgcn_perm(0x64646464u, u, 0x04010400u)) - bias;
    hi = __builtin_bit_cast(h2m, __builtin_amdgcn_perm(0x64646464u, u, 0x04030402u)) - bias;
}
// 4 x 4 byte transpose: t[j] = { w[0].byte j, w[1].byte j, w[2].byte j, w[3].byte j }
__device__ __forceinline__ void transpose4x4_bytes(const unsigned (&w)[4], unsigned (&t)[4]) {
    const unsigned a_lo = __builtin_amdgcn_perm(w[1], w[0], 0x05010400u);  // w0.0 w1.0 w0.1 w1.1
    const unsigned a_hi = __builtin_amdgcn_perm(w[1], w[0], 0x07030602u);  // w0.2 w1.2 w0.3 w1.3
    const unsigned b_lo = __builtin_amdgcn_perm(w[3], w[2], 0x05010400u);
    const unsigned b_hi = __builtin_amdgcn_perm(w[3], w[2], 0x07030602u);
    t[0] = __builtin_amdgcn_perm(b_lo, a_lo, 0x05040100u);
    t[1] = __builtin_amdgcn_perm(b_lo, a_lo, 0x07060302u);
    t[2] = __builtin_amdgcn_perm(b_hi, a_hi, 0x05040100u);
    t[3] = __builtin_amdgcn_perm(b_hi, a_hi, 0x07060302u);
}

// The exact two-term f16 form of code * scale for a scale given as s_hi + s_lo: hi = f16(code *
// s_hi), its remainder (at most 7 significant bits, a representable f16 number) plus code * s_lo
// in lo.
__device__ __forceinline__ void scaled_hi_lo(h2m code, h2m s_hi, h2m s_lo, h2m& hi, h2m& lo) {
    hi = code * s_hi;
    lo = __builtin_elementwise_fma(code, s_lo, __builtin_elementwise_fma(code, s_hi, -hi));
}

}  // namespace bkv
