// Reductions across the four 16-lane groups of a wave64, for kernels whose lane (c = lane % 16,
// g = lane / 16) keeps one value per (c, g) and needs the combination over g in every lane.
#pragma once

#include <hip/hip_runtime.h>

namespace bkv {

// Reductions over the four lanes {c, c + 16, c + 32, c + 48}, result in every one of them, on the
// VALU: v_permlane32_swap exchanges the upper half of its first register with the lower half of
// its second, v_permlane16_swap the odd rows of the first with the even rows of the second, so
// with two copies of x the two registers then hold x[l] and x[l ^ 32] (x[l ^ 16]) side by side.
// Written as asm with both registers as in/out operands: the compiler's two-result builtin for
// these instructions hands back its first result twice.  The s_nop covers the wait states the
// swap needs after a VALU write of its operands.
struct LanePair {
    float a, b;
};
__device__ __forceinline__ LanePair swap_halves(float x) {
    LanePair p{x, x};
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(p.a), "+v"(p.b));
    return p;
}
__device__ __forceinline__ LanePair swap_rows(float x) {
    LanePair p{x, x};
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(p.a), "+v"(p.b));
    return p;
}
__device__ __forceinline__ float max_over_lane_groups(float x) {
    const LanePair p = swap_halves(x);
    const LanePair q = swap_rows(fmaxf(p.a, p.b));
    return fmaxf(q.a, q.b);
}
__device__ __forceinline__ float sum_over_lane_groups(float x) {
    const LanePair p = swap_halves(x);
    const LanePair q = swap_rows(p.a + p.b);
    return q.a + q.b;
}

// x of the lane a DPP control names (row_ror:4 = 0x124, row_ror:8 = 0x128, quad_perm broadcasts
// 0x00 / 0x55 / 0xAA / 0xFF), within the lane's row of 16
template <int CTRL>
__device__ __forceinline__ float dpp_mov(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, false));
}

}  // namespace bkv
