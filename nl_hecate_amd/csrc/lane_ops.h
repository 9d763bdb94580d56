// Cross-lane primitives for wave64 on gfx950 (CDNA4).
//
// A wavefront is 4 DPP rows of 16 lanes.  Inside a row, sums use DPP-modified
// adds (no LDS, no extra instruction); across rows they use the gfx950
// v_permlane16_swap / v_permlane32_swap instructions, which exchange whole
// rows between two registers in one VALU op.
#pragma once
#include <hip/hip_runtime.h>

namespace nlh {

template <int CTRL>
__device__ __forceinline__ float dpp_mov(float x) {
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xF, 0xF, true));
}

constexpr int DPP_XOR1 = 0xB1;         // quad_perm [1,0,3,2]
constexpr int DPP_XOR2 = 0x4E;         // quad_perm [2,3,0,1]
constexpr int DPP_HALF_MIRROR = 0x141; // lane i <-> 7-i within 8
constexpr int DPP_MIRROR = 0x140;      // lane i <-> 15-i within 16
constexpr int DPP_ROR8 = 0x128;        // rotate right by 8 within 16 (== xor 8)

// The two row-exchange instructions are issued through inline asm: both
// registers are read and written, and the compiler's builtin returns the first
// result twice.  The s_nop pads cover the VALU-write -> permlane-read and
// permlane-write -> VALU-read wait states, which the hazard pass does not see
// inside an asm block.
//
// v_permlane16_swap(a, b): odd rows of a <-> even rows of b.
//   a' = [a.r0, b.r0, a.r2, b.r2]   b' = [a.r1, b.r1, a.r3, b.r3]
// so a'+b' holds (a.r0+a.r1) in row 0, (b.r0+b.r1) in row 1, (a.r2+a.r3) in
// row 2, (b.r2+b.r3) in row 3: a two-value reduce-scatter over row pairs.
__device__ __forceinline__ float swapadd16(float a, float b) {
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    return a + b;
}

// v_permlane32_swap(a, b): upper half of a <-> lower half of b.
//   a' = [a.lo, b.lo]   b' = [a.hi, b.hi]
// so a'+b' holds (a.lo+a.hi) in lanes 0-31 and (b.lo+b.hi) in lanes 32-63.
__device__ __forceinline__ float swapadd32(float a, float b) {
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
    return a + b;
}

// Sum over an aligned group of G consecutive lanes; every lane of the group
// receives the sum.  G is a power of two in [1, 64].
template <int G>
__device__ __forceinline__ float group_allreduce(float x) {
    if constexpr (G >= 2) x += dpp_mov<DPP_XOR1>(x);
    if constexpr (G >= 4) x += dpp_mov<DPP_XOR2>(x);
    if constexpr (G >= 8) x += dpp_mov<DPP_HALF_MIRROR>(x);  // x is quad-uniform here
    if constexpr (G >= 16) x += dpp_mov<DPP_MIRROR>(x);      // x is 8-uniform here
    if constexpr (G >= 32) x = swapadd16(x, x);
    if constexpr (G >= 64) x = swapadd32(x, x);
    return x;
}

// x + (value of x in lane ^ MASK), for values that differ between lanes.
template <int MASK>
__device__ __forceinline__ float xor_add(float x) {
    if constexpr (MASK == 1) return x + dpp_mov<DPP_XOR1>(x);
    else if constexpr (MASK == 2) return x + dpp_mov<DPP_XOR2>(x);
    else if constexpr (MASK == 8) return x + dpp_mov<DPP_ROR8>(x);
    else if constexpr (MASK == 16) return swapadd16(x, x);
    else if constexpr (MASK == 32) return swapadd32(x, x);
    else return x + __shfl_xor(x, MASK, 64);
}

// Sum over the lanes that share (lane % LPR): the "column" reduction across
// the 64/LPR row-groups of a wave.  Every lane receives the sum.
template <int LPR>
__device__ __forceinline__ float stride_allreduce(float x) {
    if constexpr (LPR <= 1) x = xor_add<1>(x);
    if constexpr (LPR <= 2) x = xor_add<2>(x);
    if constexpr (LPR <= 4) x = xor_add<4>(x);
    if constexpr (LPR <= 8) x = xor_add<8>(x);
    if constexpr (LPR <= 16) x = xor_add<16>(x);
    if constexpr (LPR <= 32) x = xor_add<32>(x);
    return x;
}

__device__ __forceinline__ float wave_allreduce(float x) { return group_allreduce<64>(x); }

__device__ __forceinline__ float dot4(const float4 &a, const float4 &b) {
    return a.x * b.x + a.y * b.y + a.z * b.z + a.w * b.w;
}

}  // namespace nlh
