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
// result twice.  Measured on gfx950: a VALU write of an operand needs 2 wait
// states before the swap reads it (the hazard pass cannot see inside an asm
// block, hence the leading s_nop 1); the swapped registers can be read by the
// very next VALU instruction.
//
// v_permlane16_swap(a, b): odd rows of a <-> even rows of b.
//   a' = [a.r0, b.r0, a.r2, b.r2]   b' = [a.r1, b.r1, a.r3, b.r3]
// so a'+b' holds (a.r0+a.r1) in row 0, (b.r0+b.r1) in row 1, (a.r2+a.r3) in
// row 2, (b.r2+b.r3) in row 3: a two-value reduce-scatter over row pairs.
__device__ __forceinline__ float swapadd16(float a, float b) {
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
    return a + b;
}

// v_permlane32_swap(a, b): upper half of a <-> lower half of b.
//   a' = [a.lo, b.lo]   b' = [a.hi, b.hi]
// so a'+b' holds (a.lo+a.hi) in lanes 0-31 and (b.lo+b.hi) in lanes 32-63.
__device__ __forceinline__ float swapadd32(float a, float b) {
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
    return a + b;
}

// Column reduce-scatter of two float4 partials over the 4 DPP rows of a wave
// (D = 64 layout: lane = g*16 + cb holds columns 4*cb..4*cb+3 of row group g).
// On return fq / fk hold the sum over the 4 row groups for column 4*cb + g.
// One asm block: 6 exchanges, 6 adds, and only the wait states that are needed.
__device__ __forceinline__ void colreduce4x2(float4 q, float4 k, float &fq, float &fk) {
    asm volatile(
        "s_nop 1\n\t"
        "v_permlane32_swap_b32 %0, %2\n\t"   // (q.x, q.z)
        "v_permlane32_swap_b32 %1, %3\n\t"   // (q.y, q.w)
        "v_permlane32_swap_b32 %4, %6\n\t"   // (k.x, k.z)
        "v_permlane32_swap_b32 %5, %7\n\t"   // (k.y, k.w)
        "v_add_f32 %0, %0, %2\n\t"           // uq: x over halves (lo) / z (hi)
        "v_add_f32 %1, %1, %3\n\t"           // wq: y / w
        "v_add_f32 %4, %4, %6\n\t"           // uk
        "v_add_f32 %5, %5, %7\n\t"           // wk
        "v_permlane16_swap_b32 %0, %1\n\t"   // %1 was written 2 instructions ago
        "s_nop 0\n\t"
        "v_permlane16_swap_b32 %4, %5\n\t"   // %5: add, swap, nop -> 2 wait states
        "v_add_f32 %0, %0, %1\n\t"
        "v_add_f32 %4, %4, %5"
        : "+v"(q.x), "+v"(q.y), "+v"(q.z), "+v"(q.w), "+v"(k.x), "+v"(k.y), "+v"(k.z), "+v"(k.w));
    fq = q.x;
    fk = k.x;
}

// Four independent exchanges behind one wait-state pad.
__device__ __forceinline__ void swap32x4(float &a0, float &b0, float &a1, float &b1, float &a2,
                                         float &b2, float &a3, float &b3) {
    asm volatile(
        "s_nop 1\n\t"
        "v_permlane32_swap_b32 %0, %1\n\t"
        "v_permlane32_swap_b32 %2, %3\n\t"
        "v_permlane32_swap_b32 %4, %5\n\t"
        "v_permlane32_swap_b32 %6, %7"
        : "+v"(a0), "+v"(b0), "+v"(a1), "+v"(b1), "+v"(a2), "+v"(b2), "+v"(a3), "+v"(b3));
}
__device__ __forceinline__ void swap16x2(float &a0, float &b0, float &a1, float &b1) {
    asm volatile(
        "s_nop 1\n\t"
        "v_permlane16_swap_b32 %0, %1\n\t"
        "v_permlane16_swap_b32 %2, %3"
        : "+v"(a0), "+v"(b0), "+v"(a1), "+v"(b1));
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

// Wave-wide sums of N per-lane values at once (N a multiple of 8).  Two
// reduce-scatter steps over the DPP rows leave N/4 partial sums per lane, which
// are then summed inside each 16-lane row.  On return every lane of DPP row r
// holds, in out[n] for n < N/4, the wave total of v[4*n + 2*(r&1) + (r>>1)].
// Cost: N/2 + N/4 exchanges instead of 2*N for N separate reductions.
template <int N>
__device__ __forceinline__ void wave_reduce_scatter(float (&v)[N], float (&out)[N / 4]) {
    static_assert(N % 8 == 0, "N must be a multiple of 8");
    float h[N / 2];
#pragma unroll
    for (int m = 0; m < N / 2; m += 4) {
        swap32x4(v[2 * m], v[2 * m + 1], v[2 * m + 2], v[2 * m + 3], v[2 * m + 4], v[2 * m + 5],
                 v[2 * m + 6], v[2 * m + 7]);
#pragma unroll
        for (int u = 0; u < 4; u++) h[m + u] = v[2 * (m + u)] + v[2 * (m + u) + 1];
    }
#pragma unroll
    for (int n = 0; n < N / 4; n += 2) {
        swap16x2(h[2 * n], h[2 * n + 1], h[2 * n + 2], h[2 * n + 3]);
        out[n] = h[2 * n] + h[2 * n + 1];
        out[n + 1] = h[2 * n + 2] + h[2 * n + 3];
    }
#pragma unroll
    for (int n = 0; n < N / 4; n++) out[n] = group_allreduce<16>(out[n]);
}

__device__ __forceinline__ float dot4(const float4 &a, const float4 &b) {
    return a.x * b.x + a.y * b.y + a.z * b.z + a.w * b.w;
}

}  // namespace nlh
