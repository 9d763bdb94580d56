// Building blocks of the fp32 matrix-core kernels (v_mfma_f32_16x16x4_f32) that work on 64 x 64 tiles held in
// LDS: staging of global tiles, a wave's 16 x 32 output strip, products with operands given as functions of
// (row, contraction index) so that any orientation, scaling or masking of an LDS matrix can feed a product.
// Workgroups of 512 threads (8 waves, two per SIMD).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "rule_common.h"

namespace nlh {
namespace mmt {

using f32x4 = __attribute__((ext_vector_type(4))) float;

constexpr int CW = 64;          // tokens per chunk tile
constexpr int HD = 64;          // head size
constexpr int LDM = 65;         // LDS row stride in floats (odd: conflict-free rows and columns)
constexpr int MAT = 64 * LDM;   // floats per 64x64 LDS matrix
constexpr int kThr = 512;       // 8 waves (two per SIMD), one 16x32 output strip each

__device__ __forceinline__ float to_f32(float x) { return x; }
__device__ __forceinline__ float to_f32(uint16_t u) { return __uint_as_float((uint32_t)u << 16); }

// Staging of a row-major [nrows <= 64][64] global tile into LDS in two halves, so that the
// loads of every tile of a phase are in flight together: fetch() issues the global loads
// into registers (rows >= nrows read as zero), commit() converts and stores to LDS.
template <class T> struct Tile;
template <> struct Tile<float> { float4 x[2]; };
template <> struct Tile<uint16_t> { uint2 x[2]; };

// The helpers below take the thread (or lane) index as an optional last argument.  A kernel that loops over tasks
// passes a copy that is opaque to the compiler per task: otherwise every LDS address of every phase is loop-invariant,
// gets hoisted out of the loop and lives in a register for its whole length.
template <class T>
__device__ __forceinline__ void fetch(Tile<T> &r, const T *src, int nrows, int tid = threadIdx.x) {
#pragma unroll
    for (int it = 0; it < 2; it++) {
        const int e = (it * kThr + tid) * 4, rr = e >> 6, cc = e & 63;
        if constexpr (sizeof(T) == 4)
            r.x[it] = rr < nrows ? *reinterpret_cast<const float4 *>(src + rr * 64 + cc) : make_float4(0, 0, 0, 0);
        else
            r.x[it] = rr < nrows ? *reinterpret_cast<const uint2 *>(src + rr * 64 + cc) : make_uint2(0, 0);
    }
}
template <class T>
__device__ __forceinline__ void commit(float *dst, const Tile<T> &r, int tid = threadIdx.x) {
#pragma unroll
    for (int it = 0; it < 2; it++) {
        const int e = (it * kThr + tid) * 4, rr = e >> 6, cc = e & 63;
        float *p = dst + rr * LDM + cc;
        if constexpr (sizeof(T) == 4) {
            p[0] = r.x[it].x; p[1] = r.x[it].y; p[2] = r.x[it].z; p[3] = r.x[it].w;
        } else {
            p[0] = __uint_as_float(r.x[it].x << 16); p[1] = __uint_as_float(r.x[it].x & 0xffff0000u);
            p[2] = __uint_as_float(r.x[it].y << 16); p[3] = __uint_as_float(r.x[it].y & 0xffff0000u);
        }
    }
}
template <class T>
__device__ __forceinline__ void stage(float *dst, const T *src, int nrows) {
    Tile<T> r;
    fetch(r, src, nrows);
    commit(dst, r);
}

// dot product of two staged tiles' registers (this thread's eight elements of each)
__device__ __forceinline__ float tile_dot(const Tile<float> &a, const Tile<float> &b) {
    float x = 0.f;
#pragma unroll
    for (int it = 0; it < 2; it++)
        x += a.x[it].x * b.x[it].x + a.x[it].y * b.x[it].y + a.x[it].z * b.x[it].z + a.x[it].w * b.x[it].w;
    return x;
}

// the same against a tile that this thread committed to LDS earlier (its own eight elements: no barrier needed)
__device__ __forceinline__ float tile_dot_lds(const float *src, const Tile<float> &b, int tid = threadIdx.x) {
    float x = 0.f;
#pragma unroll
    for (int it = 0; it < 2; it++) {
        const int e = (it * kThr + tid) * 4, rr = e >> 6, cc = e & 63;
        const float *p = src + rr * LDM + cc;
        x += p[0] * b.x[it].x + p[1] * b.x[it].y + p[2] * b.x[it].z + p[3] * b.x[it].w;
    }
    return x;
}

// Output strip of one wave: 16 rows x 32 columns = two 16x16 accumulator tiles side by side.
// With 8 waves a 64x64 product is 8 strips; two waves share a SIMD, so one wave's LDS reads,
// epilogue arithmetic and stores overlap the other's matrix-core work.
struct Strip { f32x4 t[2]; };
__device__ __forceinline__ Strip zero_strip() {
    Strip z;
#pragma unroll
    for (int i = 0; i < 4; i++) { z.t[0][i] = 0.f; z.t[1][i] = 0.f; }
    return z;
}
// acc += sum_{k<64} a(m,k) b(k,n), m in [0,16), n in [0,32).
// Operand layout of v_mfma_f32_16x16x4_f32: lane l supplies A[l%16][j] and B[j][l%16] with j = l/16 of the step's four
// contraction indices.  Which four indices a step takes is free (a sum), so lane group l/16 walks through its own
// block of 16 indices: with the odd row stride LDM an operand element X[row][col] sits in bank (row + col) % banks, and
// the lanes of one read then differ by l%16 + 16 (l/16), i.e. fall on different banks whichever way the matrix is
// read (the assignment 4 i + l/16 put up to four lanes on a bank).
// Sixteen k-steps in four groups; the operands of group g+1 are read while group g runs.
template <class FA, class FB>
__device__ __forceinline__ void mma(Strip &acc, FA a, FB b, int l = threadIdx.x & 63) {
    const int r = l & 15, kb = 16 * (l >> 4);
    float av[2][4], b0[2][4], b1[2][4];
#pragma unroll
    for (int i = 0; i < 4; i++) { av[0][i] = a(r, kb + i); b0[0][i] = b(kb + i, r); b1[0][i] = b(kb + i, 16 + r); }
#pragma unroll
    for (int g = 0; g < 4; g++) {
        if (g < 3) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int kk = kb + 4 * (g + 1) + i;
                av[(g + 1) & 1][i] = a(r, kk); b0[(g + 1) & 1][i] = b(kk, r); b1[(g + 1) & 1][i] = b(kk, 16 + r);
            }
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
            acc.t[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[g & 1][i], b0[g & 1][i], acc.t[0], 0, 0, 0);
            acc.t[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[g & 1][i], b1[g & 1][i], acc.t[1], 0, 0, 0);
        }
    }
}
// The same over the contraction indices 32 p0 .. 32 p1 - 1 only (wave-uniform bounds): triangular operands.  Lane
// group j = l/16 takes the indices 32 p + 16 (j % 2) + 8 (j / 2) + 0..7 of a block of 32: the two groups of a
// half-wave stay 16 banks apart.
template <class FA, class FB>
__device__ __forceinline__ void mma_range(Strip &acc, FA a, FB b, int p0, int p1, int l = threadIdx.x & 63) {
    const int r = l & 15, kq = l >> 4, kb = 16 * (kq & 1) + 8 * (kq >> 1);
    for (int p = p0; p < p1; p++) {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            float av[4], b0[4], b1[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int kk = 32 * p + kb + 4 * h + i;
                av[i] = a(r, kk); b0[i] = b(kk, r); b1[i] = b(kk, 16 + r);
            }
#pragma unroll
            for (int i = 0; i < 4; i++) {
                acc.t[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[i], b0[i], acc.t[0], 0, 0, 0);
                acc.t[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[i], b1[i], acc.t[1], 0, 0, 0);
            }
        }
    }
}
// One 16x16 tile, contraction over the 16 indices k0 .. k0 + 15 only (block-diagonal operands):
// acc += sum_{k0 <= k < k0+16} a(m,k) b(k,n), m, n in [0,16).
template <class FA, class FB>
__device__ __forceinline__ void mma_tile16(f32x4 &acc, FA a, FB b, int k0, int l = threadIdx.x & 63) {
    const int r = l & 15, kq = l >> 4;
    float av[4], bv[4];
#pragma unroll
    for (int i = 0; i < 4; i++) { av[i] = a(r, k0 + 4 * i + kq); bv[i] = b(k0 + 4 * i + kq, r); }
#pragma unroll
    for (int i = 0; i < 4; i++) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(av[i], bv[i], acc, 0, 0, 0);
}
// Element i of tile tl of lane l is C[4*(l/16) + i][16*tl + l%16] of the strip.
template <class F>
__device__ __forceinline__ void for_c(Strip &acc, F f, int l = threadIdx.x & 63) {
#pragma unroll
    for (int tl = 0; tl < 2; tl++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float x = acc.t[tl][i];
            f(4 * (l >> 4) + i, 16 * tl + (l & 15), x);
            acc.t[tl][i] = x;
        }
}
// Row sums of a strip: afterwards t[0][i] of every lane holds the sum over the 32 columns of
// strip row 4*(l/16) + i.
__device__ __forceinline__ void strip_row_sums(Strip &x) {
#pragma unroll
    for (int i = 0; i < 4; i++) x.t[0][i] = group_allreduce<16>(x.t[0][i] + x.t[1][i]);
}
// lanes that publish the row sums (one per 16-lane group), and the strip rows they hold
__device__ __forceinline__ bool row_writer(int l = threadIdx.x & 63) { return (l & 15) == 0; }
__device__ __forceinline__ int row_of(int i, int l = threadIdx.x & 63) { return 4 * (l >> 4) + i; }

}  // namespace mmt
}  // namespace nlh
