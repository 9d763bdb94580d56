// Building blocks of the kernels that run 64x64 products of a chunk on the bf16 matrix
// cores (v_mfma_f32_16x16x32_bf16) with operands staged in LDS.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace nlh {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned short u16;

constexpr int HD = 64;             // head size
constexpr int CW = 64;             // tokens per chunk tile
constexpr int LDB = 72;            // LDS row stride of a bf16 matrix (144 B: 16-byte rows, conflict-free operand reads)
constexpr int BMAT = 64 * LDB;     // elements per bf16 matrix
constexpr int kTileThr = 512;      // 8 waves

__device__ __forceinline__ f32x4 zero4() { return f32x4{0.f, 0.f, 0.f, 0.f}; }
__device__ __forceinline__ float bf2f(u16 h) { return __uint_as_float(((unsigned)h) << 16); }
__device__ __forceinline__ f32x4 mfma32(bf16x8 a, bf16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
// Operand of one 16x16x32 step from a bf16 matrix whose rows run along the contraction:
// lane l supplies row row0 + l%16, contraction indices 32*ks + 8*(l/16) .. +8.  The same
// loader serves A (rows = output rows) and B (rows = output columns).
__device__ __forceinline__ bf16x8 ld_op(const u16 *X, int row0, int ks) {
    const int l = threadIdx.x & 63;
    return *reinterpret_cast<const bf16x8 *>(X + (row0 + (l & 15)) * LDB + 32 * ks + 8 * (l >> 4));
}
// The same operand from a matrix stored the other way round (element (contraction index k, row n) at
// X[k * STRIDE + n]), with no transposed copy: ds_read_b64_tr_b16 works on groups of 16 lanes; when lane s of
// a group addresses the four elements X[k0 + s/4][n0 + 4 (s%4) .. + 3], lane i receives X[k0 .. k0 + 3][n0 + i].
// Two such reads give the eight contraction indices 32*ks + 8*(l/16) .. + 8 of row row0 + l%16.  STRIDE in
// elements, a multiple of 4; conflict-free inside a group when STRIDE / 2 is 8 modulo 16 (48, 80, ..).
template <int STRIDE>
__device__ __forceinline__ bf16x8 ld_op_tr(const u16 *X, int row0, int ks) {
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    typedef short s16x8 __attribute__((ext_vector_type(8)));
    typedef __attribute__((address_space(3))) s16x4 *lds_ptr;
    const int l = threadIdx.x & 63, sl = l & 15;
    const u16 *p = X + (32 * ks + 8 * (l >> 4) + (sl >> 2)) * STRIDE + row0 + 4 * (sl & 3);
    const s16x4 a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)p);
    const s16x4 b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p + 4 * STRIDE));
    const s16x8 ab = __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(bf16x8, ab);
}
// x = hi + lo with hi, lo bf16; both stored as four consecutive elements at off.
__device__ __forceinline__ void split_store(u16 *H, u16 *Lo, int off, f32x4 x) {
    bf16x4 h, lo;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const __bf16 hb = (__bf16)x[i];
        h[i] = hb;
        lo[i] = (__bf16)(x[i] - (float)hb);
    }
    *reinterpret_cast<bf16x4 *>(H + off) = h;
    *reinterpret_cast<bf16x4 *>(Lo + off) = lo;
}
__device__ __forceinline__ float lane_bcast(float x, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), lane));
}

// Gates of token (lane) of a chunk; zero beyond L (eta = 0 without momentum).
struct Gates { float al, th, et; };
template <bool HAS_S>
__device__ __forceinline__ Gates fetch_gates(const float *alpha, const float *theta, const float *eta, size_t tok,
                                             int L) {
    const int t = threadIdx.x & 63;
    Gates g;
    g.al = t < L ? alpha[tok + t] : 0.f;
    g.th = t < L ? theta[tok + t] : 0.f;
    g.et = (HAS_S && t < L) ? eta[tok + t] : 0.f;
    return g;
}

// Workgroup -> (chain, half of its rows) for the chain-resident kernels (grid = 2 * batch).  Workgroups go
// to the 8 XCDs round robin in linear order and each XCD has its own L2: the two halves of a chain read the
// same K, Q and coefficient tables, so they get linear ids 8 apart (same XCD, dispatched together; with more
// workgroups than fit at once they also run in the same round and the second reader hits L2).
__device__ __forceinline__ void chain_half_of_block(int batch, int &chain, int &half) {
    const int id = blockIdx.x;
    if ((batch & 7) == 0) {
        chain = (id >> 4) * 8 + (id & 7);
        half = (id >> 3) & 1;
    } else {
        chain = id % batch;
        half = id / batch;
    }
}

// Store of four consecutive elements as bf16 (round to nearest even).
__device__ __forceinline__ void bf16_store(u16 *X, int off, f32x4 x) {
    bf16x4 h;
#pragma unroll
    for (int i = 0; i < 4; i++) h[i] = (__bf16)x[i];
    *reinterpret_cast<bf16x4 *>(X + off) = h;
}

}  // namespace
}  // namespace nlh
