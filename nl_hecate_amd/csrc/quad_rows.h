// Row-quad layout helpers shared by the kernels that keep a d x d matrix as
// "lane (r, cq) = (tid / 4, tid % 4) holds columns [cq*d/4, (cq+1)*d/4) of row r":
// a matrix-vector product is a per-lane dot plus a sum over the quad; sums over
// rows (column sums) reduce over the 16 lanes of a wave that share cq and then
// across waves through LDS.
#pragma once
#include <hip/hip_runtime.h>

#include "lane_ops.h"

namespace nlh {

constexpr int DPP_ROR4 = 0x124;

// Barrier for data exchanged through LDS only.  __syncthreads() also waits for
// every outstanding global load and store of the wave, which would put the HBM
// round trip of the per-token cache writes and of the prefetched trajectory
// reads on the critical path of each token.
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

__device__ __forceinline__ float quad_allreduce(float x) { return group_allreduce<4>(x); }

// Sum over the 16 lanes of a wave that share (lane % 4): the rows a wave owns.
__device__ __forceinline__ float rows_allreduce(float x) {
    x += dpp_mov<DPP_ROR4>(x);
    x += dpp_mov<DPP_ROR8>(x);
    x = swapadd16(x, x);
    x = swapadd32(x, x);
    return x;
}

// Column sums over the 16 rows of a wave for the CP columns a lane holds.  On
// return the lanes of DPP row rho hold in out[0..CP/4) the sums of the lane's
// columns (CP/2)*(rho>>1) + (CP/4)*(rho&1) + [0, CP/4).
template <int CP>
__device__ __forceinline__ void rows_reduce_scatter(const float (&v)[CP], float (&out)[CP / 4]) {
    float h[CP / 2];
#pragma unroll
    for (int i = 0; i < CP / 2; i++) h[i] = swapadd32(v[i], v[i + CP / 2]);
#pragma unroll
    for (int i = 0; i < CP / 4; i++) {
        float x = swapadd16(h[i], h[i + CP / 4]);
        x += dpp_mov<DPP_ROR4>(x);
        x += dpp_mov<DPP_ROR8>(x);
        out[i] = x;
    }
}

template <int CP>
__device__ __forceinline__ void lds_read(float (&dst)[CP], const float *src) {
#pragma unroll
    for (int i = 0; i < CP; i += 4) {
        const float4 t = *reinterpret_cast<const float4 *>(src + i);
        dst[i] = t.x; dst[i + 1] = t.y; dst[i + 2] = t.z; dst[i + 3] = t.w;
    }
}
template <int CP>
__device__ __forceinline__ void vec_store(float *dst, const float (&src)[CP]) {
#pragma unroll
    for (int i = 0; i < CP; i += 4)
        *reinterpret_cast<float4 *>(dst + i) = make_float4(src[i], src[i + 1], src[i + 2], src[i + 3]);
}
template <int CP>
__device__ __forceinline__ float dotn(const float (&a)[CP], const float (&b)[CP]) {
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < CP; i++) s = fmaf(a[i], b[i], s);
    return s;
}

}  // namespace nlh
