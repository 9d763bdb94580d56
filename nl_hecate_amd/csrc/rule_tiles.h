// Token-tile staging shared by the memory-rule kernels.
//
// A workgroup of 256 threads streams k/v/q (and dY for backward) through LDS in
// tiles of TB tokens.  Global loads are 16-byte and fully coalesced (a token row
// of D floats is contiguous); the next tile is fetched into registers while the
// current one is being consumed, then written to the other LDS buffer, so one
// barrier per tile is the only workgroup-wide synchronisation of the
// uncoupled kernels.
#pragma once
#include <hip/hip_runtime.h>

namespace nlh {

constexpr int kThreads = 256;  // 4 wavefronts
constexpr int kWaves = 4;

// Registers that hold one thread's share of a [TB, D] float tile.
template <int D, int TB>
struct TileRegs {
    static constexpr int N4 = TB * D / 4;                     // float4 elements in the tile
    static constexpr int NV = (N4 + kThreads - 1) / kThreads; // per thread
    float4 v[NV];

    // Tokens t0 .. t0+TB-1 of a [*, D] tensor; tokens outside [lo, hi) read as 0.
    __device__ __forceinline__ void load(const float *__restrict__ base, int t0, int lo, int hi,
                                         int tid) {
#pragma unroll
        for (int i = 0; i < NV; i++) {
            int idx = tid + i * kThreads;
            int tt = idx / (D / 4), c4 = idx % (D / 4);
            int t = t0 + tt;
            float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
            if (idx < N4 && t >= lo && t < hi)
                z = *reinterpret_cast<const float4 *>(base + (size_t)t * D + c4 * 4);
            v[i] = z;
        }
    }
    __device__ __forceinline__ void store_lds(float *tile, int tid) const {
#pragma unroll
        for (int i = 0; i < NV; i++) {
            int idx = tid + i * kThreads;
            if (idx < N4) reinterpret_cast<float4 *>(tile)[idx] = v[i];
        }
    }
};

// Per-token gates of a tile: thread j < TB of wave w loads gate w of token t0+j.
template <int TB>
struct GateRegs {
    float g;
    __device__ __forceinline__ void load(const float *__restrict__ alpha,
                                         const float *__restrict__ theta,
                                         const float *__restrict__ eta, int t0, int lo, int hi,
                                         int tid) {
        int w = tid >> 6, j = tid & 63;
        int t = t0 + j;
        g = 0.f;
        if (j < TB && t >= lo && t < hi) {
            if (w == 0) g = alpha[t];
            else if (w == 1) g = theta[t];
            else if (w == 2 && eta) g = eta[t];
        }
    }
    // gates laid out [3][TB]
    __device__ __forceinline__ void store_lds(float *gates, int tid) const {
        int w = tid >> 6, j = tid & 63;
        if (j < TB && w < 3) gates[w * TB + j] = g;
    }
};

}  // namespace nlh
