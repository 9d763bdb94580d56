// What this box sustains, measured with kernels of the simplest possible shape, so that a kernel's roofline
// fraction can be read against an achieved figure as well as against the data-sheet one:
//   * streaming copies at a stated read : write mix (16-byte accesses, grid-stride, nothing else);
//   * the matrix cores' issue peak for the two instructions the library uses
//     (v_mfma_f32_16x16x32_bf16, v_mfma_f32_16x16x4_f32): every wave keeps eight independent accumulator
//     tiles going from operands that stay in registers, no memory traffic inside the loop.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/nl_hecate_ffi.h"
#include "runtime.h"

namespace nlh {
namespace {

typedef __bf16 pbf16x8 __attribute__((ext_vector_type(8)));
typedef float pf32x4 __attribute__((ext_vector_type(4)));

// out_w[i] = sum of in_r[i] over `reads` input streams, for w < writes: reads + writes streams of n4 float4 each
__global__ __launch_bounds__(256) void stream_mix_kernel(const float4 *__restrict__ in, float4 *__restrict__ out, long long n4,
                                                         int reads, int writes) {
    const long long stride = (long long)gridDim.x * blockDim.x;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride) {
        float4 s = in[i];
        for (int r = 1; r < reads; r++) {
            const float4 x = in[r * n4 + i];
            s.x += x.x; s.y += x.y; s.z += x.z; s.w += x.w;
        }
        for (int w = 0; w < writes; w++) out[w * n4 + i] = s;
    }
}

typedef float pf32x16 __attribute__((ext_vector_type(16)));
// the 32 x 32 x 16 shape: four independent accumulator tiles of 16 registers
__global__ __launch_bounds__(256) void mfma_peak32_kernel(float *out, int iters) {
    pf32x16 acc[4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 16; j++) acc[i][j] = 0.f;
    const float seed = (float)(threadIdx.x & 7) * 0.125f;
    pbf16x8 a, b;
#pragma unroll
    for (int i = 0; i < 8; i++) { a[i] = (__bf16)(seed + i * 0.01f); b[i] = (__bf16)(0.5f - i * 0.02f); }
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int i = 0; i < 4; i++) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[i], 0, 0, 0);
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 16; j++) s += acc[i][j];
    out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = s;
}

template <bool BF16>
__global__ __launch_bounds__(256) void mfma_peak_kernel(float *out, int iters) {
    pf32x4 acc[8];
#pragma unroll
    for (int i = 0; i < 8; i++) acc[i] = pf32x4{0.f, 0.f, 0.f, 0.f};
    const float seed = (float)(threadIdx.x & 7) * 0.125f;
    if (BF16) {
        pbf16x8 a, b;
#pragma unroll
        for (int i = 0; i < 8; i++) { a[i] = (__bf16)(seed + i * 0.01f); b[i] = (__bf16)(0.5f - i * 0.02f); }
        for (int it = 0; it < iters; it++) {
#pragma unroll
            for (int i = 0; i < 8; i++) acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[i], 0, 0, 0);
        }
    } else {
        const float a = seed, b = 0.5f - seed;
        for (int it = 0; it < iters; it++) {
#pragma unroll
            for (int i = 0; i < 8; i++) acc[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, acc[i], 0, 0, 0);
        }
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++) s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
    out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = s;
}

}  // namespace
}  // namespace nlh

using namespace nlh;

extern "C" {

int nlh_probe_stream_rocm(const float *in, float *out, long long n, int reads, int writes) {
    if (n <= 0 || n % 4 || reads < 1 || writes < 1 || (((uintptr_t)in) & 15) || (((uintptr_t)out) & 15)) return -1;
    KernelTimer kt("stream_mix_kernel");
    hipLaunchKernelGGL(stream_mix_kernel, dim3(compute_units() * 8), dim3(256), 0, stream(), reinterpret_cast<const float4 *>(in),
                       reinterpret_cast<float4 *>(out), n / 4, reads, writes);
    return hipGetLastError() == hipSuccess ? 0 : -2;
}

// kind 0: v_mfma_f32_16x16x32_bf16 (16384 flop per instruction and wave), kind 1: v_mfma_f32_16x16x4_f32 (2048),
// kind 2: v_mfma_f32_32x32x16_bf16 (32768; four instructions per iteration instead of eight).
// Launches waves_per_simd * 4 waves on every compute unit, each issuing 8 * iters instructions; out needs
// compute_units * waves_per_simd * 256 floats.  Returns the number of matrix instructions issued per wave.
int nlh_probe_mfma_rocm(int kind, int iters, int waves_per_simd, float *out) {
    if (iters < 1 || waves_per_simd < 1 || waves_per_simd > 8 || kind < 0 || kind > 2) return -1;
    KernelTimer kt(kind == 0 ? "mfma_peak_kernel_bf16" : (kind == 1 ? "mfma_peak_kernel_f32" : "mfma_peak32_kernel_bf16"));
    const dim3 grid(compute_units() * waves_per_simd), block(256);
    if (kind == 0) hipLaunchKernelGGL(mfma_peak_kernel<true>, grid, block, 0, stream(), out, iters);
    else if (kind == 1) hipLaunchKernelGGL(mfma_peak_kernel<false>, grid, block, 0, stream(), out, iters);
    else hipLaunchKernelGGL(mfma_peak32_kernel, grid, block, 0, stream(), out, iters);
    return hipGetLastError() == hipSuccess ? (kind == 2 ? 4 : 8) * iters : -2;
}

}  // extern "C"
