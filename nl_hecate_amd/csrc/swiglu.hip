// SwiGLU MLP, device-to-device: Y = (silu(X Wg^T) * (X Wu^T)) Wd^T and its backward.
// Contracts of core/kernels/swiglu_forward.cu:275-355 and swiglu_backward.cu:380-510
// (core/src/cuda_ffi.rs:925-962): all pointers are device memory, the four activation buffers
// (gate, up, fused, sigmoid cache) are written by the forward and read by the backward, the output
// gradients are written fresh.  The five plain GEMMs of each direction go to rocBLAS on the library's
// stream (column-major calls on the row-major buffers, as the reference does with cuBLAS); the gating
// and its derivative are streaming kernels.  No allocation per call: the three intermediate gradient
// buffers of the backward live in the scratch arena.
#include <hip/hip_runtime.h>
#include <limits.h>
#include <rocblas/rocblas.h>

#include "../../include/nl_hecate_ffi.h"
#include "runtime.h"

namespace nlh {
namespace {

constexpr int kThreads = 256;

inline int blocks_for(size_t n) {
    const size_t b = (n + kThreads - 1) / kThreads;
    return (int)(b < 1 ? 1 : (b > 2048 ? 2048 : b));
}

// swiglu_forward.cu:144-158
__global__ void swiglu_fuse_kernel(const float *__restrict__ gate, const float *__restrict__ up,
                                   float *__restrict__ fused, float *__restrict__ gate_cache, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        const float g = gate[i];
        const float sig = 1.0f / (1.0f + expf(-g));
        gate_cache[i] = sig;
        fused[i] = g * sig * up[i];
    }
}

// swiglu_backward.cu:174-197
__global__ void swiglu_fuse_backward_kernel(const float *__restrict__ d_fused, const float *__restrict__ gate,
                                            const float *__restrict__ up, const float *__restrict__ gate_cache,
                                            float *__restrict__ d_gate, float *__restrict__ d_up, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        const float df = d_fused[i], g = gate[i], sig = gate_cache[i], u = up[i];
        d_gate[i] = df * u * (sig * (1.0f + g * (1.0f - sig)));
        d_up[i] = df * g * sig;
    }
}

rocblas_handle blas() {
    static rocblas_handle h = nullptr;
    if (!h && rocblas_create_handle(&h) != rocblas_status_success) {
        h = nullptr;
        fail("swiglu: rocblas_create_handle failed.");
        return nullptr;
    }
    if (rocblas_set_stream(h, stream()) != rocblas_status_success) {
        fail("swiglu: rocblas_set_stream failed.");
        return nullptr;
    }
    return h;
}

// C (m x n, column-major, ldc) = op(A) op(B) + beta C
bool gemm(const char *what, rocblas_operation ta, rocblas_operation tb, int m, int n, int k, const float *A, int lda,
          const float *B, int ldb, float beta, float *C, int ldc) {
    rocblas_handle h = blas();
    if (!h) return false;
    const float one = 1.0f;
    const rocblas_status st = rocblas_sgemm(h, ta, tb, m, n, k, &one, A, lda, B, ldb, &beta, C, ldc);
    if (st != rocblas_status_success) {
        fail("swiglu: rocblas_sgemm (%s) failed with status %d.", what, (int)st);
        return false;
    }
    return true;
}

bool dims_ok(const char *fn, int seq_len, int d_model, int intermediate) {
    if (seq_len <= 0 || d_model <= 0 || intermediate <= 0) {
        fail("%s: invalid dims: seq_len=%d d_model=%d intermediate=%d", fn, seq_len, d_model, intermediate);
        return false;
    }
    if ((size_t)seq_len * intermediate > (size_t)INT_MAX) {
        fail("%s: seq_len * intermediate = %zu exceeds the 32-bit element count of the contract.", fn,
             (size_t)seq_len * intermediate);
        return false;
    }
    return true;
}

}  // namespace
}  // namespace nlh

using namespace nlh;

extern "C" {

void swiglu_forward_f32_cuda_dd(const float *x, const float *gate_proj, const float *up_proj, const float *down_proj,
                                float *y, float *gate_buf, float *up_buf, float *fused_buf, float *cache_buf,
                                int seq_len, int d_model, int intermediate) {
    if (!dims_ok("swiglu_forward_f32_cuda_dd", seq_len, d_model, intermediate)) return;
    const rocblas_operation N = rocblas_operation_none, T = rocblas_operation_transpose;
    const size_t n = (size_t)seq_len * intermediate;
    // gate = X Wg^T, up = X Wu^T  (row-major [seq, inter] = column-major [inter, seq])
    if (!gemm("gate", T, N, intermediate, seq_len, d_model, gate_proj, d_model, x, d_model, 0.f, gate_buf, intermediate)) return;
    if (!gemm("up", T, N, intermediate, seq_len, d_model, up_proj, d_model, x, d_model, 0.f, up_buf, intermediate)) return;
    hipLaunchKernelGGL(swiglu_fuse_kernel, dim3(blocks_for(n)), dim3(kThreads), 0, stream(), gate_buf, up_buf, fused_buf,
                       cache_buf, n);
    check_launch("swiglu_fuse_kernel");
    // Y = fused Wd^T
    gemm("down", T, N, d_model, seq_len, intermediate, down_proj, intermediate, fused_buf, intermediate, 0.f, y, d_model);
}

void swiglu_backward_f32_cuda_dd(const float *d_y, const float *x, const float *gate_proj, const float *up_proj,
                                 const float *down_proj, const float *fused_buf, const float *gate_buf,
                                 const float *up_buf, const float *cache_buf, float *d_x, float *d_gate_proj,
                                 float *d_up_proj, float *d_down_proj, int seq_len, int d_model, int intermediate) {
    const ErrorScope es;
    if (!dims_ok("swiglu_backward_f32_cuda_dd", seq_len, d_model, intermediate)) return;
    const rocblas_operation N = rocblas_operation_none, T = rocblas_operation_transpose;
    const size_t n = (size_t)seq_len * intermediate;
    float *d_fused = scratch(6, n * sizeof(float));
    float *d_gate = scratch(7, n * sizeof(float));
    float *d_up = scratch(8, n * sizeof(float));
    if (es.failed()) return;
    // d_fused = dY Wd;  d_Wd = dY^T fused
    if (!gemm("d_fused", N, N, intermediate, seq_len, d_model, down_proj, intermediate, d_y, d_model, 0.f, d_fused, intermediate)) return;
    if (!gemm("d_down_proj", N, T, intermediate, d_model, seq_len, fused_buf, intermediate, d_y, d_model, 0.f, d_down_proj, intermediate)) return;
    hipLaunchKernelGGL(swiglu_fuse_backward_kernel, dim3(blocks_for(n)), dim3(kThreads), 0, stream(), d_fused, gate_buf,
                       up_buf, cache_buf, d_gate, d_up, n);
    check_launch("swiglu_fuse_backward_kernel");
    // d_Wg = d_gate^T X;  d_Wu = d_up^T X;  dX = d_gate Wg + d_up Wu
    if (!gemm("d_gate_proj", N, T, d_model, intermediate, seq_len, x, d_model, d_gate, intermediate, 0.f, d_gate_proj, d_model)) return;
    if (!gemm("d_up_proj", N, T, d_model, intermediate, seq_len, x, d_model, d_up, intermediate, 0.f, d_up_proj, d_model)) return;
    if (!gemm("d_x (gate)", N, N, d_model, seq_len, intermediate, gate_proj, d_model, d_gate, intermediate, 0.f, d_x, d_model)) return;
    gemm("d_x (up)", N, N, d_model, seq_len, intermediate, up_proj, d_model, d_up, intermediate, 1.f, d_x, d_model);
}

}  // extern "C"
