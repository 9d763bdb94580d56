// AdamW update and the gradient-norm / clipping pipeline.
//
// All HBM-bound: AdamW moves 28 bytes per parameter (read w, g, m, v; write
// w, m, v).  Kernels use 16-byte accesses and a grid of a few workgroups per
// CU.  The reference launches one kernel per parameter tensor
// (core/src/gpu_optimizer.rs:376); the *_multi_rocm entry points take every
// tensor of a step in one launch, because at d=512 a tensor is at most 1 MB
// and 40-odd launches cost more than the memory traffic.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdio.h>

#include "../../include/nl_hecate_ffi.h"
#include "lane_ops.h"
#include "optim_steps.h"
#include "runtime.h"

namespace nlh {

constexpr int kOptThreads = 256;

__device__ __forceinline__ void adamw_one(float &w, float g, float &m, float &v, float lr, float b1,
                                          float b2, float eps, float bc1_inv, float bc2_inv, float wd) {
    // core/kernels/adamw.cu:44-61
    const float mi = b1 * m + (1.0f - b1) * g;
    const float vi = b2 * v + (1.0f - b2) * g * g;
    m = mi;
    v = vi;
    const float m_hat = mi * bc1_inv, v_hat = vi * bc2_inv;
    w -= lr * (m_hat / (sqrtf(v_hat) + eps) + wd * w);
}

struct AdamwHyper { float lr, b1, b2, eps, wd; };

// SCALE: the gradient is first multiplied by *scale_ptr when that is below 1 (the clip factor, still on the
// device) and written back, which is what a separate in-place scaling pass before the update would leave.
template <bool SCALE>
__device__ __forceinline__ void adamw_span(float *w, const float *g, float *m, float *v, int n,
                                           int start, int stride, const AdamwHyper &h, float bc1, float bc2,
                                           const float *scale_ptr = nullptr) {
    const bool vec = ((((uintptr_t)w) | ((uintptr_t)g) | ((uintptr_t)m) | ((uintptr_t)v)) & 15) == 0;
    float sc = 1.0f;
    if (SCALE) sc = *scale_ptr;
    const bool scaled = SCALE && sc < 1.0f;
    float *gw = const_cast<float *>(g);
    if (vec) {
        const int n4 = n >> 2;
        for (int j = start; j < n4; j += stride) {
            float4 W = reinterpret_cast<float4 *>(w)[j], M = reinterpret_cast<float4 *>(m)[j];
            float4 V = reinterpret_cast<float4 *>(v)[j];
            float4 G = reinterpret_cast<const float4 *>(g)[j];
            if (scaled) {
                G.x *= sc; G.y *= sc; G.z *= sc; G.w *= sc;
                reinterpret_cast<float4 *>(gw)[j] = G;
            }
            adamw_one(W.x, G.x, M.x, V.x, h.lr, h.b1, h.b2, h.eps, bc1, bc2, h.wd);
            adamw_one(W.y, G.y, M.y, V.y, h.lr, h.b1, h.b2, h.eps, bc1, bc2, h.wd);
            adamw_one(W.z, G.z, M.z, V.z, h.lr, h.b1, h.b2, h.eps, bc1, bc2, h.wd);
            adamw_one(W.w, G.w, M.w, V.w, h.lr, h.b1, h.b2, h.eps, bc1, bc2, h.wd);
            reinterpret_cast<float4 *>(w)[j] = W;
            reinterpret_cast<float4 *>(m)[j] = M;
            reinterpret_cast<float4 *>(v)[j] = V;
        }
        for (int i = (n4 << 2) + start; i < n; i += stride) {
            float gi = g[i];
            if (scaled) { gi *= sc; gw[i] = gi; }
            adamw_one(w[i], gi, m[i], v[i], h.lr, h.b1, h.b2, h.eps, bc1, bc2, h.wd);
        }
    } else {
        for (int i = start; i < n; i += stride) {
            float gi = g[i];
            if (scaled) { gi *= sc; gw[i] = gi; }
            adamw_one(w[i], gi, m[i], v[i], h.lr, h.b1, h.b2, h.eps, bc1, bc2, h.wd);
        }
    }
}

__global__ void adamw_kernel(float *w, const float *g, float *m, float *v, int n, AdamwHyper h,
                             float bc1, float bc2) {
    adamw_span<false>(w, g, m, v, n, blockIdx.x * blockDim.x + threadIdx.x, gridDim.x * blockDim.x, h, bc1, bc2);
}

// Up to kMaxTensors tensors per launch, passed by value in the kernel argument.
constexpr int kMaxTensors = 40;
struct AdamwBatch {
    float *w[kMaxTensors];
    const float *g[kMaxTensors];
    float *m[kMaxTensors];
    float *v[kMaxTensors];
    int n[kMaxTensors];
    float bc1[kMaxTensors], bc2[kMaxTensors];
    int blk_begin[kMaxTensors + 1];  // first workgroup of each tensor
    int count;
};

template <bool SCALE>
__global__ void adamw_multi_kernel(AdamwBatch b, AdamwHyper h, const float *scale_ptr) {
    int t = 0;
    while (t + 1 < b.count && (int)blockIdx.x >= b.blk_begin[t + 1]) t++;
    const int nblk = b.blk_begin[t + 1] - b.blk_begin[t];
    const int lb = blockIdx.x - b.blk_begin[t];
    adamw_span<SCALE>(b.w[t], b.g[t], b.m[t], b.v[t], b.n[t], lb * blockDim.x + threadIdx.x, nblk * blockDim.x, h,
                      b.bc1[t], b.bc2[t], scale_ptr);
}

// One partial per 256 elements (the reference's layout, core/kernels/adamw.cu:86-127):
// a wave sums one 256-element block with one 16-byte load per lane.
template <bool DOT>
__global__ void partial_sums_kernel(const float *__restrict__ a, const float *__restrict__ b,
                                    float *__restrict__ partial, int n, int nblk) {
    const int lane = threadIdx.x & 63;
    const int wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int nwaves = (gridDim.x * blockDim.x) >> 6;
    const bool vec = ((((uintptr_t)a) | (DOT ? (uintptr_t)b : 0)) & 15) == 0;
    for (int blk = wave; blk < nblk; blk += nwaves) {
        const int base = blk * 256;
        float s = 0.f;
        if (vec && base + 256 <= n) {
            const float4 x = reinterpret_cast<const float4 *>(a + base)[lane];
            const float4 y = DOT ? reinterpret_cast<const float4 *>(b + base)[lane] : x;
            s = x.x * y.x + x.y * y.y + x.z * y.z + x.w * y.w;
        } else {
            for (int i = base + lane; i < min(base + 256, n); i += 64) s += a[i] * (DOT ? b[i] : a[i]);
        }
        s = wave_allreduce(s);
        if (lane == 0) partial[blk] = s;
    }
}

__global__ void scale_kernel(float *g, float scale, const float *scale_ptr, int n) {
    if (scale_ptr) {
        scale = *scale_ptr;
        if (scale >= 1.0f) return;  // uniform: nothing to do (core/kernels/adamw.cu:257)
    }
    const int stride = gridDim.x * blockDim.x;
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if ((((uintptr_t)g) & 15) == 0) {
        const int n4 = n >> 2;
        for (int j = i; j < n4; j += stride) {
            float4 x = reinterpret_cast<float4 *>(g)[j];
            x.x *= scale; x.y *= scale; x.z *= scale; x.w *= scale;
            reinterpret_cast<float4 *>(g)[j] = x;
        }
        for (int j = (n4 << 2) + i; j < n; j += stride) g[j] *= scale;
    } else {
        for (; i < n; i += stride) g[i] *= scale;
    }
}

// norm = sqrt(sum partials); scale = min(1, max/norm) (core/kernels/adamw.cu:203-236)
constexpr int kClipThreads = 1024;   // one workgroup; four independent partial sums per thread
__global__ __launch_bounds__(kClipThreads) void reduce_partials_clip_kernel(const float *__restrict__ partial, int total,
                                                                            float max_grad_norm, float *out_norm,
                                                                            float *out_scale) {
    __shared__ float part[kClipThreads / 64];
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    int i = threadIdx.x;
    for (; i + 3 * kClipThreads < total; i += 4 * kClipThreads) {
        a0 += partial[i];
        a1 += partial[i + kClipThreads];
        a2 += partial[i + 2 * kClipThreads];
        a3 += partial[i + 3 * kClipThreads];
    }
    for (; i < total; i += kClipThreads) a0 += partial[i];
    float acc = wave_allreduce((a0 + a1) + (a2 + a3));
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        float t = 0.f;
        for (int w = 0; w < kClipThreads / 64; w++) t += part[w];
        const float norm = sqrtf(t);
        *out_norm = norm;
        *out_scale = (norm > max_grad_norm && max_grad_norm > 0.0f) ? (max_grad_norm / norm) : 1.0f;
    }
}

struct PtrBatch {
    float *p[kMaxTensors];
    int n[kMaxTensors];
    int blk_begin[kMaxTensors + 1];  // in units of kNormBlock-element blocks (norm) or workgroups (scale)
    int count;
};

// elements per partial sum of the multi-tensor norm: eight 16-byte loads per lane in flight before the one
// reduction (one load per reduction left the pass at 1.4 TB/s)
constexpr int kNormBlock = 2048;

__global__ void norm_sq_multi_kernel(PtrBatch b, float *__restrict__ partial) {
    const int lane = threadIdx.x & 63;
    const int wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int nwaves = (gridDim.x * blockDim.x) >> 6;
    const int total = b.blk_begin[b.count];
    for (int blk = wave; blk < total; blk += nwaves) {
        int t = 0;
        while (t + 1 < b.count && blk >= b.blk_begin[t + 1]) t++;
        const float *a = b.p[t];
        const int n = b.n[t], base = (blk - b.blk_begin[t]) * kNormBlock;
        float s = 0.f;
        if (((((uintptr_t)a) & 15) == 0) && base + kNormBlock <= n) {
            float4 x[kNormBlock / 256];
#pragma unroll
            for (int r = 0; r < kNormBlock / 256; r++) x[r] = reinterpret_cast<const float4 *>(a + base + 256 * r)[lane];
            float s0 = 0.f, s1 = 0.f;
#pragma unroll
            for (int r = 0; r < kNormBlock / 256; r += 2) {
                s0 += x[r].x * x[r].x + x[r].y * x[r].y + x[r].z * x[r].z + x[r].w * x[r].w;
                s1 += x[r + 1].x * x[r + 1].x + x[r + 1].y * x[r + 1].y + x[r + 1].z * x[r + 1].z + x[r + 1].w * x[r + 1].w;
            }
            s = s0 + s1;
        } else {
            for (int i = base + lane; i < min(base + kNormBlock, n); i += 64) s += a[i] * a[i];
        }
        s = wave_allreduce(s);
        if (lane == 0) partial[blk] = s;
    }
}

__global__ void scale_multi_kernel(PtrBatch b, const float *scale_ptr) {
    const float scale = *scale_ptr;
    if (scale >= 1.0f) return;
    int t = 0;
    while (t + 1 < b.count && (int)blockIdx.x >= b.blk_begin[t + 1]) t++;
    const int nblk = b.blk_begin[t + 1] - b.blk_begin[t];
    float *g = b.p[t];
    for (int i = (blockIdx.x - b.blk_begin[t]) * blockDim.x + threadIdx.x; i < b.n[t]; i += nblk * blockDim.x)
        g[i] *= scale;
}

static inline int opt_blocks(long long n) {
    long long b = (n / 4 + kOptThreads - 1) / kOptThreads;
    return (int)(b < 1 ? 1 : (b > 2048 ? 2048 : b));
}

static unsigned launch_status(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) fprintf(stderr, "%s: kernel launch failed: %s\n", what, hipGetErrorString(e));
    return (unsigned)e;
}

}  // namespace nlh

using namespace nlh;

// ── M3 optimizer helpers (core/kernels/m3_optimizer.cu) ─────────────────────
// m3_optimizer.cu:24-42: fast momentum, second moment, and (when update_m2) the slow momentum
__global__ void m3_ema_kernel(float *__restrict__ m1, float *__restrict__ m2, float *__restrict__ v,
                              const float *__restrict__ g, int n, float b1, float b2, float b3, int update_m2) {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) {
        const float gi = g[i];
        m1[i] = b1 * m1[i] + (1.0f - b1) * gi;
        v[i] = b2 * v[i] + (1.0f - b2) * gi * gi;
        if (update_m2) m2[i] = b3 * m2[i] + (1.0f - b3) * gi;
    }
}
// m3_optimizer.cu:66-80
__global__ void m3_apply_1d_kernel(float *__restrict__ w, const float *__restrict__ m1, const float *__restrict__ m2,
                                   const float *__restrict__ v, int n, float lr, float alpha, float eps, float bc2) {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) {
        const float combined = m1[i] + alpha * m2[i];
        w[i] -= lr * combined / (sqrtf(v[i] / bc2) + eps);
    }
}
// m3_optimizer.cu:103-114 (a = -lr, b = -lr alpha) and :204-215 (Newton-Schulz polynomial): x = a x' + b y + c z
// with x' = x or, for the 2-D update, w itself with coefficient 1
__global__ void axpbypcz_kernel(float *__restrict__ x, const float *__restrict__ y, const float *__restrict__ z, int n,
                                float a, float b, float c) {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x)
        x[i] = a * x[i] + b * y[i] + c * z[i];
}
__global__ void m3_apply_2d_kernel(float *__restrict__ w, const float *__restrict__ o1, const float *__restrict__ o2,
                                   int n, float lr, float alpha) {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x)
        w[i] -= lr * (o1[i] + alpha * o2[i]);
}

extern "C" {

unsigned adamw_update_cuda(float *w, const float *g, float *m, float *v, int n, float lr, float beta1,
                           float beta2, float eps, float bc1_inv, float bc2_inv, float weight_decay) {
    if (n <= 0) return 0;
    hipLaunchKernelGGL(adamw_kernel, dim3(opt_blocks(n)), dim3(kOptThreads), 0, stream(), w, g, m, v, n,
                       AdamwHyper{lr, beta1, beta2, eps, weight_decay}, bc1_inv, bc2_inv);
    return launch_status("adamw_update_cuda");
}

unsigned adamw_update_multi_rocm(float *const *w, const float *const *g, float *const *m, float *const *v,
                                 const int *n, const float *bc1_inv, const float *bc2_inv, int count,
                                 float lr, float beta1, float beta2, float eps, float weight_decay) {
    return nlh::adamw_update_multi_scaled(w, g, m, v, n, bc1_inv, bc2_inv, count, lr, beta1, beta2, eps, weight_decay,
                                          nullptr);
}

}  // extern "C"

unsigned nlh::adamw_update_multi_scaled(float *const *w, const float *const *g, float *const *m, float *const *v,
                                        const int *n, const float *bc1_inv, const float *bc2_inv, int count, float lr,
                                        float beta1, float beta2, float eps, float weight_decay,
                                        const float *scale_ptr) {
    const AdamwHyper h{lr, beta1, beta2, eps, weight_decay};
    // a batch is the next kMaxTensors input slots (empty ones skipped), so no tensor is seen twice
    for (int first = 0; first < count; first += kMaxTensors) {
        AdamwBatch b;
        b.count = 0;
        int blocks = 0;
        for (int i = first; i < count && i < first + kMaxTensors; i++) {
            if (n[i] <= 0) continue;
            const int c = b.count++;
            b.w[c] = w[i]; b.g[c] = g[i]; b.m[c] = m[i]; b.v[c] = v[i]; b.n[c] = n[i];
            b.bc1[c] = bc1_inv[i]; b.bc2[c] = bc2_inv[i];
            b.blk_begin[c] = blocks;
            int nb = (n[i] / 4 + kOptThreads - 1) / kOptThreads;
            blocks += nb < 1 ? 1 : (nb > 256 ? 256 : nb);
        }
        if (b.count == 0) continue;
        b.blk_begin[b.count] = blocks;
        if (scale_ptr)
            hipLaunchKernelGGL(adamw_multi_kernel<true>, dim3(blocks), dim3(kOptThreads), 0, stream(), b, h, scale_ptr);
        else
            hipLaunchKernelGGL(adamw_multi_kernel<false>, dim3(blocks), dim3(kOptThreads), 0, stream(), b, h, scale_ptr);
        unsigned rc = launch_status("adamw_update_multi_rocm");
        if (rc) return rc;
    }
    return 0;
}

extern "C" {

unsigned grad_norm_sq_cuda(const float *g, float *partial_sums, int n, int *out_num_blocks) {
    const int nblk = (n + 255) / 256;
    *out_num_blocks = nblk;
    if (nblk <= 0) return 0;
    const int grid = nblk < 4 ? 1 : (nblk / 4 > 2048 ? 2048 : nblk / 4);
    hipLaunchKernelGGL((partial_sums_kernel<false>), dim3(grid), dim3(kOptThreads), 0, stream(), g, nullptr,
                       partial_sums, n, nblk);
    return launch_status("grad_norm_sq_cuda");
}

unsigned dot_product_partial_f32_cuda(const float *a, const float *b, float *partial_sums, int n,
                                      int *out_num_blocks) {
    const int nblk = (n + 255) / 256;
    *out_num_blocks = nblk;
    if (nblk <= 0) return 0;
    const int grid = nblk < 4 ? 1 : (nblk / 4 > 2048 ? 2048 : nblk / 4);
    hipLaunchKernelGGL((partial_sums_kernel<true>), dim3(grid), dim3(kOptThreads), 0, stream(), a, b,
                       partial_sums, n, nblk);
    return launch_status("dot_product_partial_f32_cuda");
}

unsigned grad_scale_cuda(float *g, float scale, int n) {
    if (n <= 0) return 0;
    hipLaunchKernelGGL(scale_kernel, dim3(opt_blocks(n)), dim3(kOptThreads), 0, stream(), g, scale, nullptr, n);
    return launch_status("grad_scale_cuda");
}

unsigned reduce_partials_clip_cuda(const float *partial_sums, int total_partials, float max_grad_norm,
                                   float *out_norm, float *out_scale) {
    hipLaunchKernelGGL(reduce_partials_clip_kernel, dim3(1), dim3(kClipThreads), 0, stream(), partial_sums,
                       total_partials, max_grad_norm, out_norm, out_scale);
    return launch_status("reduce_partials_clip_cuda");
}

unsigned grad_scale_conditional_cuda(float *g, const float *scale_ptr, int n) {
    if (n <= 0) return 0;
    hipLaunchKernelGGL(scale_kernel, dim3(opt_blocks(n)), dim3(kOptThreads), 0, stream(), g, 1.0f, scale_ptr, n);
    return launch_status("grad_scale_conditional_cuda");
}

unsigned grad_norm_clip_multi_rocm(float *const *g, const int *n, int count, float max_grad_norm,
                                   float *out_norm, float *out_scale) {
    unsigned rc = nlh::grad_norm_scale_multi(g, n, count, max_grad_norm, out_norm, out_scale);
    if (rc) return rc;
    return nlh::grad_scale_multi(g, n, count, out_scale);
}

}  // extern "C"

// norm and clip factor of a set of tensors, left on the device: {norm} -> out_norm, {min(1, max / norm)} -> out_scale
unsigned nlh::grad_norm_scale_multi(float *const *g, const int *n, int count, float max_grad_norm, float *out_norm,
                                    float *out_scale) {
    const ErrorScope es;
    // pass 1: partial sums of every tensor into one scratch array
    long long total_blocks = 0;
    for (int i = 0; i < count; i++) total_blocks += n[i] > 0 ? (n[i] + kNormBlock - 1) / kNormBlock : 0;
    float *partial = scratch(11, (size_t)(total_blocks > 0 ? total_blocks : 1) * sizeof(float));
    if (es.failed()) return 1;
    int off = 0;
    for (int first = 0; first < count; first += kMaxTensors) {
        PtrBatch b;
        b.count = 0;
        int blocks = 0;
        for (int i = first; i < count && i < first + kMaxTensors; i++) {
            if (n[i] <= 0) continue;
            const int c = b.count++;
            b.p[c] = g[i]; b.n[c] = n[i]; b.blk_begin[c] = blocks;
            blocks += (n[i] + kNormBlock - 1) / kNormBlock;
        }
        if (b.count == 0) continue;
        b.blk_begin[b.count] = blocks;
        const int grid = blocks < 4 ? 1 : ((blocks + 3) / 4 > 2048 ? 2048 : (blocks + 3) / 4);   // a wave per block
        hipLaunchKernelGGL(norm_sq_multi_kernel, dim3(grid), dim3(kOptThreads), 0, stream(), b, partial + off);
        unsigned rc = launch_status("grad_norm_clip_multi_rocm/norm");
        if (rc) return rc;
        off += blocks;
    }
    return reduce_partials_clip_cuda(partial, off, max_grad_norm, out_norm, out_scale);
}

// every tensor times *scale_ptr, in place, when that is below 1
unsigned nlh::grad_scale_multi(float *const *g, const int *n, int count, const float *out_scale) {
    unsigned rc = 0;
    for (int first = 0; first < count; first += kMaxTensors) {
        PtrBatch b;
        b.count = 0;
        int blocks = 0;
        for (int i = first; i < count && i < first + kMaxTensors; i++) {
            if (n[i] <= 0) continue;
            const int c = b.count++;
            b.p[c] = g[i]; b.n[c] = n[i]; b.blk_begin[c] = blocks;
            int nb = (n[i] + kOptThreads * 4 - 1) / (kOptThreads * 4);
            blocks += nb > 256 ? 256 : nb;
        }
        if (b.count == 0) continue;
        b.blk_begin[b.count] = blocks;
        hipLaunchKernelGGL(scale_multi_kernel, dim3(blocks), dim3(kOptThreads), 0, stream(), b, out_scale);
        rc = launch_status("grad_norm_clip_multi_rocm/scale");
        if (rc) return rc;
    }
    return 0;
}


extern "C" {

// ── M3 optimizer helpers ────────────────────────────────────────────────────
unsigned m3_ema_update_cuda(float *m1, float *m2, float *v, const float *g, int n, float beta1, float beta2,
                            float beta3, int update_m2) {
    if (n <= 0) return 0;
    hipLaunchKernelGGL(m3_ema_kernel, dim3(opt_blocks(n)), dim3(kOptThreads), 0, stream(), m1, m2, v, g, n, beta1,
                       beta2, beta3, update_m2);
    return launch_status("m3_ema_update_cuda");
}

unsigned m3_apply_1d_cuda(float *w, const float *m1, const float *m2, const float *v, int n, float lr, float alpha,
                          float eps, float bc2) {
    if (n <= 0) return 0;
    hipLaunchKernelGGL(m3_apply_1d_kernel, dim3(opt_blocks(n)), dim3(kOptThreads), 0, stream(), w, m1, m2, v, n, lr,
                       alpha, eps, bc2);
    return launch_status("m3_apply_1d_cuda");
}

unsigned m3_apply_2d_cuda(float *w, const float *o1, const float *o2, int n, float lr, float alpha) {
    if (n <= 0) return 0;
    hipLaunchKernelGGL(m3_apply_2d_kernel, dim3(opt_blocks(n)), dim3(kOptThreads), 0, stream(), w, o1, o2, n, lr, alpha);
    return launch_status("m3_apply_2d_cuda");
}

// same partial-sum layout as grad_norm_sq_cuda: one partial per 256 elements (m3_optimizer.cu:141-178)
unsigned frob_norm_sq_cuda(const float *x, float *partial_sums, int n, int *out_num_blocks) {
    return grad_norm_sq_cuda(x, partial_sums, n, out_num_blocks);
}

unsigned scale_buf_cuda(float *x, float scale, int n) { return grad_scale_cuda(x, scale, n); }

unsigned m3_ns_poly_cuda(float *x, const float *y, const float *z, int n, float a, float b, float c) {
    if (n <= 0) return 0;
    hipLaunchKernelGGL(axpbypcz_kernel, dim3(opt_blocks(n)), dim3(kOptThreads), 0, stream(), x, y, z, n, a, b, c);
    return launch_status("m3_ns_poly_cuda");
}

}  // extern "C"
