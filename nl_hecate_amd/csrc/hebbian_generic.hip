// Hebbian rule M <- (1 - alpha) M + v k^T, y = M q (core/src/dispatch.rs:1566-1660) for any head size.
// The reference's kernels take any d (its tests run them at d = 2048, core/tests/test_cuda_large_d.rs:353-425);
// the tiled kernels of hebbian.hip hold d in {8, 16, 32, 64, 128} in registers, everything else comes here.
// Forward: rows of M never mix, so every row is a wave's own sequential job over the tokens, its state read
// from the slot before and written to the next one (the trajectory is the output anyway): no barrier at all,
// d x batch waves.  Backward: per token a row pass (dM += dy q^T, d_v, the d_alpha inner product) and a column
// pass (d_q, d_k are sums over rows), one workgroup per chain with dM in its output buffer; the retention of
// a token is applied by the next token's row pass.  Correct and simple, not tuned.
#include "hebbian_generic.h"
#include "lane_ops.h"
#include "runtime.h"

namespace nlh {
namespace {

constexpr int kFwdThreads = 256, kBwdThreads = 1024;

__global__ __launch_bounds__(kFwdThreads) void hebbian_fwd_generic_kernel(
    const float *__restrict__ k, const float *__restrict__ v, const float *__restrict__ q,
    const float *__restrict__ alpha, const float *__restrict__ m_initial, float *__restrict__ m_states,
    float *__restrict__ y, int s, int d, int input_stride, int m_stride, int ckpt, long long states_per_chain) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, b = blockIdx.x;
    const size_t dd = (size_t)d * d;
    float *st = m_states + (size_t)b * states_per_chain * dd;
    for (int row = blockIdx.y * (kFwdThreads / 64) + wave; row < d; row += gridDim.y * (kFwdThreads / 64)) {
        const float *m0 = m_initial + (size_t)b * m_stride + (size_t)row * d;
        float *slot0 = st + (size_t)row * d;
        for (int j = lane; j < d; j += 64) slot0[j] = m0[j];
        int slot = 0;
        bool seg_start = true;
        for (int t = 0; t < s; t++) {
            const size_t tok = (size_t)b * input_stride + t;
            const float keep = 1.f - alpha[tok], vi = v[tok * d + row];
            const float *kt = k + tok * d, *qt = q + tok * d;
            const float *src;
            float *dst;
            if (ckpt == 0) {
                src = st + (size_t)t * dd + (size_t)row * d;
                dst = st + (size_t)(t + 1) * dd + (size_t)row * d;
            } else {   // the running state lives in the slot after the segment's checkpoint
                dst = st + (size_t)(slot + 1) * dd + (size_t)row * d;
                src = seg_start ? st + (size_t)slot * dd + (size_t)row * d : dst;
                seg_start = false;
            }
            float acc = 0.f;
            for (int j = lane; j < d; j += 64) {
                const float r = fmaf(keep, src[j], vi * kt[j]);
                dst[j] = r;
                acc = fmaf(r, qt[j], acc);
            }
            acc = wave_allreduce(acc);
            if (lane == 0) y[((size_t)b * s + t) * d + row] = acc;
            if (ckpt > 0 && ((t + 1) % ckpt == 0 || t + 1 == s)) { slot++; seg_start = true; }
        }
    }
}

__global__ __launch_bounds__(kBwdThreads) void hebbian_bwd_generic_kernel(
    const float *__restrict__ k, const float *__restrict__ v, const float *__restrict__ q,
    const float *__restrict__ alpha, const float *__restrict__ m_states, const float *__restrict__ d_y,
    const float *__restrict__ d_m_seed, float *__restrict__ d_k, float *__restrict__ d_v, float *__restrict__ d_q,
    float *__restrict__ d_alpha, float *__restrict__ d_m_out, int seq_len, int t_start, int t_end, int d) {
    extern __shared__ float sh[];
    float *ks = sh, *vs = ks + d, *qs = vs + d, *dys = qs + d, *red = dys + d;   // red [kBwdThreads / 64]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, b = blockIdx.x;
    constexpr int kWaves = kBwdThreads / 64;
    const size_t dd = (size_t)d * d;
    const int len = t_end - t_start;
    float *dM = d_m_out + (size_t)b * dd;
    const float *traj = m_states + (size_t)b * (len + 1) * dd;
    for (size_t e = tid; e < dd; e += kBwdThreads) dM[e] = d_m_seed ? d_m_seed[(size_t)b * dd + e] : 0.f;
    float pending = 1.f;   // retention of the token before, not yet applied to dM
    __syncthreads();
    for (int t = t_end - 1; t >= t_start; t--) {
        const size_t tok = (size_t)b * seq_len + t;
        for (int j = tid; j < d; j += kBwdThreads) {
            ks[j] = k[tok * d + j]; vs[j] = v[tok * d + j]; qs[j] = q[tok * d + j]; dys[j] = d_y[tok * d + j];
        }
        const float *mt = traj + (size_t)(t - t_start) * dd, *mn = mt + dd;
        __syncthreads();
        float pa = 0.f;
        for (int row = wave; row < d; row += kWaves) {
            const float dyi = dys[row];
            float *g = dM + (size_t)row * d;
            const float *m = mt + (size_t)row * d;
            float av = 0.f, aa = 0.f;
            for (int j = lane; j < d; j += 64) {
                const float x = fmaf(pending, g[j], dyi * qs[j]);
                g[j] = x;
                av = fmaf(x, ks[j], av);
                aa = fmaf(m[j], x, aa);
            }
            av = wave_allreduce(av);
            pa += wave_allreduce(aa);
            if (lane == 0) d_v[tok * d + row] = av;
        }
        if (lane == 0) red[wave] = pa;
        __syncthreads();
        for (int j = tid; j < d; j += kBwdThreads) {
            float sq = 0.f, sk = 0.f;
            for (int i = 0; i < d; i++) {
                sq = fmaf(mn[(size_t)i * d + j], dys[i], sq);
                sk = fmaf(dM[(size_t)i * d + j], vs[i], sk);
            }
            d_q[tok * d + j] = sq;
            d_k[tok * d + j] = sk;
        }
        if (tid == 0) {
            float da = 0.f;
            for (int w = 0; w < kWaves; w++) da += red[w];
            d_alpha[tok] = -da;
        }
        pending = 1.f - alpha[tok];
        __syncthreads();
    }
    for (size_t e = tid; e < dd; e += kBwdThreads) dM[e] *= pending;
}

}  // namespace

bool hebbian_generic_check(const char *fn, int d) {
    if (d < 1 || d > kHebGenericMaxD) {
        fail("%s: d=%d is beyond the general kernels (1 .. %d)", fn, d, kHebGenericMaxD);
        return false;
    }
    return true;
}

void hebbian_forward_generic(const float *k, const float *v, const float *q, const float *alpha,
                             const float *m_initial, float *m_states, float *y, int seq_len, int d, int batch,
                             int input_stride, int m_stride, int ckpt, long long states_per_chain) {
    const int row_blocks = (d + kFwdThreads / 64 - 1) / (kFwdThreads / 64);
    KernelTimer kt("hebbian_fwd_generic_kernel");
    hipLaunchKernelGGL(hebbian_fwd_generic_kernel, dim3(batch, row_blocks < 4096 ? row_blocks : 4096), dim3(kFwdThreads), 0,
                       stream(), k, v, q, alpha, m_initial, m_states, y, seq_len, d, input_stride, m_stride, ckpt,
                       states_per_chain);
    check_launch("hebbian_fwd_generic_kernel");
}

void hebbian_backward_generic(const float *k, const float *v, const float *q, const float *alpha,
                              const float *m_states, const float *d_y, const float *d_m_seed, float *d_k, float *d_v,
                              float *d_q, float *d_alpha, float *d_m_out, int seq_len, int t_start, int t_end, int d,
                              int batch) {
    const size_t lds = ((size_t)4 * d + kBwdThreads / 64) * sizeof(float);
    KernelTimer kt("hebbian_bwd_generic_kernel");
    hipLaunchKernelGGL(hebbian_bwd_generic_kernel, dim3(batch), dim3(kBwdThreads), lds, stream(), k, v, q, alpha, m_states,
                       d_y, d_m_seed, d_k, d_v, d_q, d_alpha, d_m_out, seq_len, t_start, t_end, d);
    check_launch("hebbian_bwd_generic_kernel");
}

}  // namespace nlh
