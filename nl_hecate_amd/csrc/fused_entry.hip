// Entry points of the reference that are compositions of other steps:
//   {titans,dgd}_fused_forward_f32_cuda  (core/kernels/titans_forward.cu:492-785, dgd_forward.cu):
//       L2-normalise k and q rows in place, compute the gates from the normalised k and raw v,
//       clamp alpha / theta, then run the recurrence over the full trajectory.
//   error_subtract_clip_f32_cuda         (core/kernels/error_subtract_clip.cu): pred -= v per
//       row, then L2-clip each row.
// The recurrence dominates; normalisation, gates and clamps are one streaming pass (fused_prep_kernel, a wave
// per token) launched ahead of it on the same stream: two launches per call.
#include <hip/hip_runtime.h>

#include "../../include/nl_hecate_ffi.h"
#include "lane_ops.h"
#include "runtime.h"

namespace nlh {
namespace {

// one wave per row
__global__ void error_subtract_clip_kernel(float *__restrict__ pred, const float *__restrict__ v, int rows, int d,
                                           float clip) {
    const int lane = threadIdx.x & 63;
    const int wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6, nwaves = (gridDim.x * blockDim.x) >> 6;
    for (int r = wave; r < rows; r += nwaves) {
        float *p = pred + (size_t)r * d;
        const float *vr = v + (size_t)r * d;
        float s = 0.f;
        for (int j = lane; j < d; j += 64) {
            const float e = p[j] - vr[j];
            p[j] = e;
            s = fmaf(e, e, s);
        }
        if (clip <= 0.f) continue;
        const float norm = sqrtf(wave_allreduce(s));
        if (norm > clip) {
            const float sc = clip / norm;
            for (int j = lane; j < d; j += 64) p[j] *= sc;
        }
    }
}

__device__ __forceinline__ float sigmoid_(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float softplus_(float x) { return x > 20.0f ? x : logf(1.0f + expf(x)); }

// What l2_normalize_rows x 2, gate_compute x 2 or 3 and clamp x 2 do, in one pass: one wave per token, the
// sums over the same lane pattern as those kernels.
template <bool HAS_ETA>
__global__ void fused_prep_kernel(float *__restrict__ k, const float *__restrict__ v, float *__restrict__ q,
                                  const float *__restrict__ w_alpha, const float *__restrict__ b_alpha,
                                  const float *__restrict__ w_theta, const float *__restrict__ b_theta,
                                  const float *__restrict__ w_eta, const float *__restrict__ b_eta, float alpha_floor,
                                  float alpha_ceil, float theta_floor, float theta_ceil, float *__restrict__ alpha,
                                  float *__restrict__ theta, float *__restrict__ eta, float *__restrict__ k_norms,
                                  float *__restrict__ q_norms, int rows, int d) {
    const int lane = threadIdx.x & 63;
    const int wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6, nwaves = (gridDim.x * blockDim.x) >> 6;
    const float ba = b_alpha[0], bt = b_theta[0], be = HAS_ETA ? b_eta[0] : 0.f;
    for (int r = wave; r < rows; r += nwaves) {
        float *kr = k + (size_t)r * d, *qr = q + (size_t)r * d;
        const float *vr = v + (size_t)r * d;
        float sk = 0.f, sq = 0.f;
        for (int j = lane; j < d; j += 64) { const float a = kr[j], b = qr[j]; sk += a * a; sq += b * b; }
        const float kn = sqrtf(wave_allreduce(sk)), qn = sqrtf(wave_allreduce(sq));
        const float ki = 1.0f / fmaxf(kn, 1e-8f), qi = 1.0f / fmaxf(qn, 1e-8f);
        float ga = 0.f, gt = 0.f, ge = 0.f;
        for (int j = lane; j < d; j += 64) {
            const float a = kr[j] * ki, b = vr[j];
            kr[j] = a;
            qr[j] *= qi;
            ga += a * w_alpha[j] + b * w_alpha[d + j];
            gt += a * w_theta[j] + b * w_theta[d + j];
            if (HAS_ETA) ge += a * w_eta[j] + b * w_eta[d + j];
        }
        ga = wave_allreduce(ga) + ba;
        gt = wave_allreduce(gt) + bt;
        if (HAS_ETA) ge = wave_allreduce(ge) + be;
        if (lane == 0) {
            k_norms[r] = kn;
            q_norms[r] = qn;
            alpha[r] = fmaxf(alpha_floor, fminf(alpha_ceil, sigmoid_(ga)));
            theta[r] = fmaxf(theta_floor, fminf(theta_ceil, softplus_(gt)));
            if (HAS_ETA) eta[r] = sigmoid_(ge);
        }
    }
}

template <bool HAS_ETA>
void fused_prep(float *k, const float *v, float *q, const float *w_alpha, const float *b_alpha, const float *w_theta,
                const float *b_theta, const float *w_eta, const float *b_eta, float alpha_floor, float alpha_ceil,
                float theta_floor, float theta_ceil, float *alpha, float *theta, float *eta, float *k_norms, float *q_norms,
                int rows, int d) {
    const long long threads = (long long)rows * 64;
    const int blocks = (int)((threads + 255) / 256 > 65535 * 16 ? 65535 * 16 : (threads + 255) / 256);
    hipLaunchKernelGGL(fused_prep_kernel<HAS_ETA>, dim3(blocks), dim3(256), 0, stream(), k, v, q, w_alpha, b_alpha, w_theta,
                       b_theta, w_eta, b_eta, alpha_floor, alpha_ceil, theta_floor, theta_ceil, alpha, theta, eta, k_norms,
                       q_norms, rows, d);
    check_launch("fused_prep_kernel");
}

}  // namespace
}  // namespace nlh

using namespace nlh;

extern "C" void error_subtract_clip_f32_cuda(float *predictions, const float *v, int total_rows, int d,
                                             float error_clip) {
    if (total_rows <= 0 || d <= 0) return;
    const long long threads = (long long)total_rows * 64;
    const int blocks = (int)((threads + 255) / 256 > 65535 * 16 ? 65535 * 16 : (threads + 255) / 256);
    hipLaunchKernelGGL(error_subtract_clip_kernel, dim3(blocks), dim3(256), 0, stream(), predictions, v, total_rows,
                       d, error_clip);
    check_launch("error_subtract_clip_kernel");
}

extern "C" void titans_fused_forward_f32_cuda(float *k_mem, const float *v_mem, float *q_mem, const float *w_alpha,
                                              const float *b_alpha_ptr, const float *w_theta,
                                              const float *b_theta_ptr, const float *w_eta, const float *b_eta_ptr,
                                              float alpha_floor, float alpha_ceil, float theta_floor,
                                              float theta_ceil, const float *m_initial, const float *s_initial,
                                              float *m_states, float *s_states, float *y, float *alpha_out,
                                              float *theta_out, float *eta_out, float *k_norms_out,
                                              float *q_norms_out, int seq_len, int d, int batch_size,
                                              float error_clip, float m_norm_max) {
    const ErrorScope es;
    if (seq_len <= 0 || d <= 0 || batch_size <= 0) {
        fail("titans_fused_forward_f32_cuda: seq_len, d and batch_size must be positive");
        return;
    }
    const int rows = batch_size * seq_len;
    fused_prep<true>(k_mem, v_mem, q_mem, w_alpha, b_alpha_ptr, w_theta, b_theta_ptr, w_eta, b_eta_ptr, alpha_floor, alpha_ceil,
                     theta_floor, theta_ceil, alpha_out, theta_out, eta_out, k_norms_out, q_norms_out, rows, d);
    if (es.failed()) return;
    titans_forward_f32_cuda(k_mem, v_mem, q_mem, alpha_out, theta_out, eta_out, m_initial, s_initial, m_states,
                            s_states, y, seq_len, d, batch_size, seq_len, d * d, error_clip, m_norm_max);
}

extern "C" void dgd_fused_forward_f32_cuda(float *k_mem, const float *v_mem, float *q_mem, const float *w_alpha,
                                           const float *b_alpha_ptr, const float *w_theta, const float *b_theta_ptr,
                                           float alpha_floor, float alpha_ceil, float theta_floor, float theta_ceil,
                                           const float *m_initial, float *m_states, float *y, float *alpha_out,
                                           float *theta_out, float *k_norms_out, float *q_norms_out, int seq_len,
                                           int d, int batch_size, float error_clip) {
    const ErrorScope es;
    if (seq_len <= 0 || d <= 0 || batch_size <= 0) {
        fail("dgd_fused_forward_f32_cuda: seq_len, d and batch_size must be positive");
        return;
    }
    const int rows = batch_size * seq_len;
    fused_prep<false>(k_mem, v_mem, q_mem, w_alpha, b_alpha_ptr, w_theta, b_theta_ptr, nullptr, nullptr, alpha_floor, alpha_ceil,
                      theta_floor, theta_ceil, alpha_out, theta_out, nullptr, k_norms_out, q_norms_out, rows, d);
    if (es.failed()) return;
    dgd_forward_f32_cuda(k_mem, v_mem, q_mem, alpha_out, theta_out, m_initial, m_states, y, seq_len, d, batch_size,
                         seq_len, d * d, error_clip);
}
