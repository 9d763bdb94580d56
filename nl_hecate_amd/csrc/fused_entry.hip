// Entry points of the reference that are compositions of other steps:
//   {titans,dgd}_fused_forward_f32_cuda  (core/kernels/titans_forward.cu:492-785, dgd_forward.cu):
//       L2-normalise k and q rows in place, compute the gates from the normalised k and raw v,
//       clamp alpha / theta, then run the recurrence over the full trajectory.
//   error_subtract_clip_f32_cuda         (core/kernels/error_subtract_clip.cu): pred -= v per
//       row, then L2-clip each row.
// The recurrence dominates; normalisation and gates are streaming kernels launched ahead of it
// on the same stream.
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
    l2_normalize_rows_f32_cuda(k_mem, k_norms_out, rows, d, 1e-8f);
    l2_normalize_rows_f32_cuda(q_mem, q_norms_out, rows, d, 1e-8f);
    gate_compute_cuda(k_mem, v_mem, w_alpha, b_alpha_ptr, alpha_out, rows, d, 0);
    clamp_f32_cuda(alpha_out, rows, alpha_floor, alpha_ceil);
    gate_compute_cuda(k_mem, v_mem, w_theta, b_theta_ptr, theta_out, rows, d, 1);
    clamp_f32_cuda(theta_out, rows, theta_floor, theta_ceil);
    gate_compute_cuda(k_mem, v_mem, w_eta, b_eta_ptr, eta_out, rows, d, 0);
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
    l2_normalize_rows_f32_cuda(k_mem, k_norms_out, rows, d, 1e-8f);
    l2_normalize_rows_f32_cuda(q_mem, q_norms_out, rows, d, 1e-8f);
    gate_compute_cuda(k_mem, v_mem, w_alpha, b_alpha_ptr, alpha_out, rows, d, 0);
    clamp_f32_cuda(alpha_out, rows, alpha_floor, alpha_ceil);
    gate_compute_cuda(k_mem, v_mem, w_theta, b_theta_ptr, theta_out, rows, d, 1);
    clamp_f32_cuda(theta_out, rows, theta_floor, theta_ceil);
    if (es.failed()) return;
    dgd_forward_f32_cuda(k_mem, v_mem, q_mem, alpha_out, theta_out, m_initial, m_states, y, seq_len, d, batch_size,
                         seq_len, d * d, error_clip);
}
