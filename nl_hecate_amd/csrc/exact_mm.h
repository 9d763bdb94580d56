// Checkpointed backward of the exact Titans / Delta rule in chunk-parallel matrix form (exact_mm.hip): head size 64,
// checkpoints every C <= 64 tokens, m_ckpt / s_ckpt [batch][n_ckpt_count(seq_len, C)][64*64].
#pragma once

namespace nlh {

bool exact_backward_mm_applies(int d, int C);
bool exact_backward_mm_pays(int seq_len, int batch, int C);   // faster than the fused sequential kernel at this shape
// error_clip / m_norm_guard > 0: the pass also leaves the error and state norms behind and ends with the test of
// whether a coupling could have fired, BEFORE anything is added to d_m_initial / d_s_initial; false: one may have,
// the caller runs the kernels that apply the couplings, which overwrite every other output.  s_ckpt, eta, d_eta,
// d_s_initial null without momentum (has_s false).
bool exact_backward_mm(const char *fn, bool has_s, const float *k, const float *v, const float *q, const float *alpha,
                       const float *theta, const float *eta, const float *m_ckpt, const float *s_ckpt, const float *d_y,
                       float *d_k, float *d_v, float *d_q, float *d_alpha, float *d_theta, float *d_eta, float *d_m_initial,
                       float *d_s_initial, int seq_len, int batch, int C, float error_clip, float m_norm_guard);

}  // namespace nlh
