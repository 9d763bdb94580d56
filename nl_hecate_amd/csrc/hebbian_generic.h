// Hebbian rule for head sizes the tiled kernels of hebbian.hip do not cover (hebbian_generic.hip):
// any d from 1 to kHebGenericMaxD.  Layouts as in the entry points of hebbian.hip.
#pragma once

namespace nlh {

constexpr int kHebGenericMaxD = 3840;   // four d-vectors of LDS per workgroup in the backward

bool hebbian_generic_check(const char *fn, int d);
// ckpt = 0: trajectory (seq_len + 1 states per chain); ckpt > 0: slot 0, then one slot per boundary
void hebbian_forward_generic(const float *k, const float *v, const float *q, const float *alpha,
                             const float *m_initial, float *m_states, float *y, int seq_len, int d, int batch,
                             int input_stride, int m_stride, int ckpt, long long states_per_chain);
// tokens [t_start, t_end) in reverse; m_states local to the range; d_m_seed may be null; d_m_out [batch, d*d]
void hebbian_backward_generic(const float *k, const float *v, const float *q, const float *alpha,
                              const float *m_states, const float *d_y, const float *d_m_seed, float *d_k, float *d_v,
                              float *d_q, float *d_alpha, float *d_m_out, int seq_len, int t_start, int t_end, int d,
                              int batch);

}  // namespace nlh
