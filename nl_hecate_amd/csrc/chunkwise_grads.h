// Backward of the chunkwise rule on bf16 tokens (head size 64, chunks of up to 64 tokens), three
// launches on the library's stream:
//   chunkwise_backward_coefficients: per-chunk coefficient table tab_b (table_floats per
//     chunk) and vectors vecs (vec_floats per chunk) from the gates
//   chunkwise_adjoint_bf16: the adjoint scan; dm_snap / ds_snap [batch][num_chunks + 1][64*64] in bf16,
//     slot c = adjoint of the state at the start of chunk c as the gradient pass takes it (one bf16
//     operand; slot 0 is not written), and dm_first / ds_first [batch][64*64] in fp32 = slot 0, the
//     gradient of the initial state
//   chunkwise_grads_bf16: d_q, d_k, d_v, d_theta, and for the gate pass
//     pvec [token][4] = p0_t = dy_t^T M0 q_t, ps_t = dy_t^T S0 q_t, -theta_t e_t^T dMo k_t, -theta_t e_t^T dSo k_t
//     xs [chunk][j][t] = -theta_j (dy_t . e_j)(q_t . k_j) (16 x 16 tiles with every t < j are not written)
//     scal [chunk][4] = <M0,dMo>, <S0,dMo>, <S0,dSo>
//   chunkwise_gate_gradients: d_alpha, d_eta from those (chunkwise_gates.hip; also serves the fp32 path)
#pragma once
#include <stddef.h>
#include <stdint.h>

#include "chunkwise_chain.h"
#include "head_rows.h"

namespace nlh {

size_t chunkwise_grads_table_floats();
size_t chunkwise_grads_vec_floats();

void chunkwise_backward_coefficients(const float *alpha, const float *theta, const float *eta,
                                     float *tab_b, float *vecs, int seq_len, int batch, int chunk_size, bool has_s);

bool chunkwise_adjoint_bf16(const uint16_t *k, const uint16_t *q, const float *d_y, const float *tab_b,
                            const float *vecs, uint16_t *dm_snap, uint16_t *ds_snap, float *dm_first,
                            float *ds_first, int seq_len, int batch, int chunk_size, bool has_s,
                            const HeadRows *dy_rows = nullptr);

// d_k, d_v, d_q as bf16 in token-major slabs instead of fp32 head-major tensors: chain c = (level, batch element,
// head) writes its 64 columns of token t at slab + rows.offset(c) + t * rows.row_stride
struct GradOut16 {
    uint16_t *gk, *gv, *gq;
    HeadRows rows;
};

bool chunkwise_grads_bf16(const uint16_t *k, const uint16_t *v, const uint16_t *q, const float *d_y,
                          const float *m_states, const float *s_states, const uint16_t *dm_snap,
                          const uint16_t *ds_snap, float *d_k, float *d_v, float *d_q, float *d_theta, float *pvec,
                          float *xs, float *scal, const float *tab_b, const float *vecs,
                          int seq_len, int batch, int chunk_size, bool has_s, int grid,
                          const HeadRows *dy_rows = nullptr, const GradOut16 *out16 = nullptr,
                          const ChainTracks *tracks = nullptr);   // tracks: also leave the side outputs of chunkwise_chain.h

// titans_chunkwise_backward_bf16_tokens_rocm with d_k, d_v, d_q leaving as bf16 token-major slabs (the level step's
// GEMM operand): same arguments otherwise
void titans_chunkwise_backward_bf16_tokens_g16(const uint16_t *k_mem, const uint16_t *v_mem, const uint16_t *q_mem,
                                               const float *alpha, const float *theta, const float *eta,
                                               const float *m_chunk_states, const float *s_chunk_states,
                                               const float *d_y_tokens, const GradOut16 &out, float *d_alpha, float *d_theta,
                                               float *d_eta, float *d_m_initial, float *d_s_initial, int seq_len, int d,
                                               int batch_size, int chunk_size, int heads, int levels, int d_y_per_level);

// also runs the first stage of the batch sum of the initial-state gradients: tmp [nsum][ceil(batch / per)][64*64]
// receives the sums of `per` consecutive chains of dm_first (and ds_first when nsum = 2), [batch][chain_stride]
void chunkwise_gate_gradients(const float *alpha, const float *eta, const float *pvec, const float *xs,
                              const float *scal, float *d_alpha, float *d_eta, int seq_len, int batch,
                              int chunk_size, bool has_s, const float *dm_first, const float *ds_first,
                              size_t chain_stride, int per, int nsum, float *tmp);

}  // namespace nlh
