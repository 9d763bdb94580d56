// Per-chunk gradient pass of the chunkwise rule on bf16 tokens (head size 64, chunks of up
// to 64 tokens): d_q, d_k, d_v, d_theta, and for the gate pass pvec [token][4], xs
// [chunk][64*64] in accumulator-tile order, scal [chunk][4].  tab_a, tab_b (table_floats per
// chunk) and vecs (vec_floats per chunk) are scratch the pass fills itself.
#pragma once
#include <stddef.h>
#include <stdint.h>

namespace nlh {

size_t chunkwise_grads_table_floats();
size_t chunkwise_grads_vec_floats();

bool chunkwise_grads_bf16(const uint16_t *k, const uint16_t *v, const uint16_t *q, const float *d_y,
                          const float *alpha, const float *theta, const float *eta, const float *m_states,
                          const float *s_states, const float *dm_states, const float *ds_states, float *d_k,
                          float *d_v, float *d_q, float *d_theta, float *pvec, float *xs, float *scal,
                          float *tab_a, float *tab_b, float *vecs, int seq_len, int batch, int chunk_size,
                          bool has_s, int grid);

}  // namespace nlh
