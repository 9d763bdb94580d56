// Frozen-M0 chunkwise Titans / Delta rule on bf16 tokens, one workgroup per chain with
// the memory (and momentum) resident on chip across the whole sequence.  Head size 64,
// chunks of up to 64 tokens.  Each returns false without launching when the shape is
// not covered.  y_rows: where the output rows go (null: head-major [batch, seq_len, 64]).
#pragma once
#include <stdint.h>

#include "head_rows.h"

namespace nlh {

// What a test of the reference's couplings needs from the forward (chunkwise_guard.hip), left behind by the chain
// kernel as it goes: e2 [batch, 2 halves, num_chunks * 64] = the sum over the half's 32 memory rows of the squared
// frozen-M0 errors of every token (zero past a short chunk), nrm [batch, num_chunks, 2 halves, 4, 2] = partial sums
// of squares of the chunk-start M and S (eight partials per chunk and matrix).  Null: not wanted.
struct ChainTracks { float *e2, *nrm; };

bool chunkwise_chain_forward_bf16(const char *fn, const uint16_t *k, const uint16_t *v, const uint16_t *q,
                                  const float *alpha, const float *theta, const float *eta, const float *m_initial,
                                  const float *s_initial, float *m_states, float *s_states, float *y, int seq_len,
                                  int d, int batch, int chunk_size, bool has_s, const HeadRows *y_rows = nullptr,
                                  const ChainTracks *tracks = nullptr);

// The float-token matrix form (chunkwise_mm.hip) with the same side outputs; eta / s_initial / s_states null without
// momentum.
void chunkwise_forward_mm_f32_tracked(const char *fn, const float *k, const float *v, const float *q, const float *alpha,
                                      const float *theta, const float *eta, const float *m_initial, const float *s_initial,
                                      float *m_states, float *s_states, float *y, int seq_len, int d, int batch,
                                      int chunk_size, bool has_s, const ChainTracks &tracks);

// The float-token matrix-form backward whose gradient pass leaves the same side outputs and which ends with the test
// of the couplings on them, before anything is added to d_m_initial / d_s_initial.  false: a coupling may have
// fired; the caller runs the sequential kernels, which overwrite every other output.
bool chunkwise_backward_mm_f32_guarded(const char *fn, const float *k, const float *v, const float *q, const float *alpha,
                                       const float *theta, const float *eta, const float *m_states, const float *s_states,
                                       const float *d_y, float *d_k, float *d_v, float *d_q, float *d_alpha, float *d_theta,
                                       float *d_eta, float *d_m_initial, float *d_s_initial, int seq_len, int d, int batch,
                                       int chunk_size, bool has_s, float error_clip, float m_norm_max);

// the same for bf16 tokens (the chain-resident kernels' backward)
bool chunkwise_backward_bf16_guarded(const char *fn, const uint16_t *k, const uint16_t *v, const uint16_t *q, const float *alpha,
                                     const float *theta, const float *eta, const float *m_states, const float *s_states,
                                     const float *d_y, float *d_k, float *d_v, float *d_q, float *d_alpha, float *d_theta,
                                     float *d_eta, float *d_m_initial, float *d_s_initial, int seq_len, int d, int batch,
                                     int chunk_size, bool has_s, float error_clip, float m_norm_max);

}  // namespace nlh
