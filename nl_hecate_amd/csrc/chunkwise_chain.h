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

}  // namespace nlh
