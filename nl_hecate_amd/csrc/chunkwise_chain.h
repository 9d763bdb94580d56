// Frozen-M0 chunkwise Titans / Delta rule on bf16 tokens, one workgroup per chain with
// the memory (and momentum) resident on chip across the whole sequence.  Head size 64,
// chunks of up to 64 tokens.  Each returns false without launching when the shape is
// not covered.  y_rows: where the output rows go (null: head-major [batch, seq_len, 64]).
#pragma once
#include <stdint.h>

#include "head_rows.h"

namespace nlh {

bool chunkwise_chain_forward_bf16(const char *fn, const uint16_t *k, const uint16_t *v, const uint16_t *q,
                                  const float *alpha, const float *theta, const float *eta, const float *m_initial,
                                  const float *s_initial, float *m_states, float *s_states, float *y, int seq_len,
                                  int d, int batch, int chunk_size, bool has_s, const HeadRows *y_rows = nullptr);

}  // namespace nlh
