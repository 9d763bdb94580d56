// Device-side test of whether the error clip or the Frobenius projection of the reference's chunkwise kernels
// can fire for a call, given the chunk-start states (chunkwise_guard.hip).  Costs one chunk-parallel kernel, a
// 4-byte copy to the host and a synchronisation of the launch stream (the reference's chunkwise wrappers
// synchronise the device themselves); not available while the launch stream is being captured.
#pragma once
#include <stdint.h>

#include "chunkwise_chain.h"

namespace nlh {

bool guard_possible();   // false while the launch stream is being captured into a graph, or while force_sequential is set
// how the last test of either kind came out: a hint for the order of work in the next call (a backward after a
// forward whose test fired does the stand-alone test first instead of a matrix-form pass it would throw away)
extern bool last_test_fired;
extern bool force_sequential;   // set around a call that has already run the test and lost
// true: a coupling may fire somewhere (or the test could not run): use the sequential kernels.  s_states null:
// the Delta rule (no momentum).  m_states / s_states [batch, num_chunks + 1, 64 * 64]; head size 64, chunk <= 64.
bool couplings_may_fire(const float *k, const float *v, const float *alpha, const float *theta, const float *eta,
                        const float *m_states, const float *s_states, int seq_len, int batch, int chunk_size,
                        float error_clip, float m_norm_max);
bool couplings_may_fire_bf16(const uint16_t *k, const uint16_t *v, const float *alpha, const float *theta, const float *eta,
                             const float *m_states, const float *s_states, int seq_len, int batch, int chunk_size,
                             float error_clip, float m_norm_max);

// The same decision from what a forward kernel left behind (ChainTracks, chunkwise_chain.h): a scalar recurrence per
// chunk, no product.  chain_tracks: the side buffers for a call, in the library's scratch.
ChainTracks chain_tracks(int seq_len, int batch, int chunk_size);
bool couplings_may_fire_tracked(const uint16_t *k, const float *alpha, const float *theta, const float *eta,
                                const ChainTracks &tr, bool has_s, int seq_len, int batch, int chunk_size, float error_clip,
                                float m_norm_max);
bool couplings_may_fire_tracked(const float *k, const float *alpha, const float *theta, const float *eta,
                                const ChainTracks &tr, bool has_s, int seq_len, int batch, int chunk_size, float error_clip,
                                float m_norm_max);

// For the exact rules and the sequential frozen-M0 kernels: msq_part [batch, parts] holds, per workgroup of a chain,
// an upper bound of max_t of the sum of squares of its rows of M_t.  true: the bound (plus rounding slack) reaches
// m_norm_max^2 for some chain, or the test could not run.  Same cost as above.
bool norm_bound_exceeded(const float *msq_part, int batch, int parts, float m_norm_max);

}  // namespace nlh
