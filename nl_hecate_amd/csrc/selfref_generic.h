// HOPE self-referential memory, any head size from 1 to kSelfrefGenericMaxD (selfref_generic.hip).
// C = min(chunk_size, seq_len), nc = number of chunks; buffers as in the entry points of selfref.hip.
#pragma once
#include <stddef.h>

namespace nlh {

constexpr int kSelfrefGenericMaxD = 512;   // 20 d floats of LDS per workgroup

bool selfref_generic_check(const char *fn, int d);
void selfref_forward_generic(float *mems, const float *emb, float *y, float *kc, float *vc, float *qc, float *al,
                             float *th, float *am, float *em, float *frozen, int s, int d, int batch, int C, int nc,
                             bool sg);
void selfref_backward_generic(const float *emb, const float *dy, const float *kc, const float *vc, const float *qc,
                              const float *al, const float *th, const float *am, const float *em,
                              const float *frozen, float *d_emb, float *d_mems, int s, int d, int batch, int C,
                              int nc, bool sg);

}  // namespace nlh
