// Matrix-core sliding-window attention paths (head size 64 or 32, no persistent prefix,
// window <= 512).  Each returns false without launching when the shape is not covered.
// With stats non-null ([batch, heads, seq_len, 2] fp32: the row maximum of the scaled scores in
// base-2 units and the reciprocal of the row sum) the forward stores those instead of the weight
// tensor and the backward rebuilds the weights from Q K^T; attn_weights is then not touched.
#pragma once
#include <stdint.h>

namespace nlh {

bool swa_forward_mfma(const uint16_t *q, const uint16_t *k, const uint16_t *v, uint16_t *out, uint16_t *attn_weights,
                      int seq_len, int num_heads, int head_dim, int window, int batch, int n_persistent,
                      float *stats = nullptr);

// cols (statistics pair only): the three gradients leave as bf16 into columns of a wider row-major matrix, row stride
// ld elements, written rather than accumulated; d_q, d_k, d_v are then not touched.
struct SwaGradCols { uint16_t *q, *k, *v; long long ld; };

bool swa_backward_mfma(const uint16_t *q, const uint16_t *k, const uint16_t *v, const uint16_t *attn_weights,
                       const float *d_attn_out, float *d_q, float *d_k, float *d_v, int seq_len, int num_heads,
                       int head_dim, int window, int batch, int n_persistent, const float *stats = nullptr,
                       const SwaGradCols *cols = nullptr);

}  // namespace nlh
