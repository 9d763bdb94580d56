/* TEST INFRASTRUCTURE ONLY.
 *
 * CPU oracle for the pieces around the memory rules: AdamW, gradient-norm
 * clipping, gate projections and their backward, row L2 normalisation, the
 * Conductor's pulse rule, sliding-window attention.  Plain C restatement of
 * the reference's CPU code (file:line cited per function); never linked into
 * the product library.
 *
 * What pins each function (tests/test_oracle_layer.py):
 *   orc_adamw_step       : textbook closed form for step 1, torch.optim.AdamW
 *                          on CPU for several steps, per-level step counters
 *                          under a scripted pulse sequence
 *                          (core/src/adamw.rs:437-500).
 *   orc_gate_compute/_backward : numpy, finite differences.
 *   orc_l2_normalize*    : numpy, finite differences, unit-norm invariant.
 *   orc_pulse            : truth tables of core/src/conductor.rs:268-300,387-427.
 *   orc_swa_*            : window=1 copies V, identical keys give the uniform
 *                          average (core/src/swa.rs:286-344), torch SDPA with a
 *                          banded mask, finite differences.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* core/src/adamw.rs:102-126 adamw_step_buf */
void orc_adamw_step(float *params, const float *grads, float *m, float *v, int64_t n,
                    float lr, float beta1, float beta2, float eps,
                    float bc1_inv, float bc2_inv, float weight_decay) {
    for (int64_t i = 0; i < n; i++) {
        float g = grads[i];
        m[i] = beta1 * m[i] + (1.0f - beta1) * g;
        v[i] = beta2 * v[i] + (1.0f - beta2) * g * g;
        float m_hat = m[i] * bc1_inv;
        float v_hat = v[i] * bc2_inv;
        params[i] -= lr * (m_hat / (sqrtf(v_hat) + eps) + weight_decay * params[i]);
    }
}

/* Global L2 norm in f64 and clip scale: core/src/adamw.rs:203-262.
 * Returns the pre-clip norm; *scale = max/norm when norm > max > 0, else 1. */
float orc_grad_norm_clip(const float *const *grads, const int64_t *n, int count,
                         float max_grad_norm, float *scale) {
    double sq = 0.0;
    for (int t = 0; t < count; t++)
        for (int64_t i = 0; i < n[t]; i++) sq += (double)grads[t][i] * (double)grads[t][i];
    float norm = (float)sqrt(sq);
    *scale = (max_grad_norm > 0.0f && norm > max_grad_norm) ? max_grad_norm / norm : 1.0f;
    return norm;
}

/* Conductor::pulse, core/src/conductor.rs:136-144: level l is active iff
 * step % chunk_sizes[l] == 0, or seq_len > 0 and seq_len >= chunk_sizes[l]. */
void orc_pulse(int64_t step, const int64_t *chunk_sizes, int k, int64_t seq_len, int *active) {
    for (int l = 0; l < k; l++)
        active[l] = (step % chunk_sizes[l] == 0) || (seq_len > 0 && seq_len >= chunk_sizes[l]);
}

/* Gate projection as the GPU path computes it, core/kernels/elementwise.cu:167-214:
 * act(k.w[:d] + v.w[d:] + bias); sigmoid unclamped, softplus identity above 20. */
void orc_gate_compute(const float *k, const float *v, const float *w, float bias, float *out,
                      int n_tok, int d, int activation) {
    for (int t = 0; t < n_tok; t++) {
        float sum = 0.0f;
        for (int i = 0; i < d; i++) {
            sum += k[(size_t)t * d + i] * w[i];
            sum += v[(size_t)t * d + i] * w[d + i];
        }
        sum += bias;
        out[t] = activation == 0 ? 1.0f / (1.0f + expf(-sum))
                                 : (sum > 20.0f ? sum : logf(1.0f + expf(sum)));
    }
}

/* core/kernels/gate_backward.cu:29-106: d_w[2D], d_b from cached gate outputs. */
void orc_gate_backward(const float *d_alpha, const float *alpha, const float *d_theta,
                       const float *theta, const float *d_eta, const float *eta,
                       const float *k, const float *v,
                       float *d_w_alpha, float *d_b_alpha, float *d_w_theta, float *d_b_theta,
                       float *d_w_eta, float *d_b_eta, int T, int D, int has_theta, int has_eta) {
    for (int i = 0; i < 2 * D; i++) {
        float wa = 0.0f, wt = 0.0f, we = 0.0f;
        for (int t = 0; t < T; t++) {
            float x = i < D ? k[(size_t)t * D + i] : v[(size_t)t * D + (i - D)];
            float a = alpha[t];
            wa += d_alpha[t] * a * (1.0f - a) * x;
            if (has_theta) wt += d_theta[t] * (1.0f - expf(-theta[t])) * x;
            if (has_eta) { float e = eta[t]; we += d_eta[t] * e * (1.0f - e) * x; }
        }
        d_w_alpha[i] = wa;
        if (has_theta) d_w_theta[i] = wt;
        if (has_eta) d_w_eta[i] = we;
    }
    float ba = 0.0f, bt = 0.0f, be = 0.0f;
    for (int t = 0; t < T; t++) {
        float a = alpha[t];
        ba += d_alpha[t] * a * (1.0f - a);
        if (has_theta) bt += d_theta[t] * (1.0f - expf(-theta[t]));
        if (has_eta) { float e = eta[t]; be += d_eta[t] * e * (1.0f - e); }
    }
    d_b_alpha[0] = ba;
    if (has_theta) d_b_theta[0] = bt;
    if (has_eta) d_b_eta[0] = be;
}

/* core/src/tensor.rs:296-316 l2_normalize_rows (eps = 1e-8 there; argument here) */
void orc_l2_normalize_rows(float *x, float *norms, int n_rows, int d, float eps) {
    for (int i = 0; i < n_rows; i++) {
        float *row = x + (size_t)i * d;
        float sq = 0.0f;
        for (int j = 0; j < d; j++) sq += row[j] * row[j];
        float norm = sqrtf(sq);
        norms[i] = norm;
        float inv = 1.0f / (norm > eps ? norm : eps);
        for (int j = 0; j < d; j++) row[j] *= inv;
    }
}

/* core/src/tensor.rs:322-351 l2_normalize_rows_backward */
void orc_l2_normalize_backward(const float *d_out, const float *x_norm, const float *norms,
                               float *d_in, int n_rows, int d, float eps) {
    for (int i = 0; i < n_rows; i++) {
        const float *g = d_out + (size_t)i * d, *x = x_norm + (size_t)i * d;
        float *o = d_in + (size_t)i * d;
        if (norms[i] >= eps) {
            float inv = 1.0f / norms[i], dot = 0.0f;
            for (int j = 0; j < d; j++) dot += g[j] * x[j];
            for (int j = 0; j < d; j++) o[j] = (g[j] - x[j] * dot) * inv;
        } else {
            float inv_eps = 1.0f / eps;
            for (int j = 0; j < d; j++) o[j] = g[j] * inv_eps;
        }
    }
}

/* bf16 round-to-nearest-even, core/src/tensor.rs:37-42 style */
static uint16_t f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
static float bf16_to_f32(uint16_t h) {
    uint32_t u = ((uint32_t)h) << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}
void orc_f32_to_bf16(const float *src, uint16_t *dst, int64_t n) {
    for (int64_t i = 0; i < n; i++) dst[i] = f32_to_bf16(src[i]);
}
void orc_bf16_to_f32(const uint16_t *src, float *dst, int64_t n) {
    for (int64_t i = 0; i < n; i++) dst[i] = bf16_to_f32(src[i]);
}

/* ── Sliding-window attention ────────────────────────────────────────────────
 * Window geometry of one query (core/kernels/swa_forward.cu:49-60): prefix keys
 * [0, n_p), n_p = min(t+1, n_persistent); local keys [ls, ls+ll) with
 * ls = max(t+1-window, n_persistent), ll = t+1-ls when t >= n_persistent, else
 * ll = 0.  Weight slot of prefix key p is p; of local key ls+w is n_persistent+w.
 * With n_persistent = 0 this is the causal window [max(0,t-window+1), t] of
 * core/src/swa.rs:33-92. */
static void swa_geometry(int t, int window, int n_persistent, int *n_p, int *ls, int *ll) {
    *n_p = t + 1 < n_persistent ? t + 1 : n_persistent;
    if (t >= n_persistent) {
        *ls = t + 1 - window > n_persistent ? t + 1 - window : n_persistent;
        *ll = t + 1 - *ls;
    } else {
        *ls = 0;
        *ll = 0;
    }
}

/* Forward: core/src/swa.rs:33-92 with the GPU kernel's storage contract
 * (core/kernels/swa_forward.cu:23-159): q,k,v,out [batch, seq, heads*hd] bf16,
 * f32 math, scale 1/sqrt(hd), softmax over the valid slots, out = sum w*v with
 * the unrounded weights, attn_weights [batch, heads, seq, n_persistent+window]
 * stored as bf16 with 0 in unused slots. */
void orc_swa_forward(const uint16_t *q, const uint16_t *k, const uint16_t *v,
                     uint16_t *out, uint16_t *attn_weights,
                     int seq_len, int num_heads, int head_dim, int window, int batch,
                     int n_persistent) {
    int td = num_heads * head_dim, aw = n_persistent + window;
    float scale = 1.0f / sqrtf((float)head_dim);
    float *sc = (float *)malloc(sizeof(float) * aw);
    float *acc = (float *)malloc(sizeof(float) * head_dim);
    for (int b = 0; b < batch; b++)
        for (int h = 0; h < num_heads; h++)
            for (int t = 0; t < seq_len; t++) {
                const uint16_t *qr = q + ((size_t)b * seq_len + t) * td + h * head_dim;
                int n_p, ls, ll;
                swa_geometry(t, window, n_persistent, &n_p, &ls, &ll);
                float mx = -INFINITY;
                for (int s = 0; s < aw; s++) {
                    int valid = s < n_persistent ? s < n_p : (s - n_persistent) < ll;
                    sc[s] = -INFINITY;
                    if (!valid) continue;
                    int key = s < n_persistent ? s : ls + (s - n_persistent);
                    const uint16_t *kr = k + ((size_t)b * seq_len + key) * td + h * head_dim;
                    float dot = 0.0f;
                    for (int j = 0; j < head_dim; j++) dot += bf16_to_f32(qr[j]) * bf16_to_f32(kr[j]);
                    sc[s] = dot * scale;
                    if (sc[s] > mx) mx = sc[s];
                }
                float sum = 0.0f;
                for (int s = 0; s < aw; s++) {
                    sc[s] = sc[s] == -INFINITY ? 0.0f : expf(sc[s] - mx);
                    sum += sc[s];
                }
                uint16_t *wr = attn_weights + (((size_t)b * num_heads + h) * seq_len + t) * aw;
                for (int j = 0; j < head_dim; j++) acc[j] = 0.0f;
                for (int s = 0; s < aw; s++) {
                    float w = sc[s] / sum;
                    wr[s] = f32_to_bf16(w);
                    int valid = s < n_persistent ? s < n_p : (s - n_persistent) < ll;
                    if (!valid) continue;
                    int key = s < n_persistent ? s : ls + (s - n_persistent);
                    const uint16_t *vr = v + ((size_t)b * seq_len + key) * td + h * head_dim;
                    for (int j = 0; j < head_dim; j++) acc[j] += w * bf16_to_f32(vr[j]);
                }
                uint16_t *orow = out + ((size_t)b * seq_len + t) * td + h * head_dim;
                for (int j = 0; j < head_dim; j++) orow[j] = f32_to_bf16(acc[j]);
            }
    free(sc); free(acc);
}

/* Backward: core/src/swa.rs:163-235 swa_backward_rust on the stored (bf16)
 * weights, as core/kernels/swa_backward.cu:24-162 does:
 *   dV[key] += w * dO ;  dW = dO . V[key] ;  dS = w * (dW - sum_s w_s dW_s) ;
 *   dQ = sum dS * scale * K[key] ;  dK[key] += dS * scale * Q.
 * d_q is overwritten, d_k / d_v are accumulated into caller-zeroed buffers. */
void orc_swa_backward(const uint16_t *q, const uint16_t *k, const uint16_t *v,
                      const uint16_t *attn_weights, const float *d_out,
                      float *d_q, float *d_k, float *d_v,
                      int seq_len, int num_heads, int head_dim, int window, int batch,
                      int n_persistent) {
    int td = num_heads * head_dim, aw = n_persistent + window;
    float scale = 1.0f / sqrtf((float)head_dim);
    float *dw = (float *)malloc(sizeof(float) * aw);
    for (int b = 0; b < batch; b++)
        for (int h = 0; h < num_heads; h++)
            for (int t = 0; t < seq_len; t++) {
                size_t qo = ((size_t)b * seq_len + t) * td + h * head_dim;
                const float *go = d_out + qo;
                const uint16_t *wr = attn_weights + (((size_t)b * num_heads + h) * seq_len + t) * aw;
                int n_p, ls, ll;
                swa_geometry(t, window, n_persistent, &n_p, &ls, &ll);
                float dot_sum = 0.0f;
                for (int s = 0; s < aw; s++) {
                    dw[s] = 0.0f;
                    int valid = s < n_persistent ? s < n_p : (s - n_persistent) < ll;
                    float w = bf16_to_f32(wr[s]);
                    if (valid) {
                        int key = s < n_persistent ? s : ls + (s - n_persistent);
                        size_t ko = ((size_t)b * seq_len + key) * td + h * head_dim;
                        float d = 0.0f;
                        for (int j = 0; j < head_dim; j++) {
                            d_v[ko + j] += w * go[j];
                            d += go[j] * bf16_to_f32(v[ko + j]);
                        }
                        dw[s] = d;
                    }
                    dot_sum += w * dw[s];
                }
                for (int j = 0; j < head_dim; j++) d_q[qo + j] = 0.0f;
                for (int s = 0; s < aw; s++) {
                    int valid = s < n_persistent ? s < n_p : (s - n_persistent) < ll;
                    if (!valid) continue;
                    int key = s < n_persistent ? s : ls + (s - n_persistent);
                    size_t ko = ((size_t)b * seq_len + key) * td + h * head_dim;
                    float w = bf16_to_f32(wr[s]);
                    float ds = w * (dw[s] - dot_sum) * scale;
                    for (int j = 0; j < head_dim; j++) {
                        d_q[qo + j] += ds * bf16_to_f32(k[ko + j]);
                        d_k[ko + j] += ds * bf16_to_f32(q[qo + j]);
                    }
                }
            }
    free(dw);
}
