/* TEST INFRASTRUCTURE ONLY.
 *
 * CPU oracle for the memory-rule kernels: a plain-C restatement of the
 * reference's kernel-level Rust loops (core/src/dispatch.rs:1226-1563) and of
 * the frozen-M0 chunkwise CUDA kernels that have no Rust mirror.  It is the
 * checker for the HIP library, never a fallback for it: only the test-suite,
 * the smoke check and the benchmark's CPU-baseline leg may load this file's
 * shared object.
 *
 * Build:  gcc -O2 -ffp-contract=off -fPIC -shared  (see oracle/Makefile)
 * -O2 mirrors the reference's release profile (core/Cargo.toml:10-11) and
 * -ffp-contract=off keeps the float loops free of fused multiply-adds, as
 * rustc does by default.
 *
 * What pins each function (tests/test_oracle_*.py):
 *   orc_titans_forward / orc_delta_forward : hand-computed known answers
 *       (core/tests/test_dgd.rs:20-72), closed forms (theta=0 decay; one-step
 *       exact store for |k|=1; eta=0 Titans == Delta), an independent numpy
 *       matrix-form implementation, clip/m-norm invariants.
 *   *_backward_range : central finite differences of the double-precision
 *       forward for every input (k, v, q, alpha, theta, eta, M0, S0).
 *   checkpoint / segment schedule : equality with the full-trajectory result
 *       for C in {1,4,8,>=s,non-divisor}; checkpoint_count table
 *       (core/src/gpu_forward.rs:2885-2897).
 *   orc_selfref_*   : finite differences of the double-precision forward for the
 *       input and all six initial memories (as core/src/chunkwise_self_ref.rs:
 *       810-917 does), an independent numpy implementation, frozen-snapshot
 *       property of the self-generated targets (:974-1015), remainder chunk.
 *   orc_chunkwise_* : C=1 equals the exact rule; finite differences of the
 *       chunkwise forward in double precision; numpy matrix form.
 */
#include <float.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define REAL float
#define SFX _f32
#define SQRT sqrtf
#define EXP expf
#define LOG logf
#define TANH tanhf
#define FABS fabsf
#define POW powf
#include "rules.inc"
#include "selfref.inc"
#undef REAL
#undef SFX
#undef SQRT
#undef EXP
#undef LOG
#undef TANH
#undef FABS
#undef POW

#define REAL double
#define SFX _f64
#define SQRT sqrt
#define EXP exp
#define LOG log
#define TANH tanh
#define FABS fabs
#define POW pow
#include "rules.inc"
#include "selfref.inc"
#undef REAL
#undef SFX
#undef SQRT
#undef EXP
#undef LOG
#undef TANH
#undef FABS
#undef POW

/* ── SimpleRng: xorshift64, core/src/tensor.rs:380-408 ──────────────────── */
void orc_simple_rng_fill_uniform(uint64_t seed, float scale, float *buf, int64_t n) {
    uint64_t s = seed ? seed : 1; /* seed.max(1) */
    for (int64_t i = 0; i < n; i++) {
        s ^= s << 13;
        s ^= s >> 7;
        s ^= s << 17;
        double u = (double)s / (double)UINT64_MAX;
        buf[i] = (2.0f * (float)u - 1.0f) * scale;
    }
}

/* checkpoint_count: core/src/gpu_forward.rs:2885-2897 */
int orc_checkpoint_count(int seq_len, int c) {
    int count = 1;
    for (int t = 0; t < seq_len; t++)
        if (((t + 1) % c == 0) || (t + 1 == seq_len)) count++;
    return count;
}

/* ── Batched float wrappers with the kernels' stride contract ────────────
 * Forward: core/kernels/titans_forward.cu:102-113 — token tensors advance by
 * b*input_stride*d, gates by b*input_stride, initial states by b*m_stride,
 * outputs by the local seq_len. */
void orc_titans_forward_batch_f32(const float *k, const float *v, const float *q,
                                  const float *alpha, const float *theta, const float *eta,
                                  const float *m_initial, const float *s_initial,
                                  float *m_states, float *s_states, float *y,
                                  int seq_len, int d, int batch, int input_stride, int m_stride,
                                  float error_clip, float m_norm_max) {
    size_t dd = (size_t)d * d;
    for (int b = 0; b < batch; b++)
        orc_titans_forward_f32(k + (size_t)b * input_stride * d, v + (size_t)b * input_stride * d,
                               q + (size_t)b * input_stride * d, alpha + (size_t)b * input_stride,
                               theta + (size_t)b * input_stride, eta + (size_t)b * input_stride,
                               m_initial + (size_t)b * m_stride, s_initial + (size_t)b * m_stride,
                               m_states + (size_t)b * (seq_len + 1) * dd,
                               s_states + (size_t)b * (seq_len + 1) * dd,
                               y + (size_t)b * seq_len * d, seq_len, d, error_clip, m_norm_max);
}

void orc_delta_forward_batch_f32(const float *k, const float *v, const float *q,
                                 const float *alpha, const float *theta,
                                 const float *m_initial, float *m_states, float *y,
                                 int seq_len, int d, int batch, int input_stride, int m_stride,
                                 float error_clip, float m_norm_max) {
    size_t dd = (size_t)d * d;
    for (int b = 0; b < batch; b++)
        orc_delta_forward_f32(k + (size_t)b * input_stride * d, v + (size_t)b * input_stride * d,
                              q + (size_t)b * input_stride * d, alpha + (size_t)b * input_stride,
                              theta + (size_t)b * input_stride, m_initial + (size_t)b * m_stride,
                              m_states + (size_t)b * (seq_len + 1) * dd,
                              y + (size_t)b * seq_len * d, seq_len, d, error_clip, m_norm_max);
}

/* Backward over the full trajectory; d_m_initial / d_s_initial are SUMMED over
 * the batch into one [dd] buffer that the caller zeroed
 * (core/kernels/titans_backward.cu:337-341, delta_backward.cu atomicAdd). */
void orc_titans_backward_batch_f32(const float *k, const float *v, const float *q,
                                   const float *alpha, const float *theta, const float *eta,
                                   const float *m_states, const float *s_states, const float *d_y,
                                   float *d_k, float *d_v, float *d_q,
                                   float *d_alpha, float *d_theta, float *d_eta,
                                   float *d_m_initial, float *d_s_initial,
                                   int seq_len, int d, int batch, float error_clip) {
    size_t dd = (size_t)d * d, sd = (size_t)seq_len * d;
    float *dm = (float *)malloc(sizeof(float) * dd), *ds = (float *)malloc(sizeof(float) * dd);
    for (int b = 0; b < batch; b++) {
        memset(dm, 0, sizeof(float) * dd);
        memset(ds, 0, sizeof(float) * dd);
        orc_titans_backward_range_f32(k + b * sd, v + b * sd, q + b * sd,
                                      alpha + (size_t)b * seq_len, theta + (size_t)b * seq_len,
                                      eta + (size_t)b * seq_len,
                                      m_states + (size_t)b * (seq_len + 1) * dd,
                                      s_states + (size_t)b * (seq_len + 1) * dd, d_y + b * sd,
                                      d_k + b * sd, d_v + b * sd, d_q + b * sd,
                                      d_alpha + (size_t)b * seq_len, d_theta + (size_t)b * seq_len,
                                      d_eta + (size_t)b * seq_len, dm, ds, 0, seq_len, d, error_clip);
        for (size_t i = 0; i < dd; i++) { d_m_initial[i] += dm[i]; d_s_initial[i] += ds[i]; }
    }
    free(dm); free(ds);
}

void orc_delta_backward_batch_f32(const float *k, const float *v, const float *q,
                                  const float *alpha, const float *theta,
                                  const float *m_states, const float *d_y,
                                  float *d_k, float *d_v, float *d_q,
                                  float *d_alpha, float *d_theta, float *d_m_initial,
                                  int seq_len, int d, int batch, float error_clip) {
    size_t dd = (size_t)d * d, sd = (size_t)seq_len * d;
    float *dm = (float *)malloc(sizeof(float) * dd);
    for (int b = 0; b < batch; b++) {
        memset(dm, 0, sizeof(float) * dd);
        orc_delta_backward_range_f32(k + b * sd, v + b * sd, q + b * sd,
                                     alpha + (size_t)b * seq_len, theta + (size_t)b * seq_len,
                                     m_states + (size_t)b * (seq_len + 1) * dd, d_y + b * sd,
                                     d_k + b * sd, d_v + b * sd, d_q + b * sd,
                                     d_alpha + (size_t)b * seq_len, d_theta + (size_t)b * seq_len,
                                     dm, 0, seq_len, d, error_clip);
        for (size_t i = 0; i < dd; i++) d_m_initial[i] += dm[i];
    }
    free(dm);
}

/* ── Checkpointed forward (one chain): titans_forward_ckpt_kernel,
 * core/kernels/titans_forward.cu:293-390.  Stores M/S at slot 0 and after
 * every token with (t+1)%C==0 or t+1==seq_len; y for every token.
 * has_s=0: delta_forward_ckpt_kernel (delta_forward.cu:280-367). */
void orc_forward_ckpt_f32(const float *k, const float *v, const float *q,
                          const float *alpha, const float *theta, const float *eta,
                          const float *m_initial, const float *s_initial,
                          float *m_ckpt, float *s_ckpt, float *y,
                          int seq_len, int d, int C, int has_s,
                          float error_clip, float m_norm_max) {
    size_t dd = (size_t)d * d;
    float *m = (float *)malloc(sizeof(float) * dd * 2);
    float *s = (float *)calloc(dd * 2, sizeof(float));
    float *yy = (float *)malloc(sizeof(float) * d);
    memcpy(m, m_initial, sizeof(float) * dd);
    memcpy(m_ckpt, m_initial, sizeof(float) * dd);
    if (has_s) { memcpy(s, s_initial, sizeof(float) * dd); memcpy(s_ckpt, s_initial, sizeof(float) * dd); }
    int slot = 1;
    for (int t = 0; t < seq_len; t++) {
        /* one-token step through the full-trajectory routine: states [2*dd] */
        if (has_s)
            orc_titans_forward_f32(k + (size_t)t * d, v + (size_t)t * d, q + (size_t)t * d,
                                   alpha + t, theta + t, eta + t, m, s, m, s, yy, 1, d,
                                   error_clip, m_norm_max);
        else
            orc_delta_forward_f32(k + (size_t)t * d, v + (size_t)t * d, q + (size_t)t * d,
                                  alpha + t, theta + t, m, m, yy, 1, d, error_clip, m_norm_max);
        memcpy(y + (size_t)t * d, yy, sizeof(float) * d);
        memcpy(m, m + dd, sizeof(float) * dd);
        if (has_s) memcpy(s, s + dd, sizeof(float) * dd);
        if (((t + 1) % C == 0) || (t + 1 == seq_len)) {
            memcpy(m_ckpt + (size_t)slot * dd, m, sizeof(float) * dd);
            if (has_s) memcpy(s_ckpt + (size_t)slot * dd, s, sizeof(float) * dd);
            slot++;
        }
    }
    free(m); free(s); free(yy);
}

/* ── Checkpointed backward (one chain): the segment schedule of
 * titans_backward_checkpointed / delta_backward_checkpointed
 * (core/src/gpu_backward.rs:1770-1962): for each C-token segment in reverse,
 * replay the forward from the segment's checkpoint into a local trajectory,
 * run the segment backward seeded with d_M/d_S from the later segment.
 * d_m / d_s: zero on entry, gradient w.r.t. the initial states on exit. */
void orc_backward_ckpt_f32(const float *k, const float *v, const float *q,
                           const float *alpha, const float *theta, const float *eta,
                           const float *m_ckpt, const float *s_ckpt, const float *d_y,
                           float *d_k, float *d_v, float *d_q,
                           float *d_alpha, float *d_theta, float *d_eta,
                           float *d_m, float *d_s,
                           int seq_len, int d, int C, int has_s,
                           float error_clip, float m_norm_max) {
    size_t dd = (size_t)d * d;
    int max_seg = C < seq_len ? C : seq_len;
    float *lm = (float *)malloc(sizeof(float) * dd * (max_seg + 1));
    float *ls = (float *)malloc(sizeof(float) * dd * (max_seg + 1));
    float *ly = (float *)malloc(sizeof(float) * (size_t)max_seg * d);
    int nseg = (seq_len + C - 1) / C;
    for (int g = nseg - 1; g >= 0; g--) {
        int t0 = g * C, t1 = t0 + C < seq_len ? t0 + C : seq_len;
        if (has_s) {
            orc_titans_forward_f32(k + (size_t)t0 * d, v + (size_t)t0 * d, q + (size_t)t0 * d,
                                   alpha + t0, theta + t0, eta + t0,
                                   m_ckpt + (size_t)g * dd, s_ckpt + (size_t)g * dd,
                                   lm, ls, ly, t1 - t0, d, error_clip, m_norm_max);
            orc_titans_backward_range_f32(k, v, q, alpha, theta, eta, lm, ls, d_y,
                                          d_k, d_v, d_q, d_alpha, d_theta, d_eta, d_m, d_s,
                                          t0, t1, d, error_clip);
        } else {
            orc_delta_forward_f32(k + (size_t)t0 * d, v + (size_t)t0 * d, q + (size_t)t0 * d,
                                  alpha + t0, theta + t0, m_ckpt + (size_t)g * dd,
                                  lm, ly, t1 - t0, d, error_clip, m_norm_max);
            orc_delta_backward_range_f32(k, v, q, alpha, theta, lm, d_y,
                                         d_k, d_v, d_q, d_alpha, d_theta, d_m,
                                         t0, t1, d, error_clip);
        }
    }
    free(lm); free(ls); free(ly);
}
