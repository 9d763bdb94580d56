/* nl_hecate_rocm — C ABI of the MI355X (gfx950) memory-rule kernel library.
 *
 * Drop-in boundary: every function whose name ends in `_cuda` has exactly the
 * name, argument order, argument types and buffer layout of the `extern "C"`
 * declaration in the reference's core/src/cuda_ffi.rs (line cited per
 * function), so a `rocm` cargo feature can bind this library with the same
 * Rust declarations.  Functions ending in `_rocm` and `nlh_*` are additions
 * with no reference symbol.
 *
 * Conventions (core/src/cuda_ffi.rs, the .cu files under core/kernels):
 *   - all pointers are device memory owned by the caller; row-major; f32 unless
 *     stated; bf16 travels as uint16_t; sizes are int.
 *   - no stream argument: work is enqueued on the null stream (or the stream
 *     given to nlh_set_stream) and is asynchronous; the caller synchronises.
 *   - void functions report a bad argument or a failed launch by printing a
 *     message and abort()ing, like the reference; nlh_set_error_mode(1) turns
 *     that into a recorded error (nlh_last_error) and an early return.
 *   - chain = one (batch, head) pair; `batch_size` counts chains.
 */
#ifndef NL_HECATE_FFI_H
#define NL_HECATE_FFI_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ── library control (no reference counterpart) ─────────────────────────── */
const char *nlh_version(void);
void nlh_set_error_mode(int mode);     /* 0 = abort (reference behaviour), 1 = record */
const char *nlh_last_error(void);      /* "" when no error is recorded */
void nlh_clear_error(void);
void nlh_set_stream(void *hip_stream); /* hipStream_t; NULL = null stream */
void nlh_release_workspace(void);      /* frees the library's device scratch */
/* Bumped whenever a scratch buffer is freed (a slot grew, or nlh_release_workspace
 * ran).  A HIP graph captured from calls into this library holds scratch addresses:
 * record the value at capture, and when it has changed drop the graph and capture
 * again instead of replaying it.  A slot never grows while the launch stream is
 * being captured: such a call fails with a message instead. */
unsigned long long nlh_workspace_generation(void);
/* hipEvent pair on the launch stream: start, then stop returns elapsed ms
 * (blocks until the stop event completes); negative on failure. */
int nlh_timer_start(void);
float nlh_timer_stop_ms(void);
/* Per-kernel timing: while enabled, every launch of the kernels the library instruments (those
 * of the memory-rule entry points) is bracketed by an event pair on the launch stream (at most
 * 256 between reads).  read_ms waits for them, returns their summed duration, the launch count
 * and the name of the last kernel, and resets.  report writes "name:launches:total_ms;" per
 * kernel name into buf, returns the number of names (< 0 on error) and resets. */
int nlh_kernel_timer_enable(int on);
float nlh_kernel_timer_read_ms(int *launches, char *name, int name_len);
int nlh_kernel_timer_report(char *buf, int buf_len);
/* Which form the checkpointed backward of the exact rules takes where several apply (see
 * titans_backward_ckpt_f32_rocm): 0 = by the cost model (default), 1 = the matrix form wherever it applies,
 * 2 = never the matrix form.  Returns the previous setting.  No counterpart in the reference; for tests and tuning. */
int nlh_exact_backward_form(int mode);
/* Runs the cross-lane primitives on known data; returns 0 when all agree. */
int nlh_selftest_lane_ops(void);
/* Gate coefficients of one chunk (L <= 64 device-resident gates each) from the in-kernel generator:
 * tj, jt [3][64][64] = c, bb, r indexed [t][j] from the two tile orders; vecs [9][64] = a, beta, h,
 * cl, bl, rl, keep, eta, theta, then a_L, beta_L, h_L.  0 on success.  For tests. */
int nlh_selftest_chunk_coef(const float *alpha, const float *theta, const float *eta, int L, float *tj,
                            float *jt, float *vecs);
/* The same chunk through the helpers of the coefficient pre-passes (scans for the vectors, per-lane column walk for
 * the table): table [64][64] = c[t][j], table_scaled = -theta_j c[t][j] (both zero outside j <= t < L);
 * vecs [5][64] = a, beta, h of G(0..t) and cl, bl of G(t+1..63).  0 on success.  For tests. */
int nlh_selftest_chunk_coef_prepass(const float *alpha, const float *theta, const float *eta, int L, float *table,
                                    float *table_scaled, float *vecs);

/* ── Titans LMM, exact per-token rule ───────────────────────────────────────
 * Per token: e = clip(M k - v); S = eta S - theta e k^T; M = (1-alpha) M + S;
 * M projected to |M|_F <= m_norm_max; y = M q.
 * k,v,q [batch, seq_len, d]; gates [batch, seq_len]; chain b reads tokens at
 * b*input_stride*d (gates at b*input_stride) and initial states at b*m_stride;
 * outputs use the local seq_len: y [batch, seq_len, d],
 * m_states / s_states [batch, seq_len+1, d*d].
 * error_clip <= 0 and m_norm_max <= 0 or >= 1e30 disable clip / projection. */
/* core/src/cuda_ffi.rs:134 */
void titans_forward_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem,
                             const float *alpha, const float *theta, const float *eta,
                             const float *m_initial, const float *s_initial,
                             float *m_states, float *s_states, float *y,
                             int seq_len, int d, int batch_size, int input_stride, int m_stride,
                             float error_clip, float m_norm_max);
/* core/src/cuda_ffi.rs:156.  d_m_initial / d_s_initial [d*d] are ACCUMULATED
 * (+=) with the sum over the batch; the caller zeroes them. */
void titans_backward_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem,
                              const float *alpha, const float *theta, const float *eta,
                              const float *m_states, const float *s_states, const float *d_y,
                              float *d_k_mem, float *d_v_mem, float *d_q_mem,
                              float *d_alpha, float *d_theta, float *d_eta,
                              float *d_m_initial, float *d_s_initial,
                              int seq_len, int d, int batch_size, float error_clip);
/* No counterpart in the reference.  titans_backward_f32_cuda for callers that
 * cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): same arguments, same kernels, same
 * results to 1e-4, but its work buffers (per-chain dM / dS [batch, d*d] each,
 * and for d = 128 the partial sums of a chain's four workgroups,
 * 4*batch*seq_len*(2d+4) floats) live in a fixed 8 MiB device array inside the
 * library, so the call makes no hipMalloc / hipFree.  d in {8,16,32,64,128};
 * 2*batch*d*d (+ partial sums) must not exceed 2 097 152 floats (256 chains at
 * d = 64), otherwise the call fails with a message and launches nothing.
 * Every call on a GPU uses that GPU's one array: calls that overlap on one
 * GPU (two streams, two threads) race. */
void titans_backward_noalloc_f32_rocm(const float *k_mem, const float *v_mem, const float *q_mem,
                                      const float *alpha, const float *theta, const float *eta,
                                      const float *m_states, const float *s_states, const float *d_y,
                                      float *d_k_mem, float *d_v_mem, float *d_q_mem,
                                      float *d_alpha, float *d_theta, float *d_eta,
                                      float *d_m_initial, float *d_s_initial,
                                      int seq_len, int d, int batch_size, float error_clip);
/* core/src/cuda_ffi.rs:230.  One chain; stores M/S at slot 0 and after every
 * token with (t+1)%C==0 or t+1==seq_len. */
void titans_forward_ckpt_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem,
                                  const float *alpha, const float *theta, const float *eta,
                                  const float *m_initial, const float *s_initial,
                                  float *m_states, float *s_states, float *y,
                                  int seq_len, int d, int checkpoint_interval, float error_clip,
                                  float m_norm_max);
/* core/src/cuda_ffi.rs:262.  Tokens [t_start, t_end); token tensors are
 * indexed by absolute t with stride seq_len; m_states / s_states are the
 * segment-local trajectory [batch, t_end-t_start+1, d*d]; seeds and outs are
 * [batch, d*d] (not summed over the batch). */
void titans_backward_segment_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem,
                                      const float *alpha, const float *theta, const float *eta,
                                      const float *m_states, const float *s_states, const float *d_y,
                                      const float *d_m_seed, const float *d_s_seed,
                                      float *d_k_mem, float *d_v_mem, float *d_q_mem,
                                      float *d_alpha, float *d_theta, float *d_eta,
                                      float *d_m_out, float *d_s_out,
                                      int t_start, int t_end, int d, int batch_size, int seq_len,
                                      float error_clip);

/* ── Hebbian rule: M <- (1 - alpha) M + v k^T.  d = 8, 16, 32, 64, 128 on tiled kernels, every other d from 1 to
 * 3840 on general ones (the reference runs these at d = 2048, core/tests/test_cuda_large_d.rs:353) ─────────── */
/* core/src/cuda_ffi.rs:186 */
void hebbian_forward_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem,
                              const float *alpha, const float *m_initial,
                              float *m_states, float *y, int seq_len, int d, int batch_size,
                              int input_stride, int m_stride);
/* core/src/cuda_ffi.rs:202 (one chain; d_m_initial is overwritten) */
void hebbian_backward_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem,
                               const float *alpha, const float *m_states, const float *d_y,
                               float *d_k_mem, float *d_v_mem, float *d_q_mem,
                               float *d_alpha, float *d_m_initial, int seq_len, int d);
/* core/src/cuda_ffi.rs:240 (one chain) */
void hebbian_forward_ckpt_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem,
                                   const float *alpha, const float *m_initial,
                                   float *m_states, float *y,
                                   int seq_len, int d, int checkpoint_interval);
/* core/src/cuda_ffi.rs:275 */
void hebbian_backward_segment_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem,
                                       const float *alpha, const float *m_states, const float *d_y,
                                       const float *d_m_seed,
                                       float *d_k_mem, float *d_v_mem, float *d_q_mem,
                                       float *d_alpha, float *d_m_out,
                                       int t_start, int t_end, int d, int batch_size, int seq_len);

/* ── Delta rule (Titans without momentum) ────────────────────────────────── */
/* core/src/cuda_ffi.rs:86 */
void delta_forward_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem,
                            const float *alpha, const float *theta, const float *m_initial,
                            float *m_states, float *y, int seq_len, int d, int batch_size,
                            int input_stride, int m_stride, float error_clip, float m_norm_max);
/* core/src/cuda_ffi.rs:109 */
void delta_backward_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem,
                             const float *alpha, const float *theta,
                             const float *m_states, const float *d_y,
                             float *d_k_mem, float *d_v_mem, float *d_q_mem,
                             float *d_alpha, float *d_theta, float *d_m_initial,
                             int seq_len, int d, int batch_size, float error_clip);
/* core/src/cuda_ffi.rs:221 */
void delta_forward_ckpt_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem,
                                 const float *alpha, const float *theta, const float *m_initial,
                                 float *m_states, float *y, int seq_len, int d,
                                 int checkpoint_interval, float error_clip, float m_norm_max);
/* core/src/cuda_ffi.rs:250 */
void delta_backward_segment_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem,
                                     const float *alpha, const float *theta,
                                     const float *m_states, const float *d_y, const float *d_m_seed,
                                     float *d_k_mem, float *d_v_mem, float *d_q_mem,
                                     float *d_alpha, float *d_theta, float *d_m_out,
                                     int t_start, int t_end, int d, int batch_size, int seq_len,
                                     float error_clip);

/* ── DGD: same update as Delta, no projection (core/kernels/dgd_forward.cu:6-11) */
/* core/src/cuda_ffi.rs:291 */
void dgd_forward_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem,
                          const float *alpha, const float *theta, const float *m_initial,
                          float *m_states, float *y, int seq_len, int d, int batch_size,
                          int input_stride, int m_stride, float error_clip);
/* core/src/cuda_ffi.rs:309 (single chain: no batch argument) */
void dgd_backward_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem,
                           const float *alpha, const float *theta,
                           const float *m_states, const float *d_y,
                           float *d_k_mem, float *d_v_mem, float *d_q_mem,
                           float *d_alpha, float *d_theta, float *d_m_initial,
                           int seq_len, int d, float error_clip);
/* core/src/cuda_ffi.rs:329 */
void dgd_forward_ckpt_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem,
                               const float *alpha, const float *theta, const float *m_initial,
                               float *m_states, float *y, int seq_len, int d,
                               int checkpoint_interval, float error_clip);
/* core/src/cuda_ffi.rs:337 */
void dgd_backward_segment_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem,
                                   const float *alpha, const float *theta,
                                   const float *m_states, const float *d_y, const float *d_m_seed,
                                   float *d_k_mem, float *d_v_mem, float *d_q_mem,
                                   float *d_alpha, float *d_theta, float *d_m_out,
                                   int t_start, int t_end, int d, int batch_size, int seq_len,
                                   float error_clip);

/* ── Frozen-M0 chunkwise rule ────────────────────────────────────────────────
 * Errors of a chunk are taken against the chunk-start M; S/M then evolve per
 * token and y reads the evolving M.  m_chunk_states / s_chunk_states
 * [batch, num_chunks+1, d*d]: slot 0 = initial, slot c+1 = end of chunk c.
 * Backward: d_M propagates by retention only, the error path goes to the
 * chunk-start M (core/kernels/titans_chunkwise_backward.cu). */
/* core/src/cuda_ffi.rs:376 */
void titans_chunkwise_forward_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem,
                                       const float *alpha, const float *theta, const float *eta,
                                       const float *m_initial, const float *s_initial,
                                       float *m_chunk_states, float *s_chunk_states, float *y,
                                       int seq_len, int d, int batch_size, int chunk_size,
                                       float error_clip, float m_norm_max);
/* core/src/cuda_ffi.rs:386 */
void titans_chunkwise_backward_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem,
                                        const float *alpha, const float *theta, const float *eta,
                                        const float *m_chunk_states, const float *s_chunk_states,
                                        const float *d_y,
                                        float *d_k_mem, float *d_v_mem, float *d_q_mem,
                                        float *d_alpha, float *d_theta, float *d_eta,
                                        float *d_m_initial, float *d_s_initial,
                                        int seq_len, int d, int batch_size, int chunk_size,
                                        float error_clip, float m_norm_max);
/* core/src/cuda_ffi.rs:356 */
void delta_chunkwise_forward_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem,
                                      const float *alpha, const float *theta, const float *m_initial,
                                      float *m_chunk_states, float *y,
                                      int seq_len, int d, int batch_size, int chunk_size,
                                      float error_clip, float m_norm_max);
/* core/src/cuda_ffi.rs:365 */
void delta_chunkwise_backward_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem,
                                       const float *alpha, const float *theta,
                                       const float *m_chunk_states, const float *d_y,
                                       float *d_k_mem, float *d_v_mem, float *d_q_mem,
                                       float *d_alpha, float *d_theta, float *d_m_initial,
                                       int seq_len, int d, int batch_size, int chunk_size,
                                       float error_clip, float m_norm_max);

/* ── Batched checkpointed forward (addition) ────────────────────────────────
 * The reference loops the single-chain *_forward_ckpt over heads
 * (core/src/gpu_forward.rs:1611-1662); these take all chains in one launch.
 * m_ckpt / s_ckpt [batch, n_ckpt, d*d], n_ckpt = checkpoint_count(seq_len, C)
 * (core/src/gpu_forward.rs:2885-2897); inputs are dense [batch, seq_len, ...]. */
void titans_forward_ckpt_batched_f32_rocm(const float *k_mem, const float *v_mem, const float *q_mem,
                                          const float *alpha, const float *theta, const float *eta,
                                          const float *m_initial, const float *s_initial,
                                          float *m_ckpt, float *s_ckpt, float *y,
                                          int seq_len, int d, int batch_size, int checkpoint_interval,
                                          float error_clip, float m_norm_max);
void delta_forward_ckpt_batched_f32_rocm(const float *k_mem, const float *v_mem, const float *q_mem,
                                         const float *alpha, const float *theta,
                                         const float *m_initial, float *m_ckpt, float *y,
                                         int seq_len, int d, int batch_size, int checkpoint_interval,
                                         float error_clip, float m_norm_max);


/* ── Checkpointed backward (addition) ───────────────────────────────────────
 * Replaces the host loop titans_backward_checkpointed /
 * delta_backward_checkpointed (core/src/gpu_backward.rs:1770-1962): one call
 * walks the C-token segments in reverse.  m_ckpt / s_ckpt are the output of
 * the batched checkpointed forward; gradients have the layout of
 * *_backward_f32_cuda, including the accumulate-over-batch contract of
 * d_m_initial / d_s_initial.
 * `_replay_`: replays every segment through a scratch trajectory in device
 * memory, the reference's schedule without its host synchronisations. */
void titans_backward_ckpt_replay_f32_rocm(const float *k_mem, const float *v_mem, const float *q_mem,
                                          const float *alpha, const float *theta, const float *eta,
                                          const float *m_ckpt, const float *s_ckpt, const float *d_y,
                                          float *d_k_mem, float *d_v_mem, float *d_q_mem,
                                          float *d_alpha, float *d_theta, float *d_eta,
                                          float *d_m_initial, float *d_s_initial,
                                          int seq_len, int d, int batch_size, int checkpoint_interval,
                                          float error_clip, float m_norm_max);
void delta_backward_ckpt_replay_f32_rocm(const float *k_mem, const float *v_mem, const float *q_mem,
                                         const float *alpha, const float *theta,
                                         const float *m_ckpt, const float *d_y,
                                         float *d_k_mem, float *d_v_mem, float *d_q_mem,
                                         float *d_alpha, float *d_theta, float *d_m_initial,
                                         int seq_len, int d, int batch_size, int checkpoint_interval,
                                         float error_clip, float m_norm_max);
/* One call over all segments (the loop of core/src/gpu_backward.rs:1770-1962 inside the library).  Three forms, chosen
 * per call: (1) head size 64, checkpoint_interval <= 64: the rule in chunk-parallel matrix form on the fp32 matrix
 * cores (a triangular solve per segment, an adjoint scan over the segments, gradients per segment), taken where a cost
 * model says it beats (2) at the call's shape (long intervals, or few chains); (2) the fused form: the replayed
 * trajectory stays in LDS and registers (two-level recomputation inside one kernel), checkpoint_interval <= 64;
 * (3) the `_replay_` schedule.  With a finite m_norm_max (1) and (2) end with a device-side test that the bound
 * could not have been reached and leave the call to (3) when it could; with an error clip (1) does the same and
 * (2) is not used. */
void titans_backward_ckpt_f32_rocm(const float *k_mem, const float *v_mem, const float *q_mem,
                                   const float *alpha, const float *theta, const float *eta,
                                   const float *m_ckpt, const float *s_ckpt, const float *d_y,
                                   float *d_k_mem, float *d_v_mem, float *d_q_mem,
                                   float *d_alpha, float *d_theta, float *d_eta,
                                   float *d_m_initial, float *d_s_initial,
                                   int seq_len, int d, int batch_size, int checkpoint_interval,
                                   float error_clip, float m_norm_max);
void delta_backward_ckpt_f32_rocm(const float *k_mem, const float *v_mem, const float *q_mem,
                                  const float *alpha, const float *theta,
                                  const float *m_ckpt, const float *d_y,
                                  float *d_k_mem, float *d_v_mem, float *d_q_mem,
                                  float *d_alpha, float *d_theta, float *d_m_initial,
                                  int seq_len, int d, int batch_size, int checkpoint_interval,
                                  float error_clip, float m_norm_max);

/* ── Glue either side of the memory rules ───────────────────────────────────
 * Elementwise kernels take n elements; all are asynchronous. */
/* core/src/cuda_ffi.rs:552 */
void sigmoid_cuda(const float *x, float *out, int n);
/* core/kernels/elementwise.cu:47 (softplus, identity above 20; not in cuda_ffi.rs) */
void softplus_cuda(const float *x, float *out, int n);
/* core/src/cuda_ffi.rs:555 */
void elemwise_mul_cuda(const float *a, const float *b, float *out, int n);
/* core/src/cuda_ffi.rs:558: d_a = d_out*b, d_b = d_out*a */
void gating_backward_cuda(const float *d_out, const float *a, const float *b, float *d_a, float *d_b, int n);
/* core/src/cuda_ffi.rs:564: d_x = d_gate*gate*(1-gate) */
void sigmoid_backward_cuda(const float *d_gate, const float *gate, float *d_x, int n);
/* core/src/cuda_ffi.rs:569 / 572: round-to-nearest-even */
void f32_to_bf16_cuda(const float *src, uint16_t *dst, int n);
void bf16_to_f32_cuda(const uint16_t *src, float *dst, int n);
/* Operand packing for a split-bf16 GEMM (no counterpart in the reference, whose projections are
 * fp32 cuBLAS calls): row r of out [n, 3*count*d] = [hi(src0..) | lo(src0..) | hi(src0..)] with
 * x = hi + lo, hi = bf16(x), lo = bf16(x - hi); srcs: count (1..4) host-side pointers to [n, d] floats. */
void split_pack_bf16_rocm(const float *const *srcs, int count, uint16_t *out, long long n, int d);
/* core/src/cuda_ffi.rs:579: gate[t] = act(k_t.w[:d] + v_t.w[d:] + *bias_ptr);
 * activation 0 = sigmoid, 1 = softplus (identity above 20) */
void gate_compute_cuda(const float *k_mem, const float *v_mem, const float *w_gate,
                       const float *bias_ptr, float *gate_out, int seq_len, int d, int activation);
/* core/src/cuda_ffi.rs:587 / 591 */
void clamp_f32_cuda(float *inout, int n, float lo, float hi);
void theta_clamp_mask_cuda(const float *theta, float *d_theta, int n, float lo, float hi);
/* core/src/cuda_ffi.rs:599: d_w / d_b of the gate projections from the cached
 * gate OUTPUTS (sigmoid' = a(1-a), softplus' = 1-exp(-theta)); outputs are
 * overwritten. */
void gate_backward_cuda(const float *d_alpha, const float *alpha, const float *d_theta,
                        const float *theta, const float *d_eta, const float *eta,
                        const float *k_mem, const float *v_mem,
                        float *d_w_alpha, float *d_b_alpha, float *d_w_theta, float *d_b_theta,
                        float *d_w_eta, float *d_b_eta, int T, int D, int has_theta, int has_eta);
/* core/src/cuda_ffi.rs:611: y += alpha*x */
void saxpy_cuda(float alpha, const float *x, float *y, int n);
/* core/src/cuda_ffi.rs:507 / 514: rows normalised in place, norms = pre-normalisation L2 norms */
void l2_normalize_rows_f32_cuda(float *x, float *norms, int n_rows, int d, float eps);
void l2_normalize_backward_f32_cuda(const float *d_out, const float *x_norm, const float *norms,
                                    float *d_in, int n_rows, int d, float eps);
/* core/src/cuda_ffi.rs:1035: [bs,s,nh*hd] -> [bs*nh,s,hd] (forward=1) or back (0) */
void transpose_heads_f32_cuda(const float *input, float *output, int bs, int s, int nh, int hd, int forward);
/* core/src/cuda_ffi.rs:1043 / 1051: [bs,s] -> [bs*nh,s] and its adjoint */
void broadcast_heads_f32_cuda(const float *input, float *output, int bs, int s, int nh);
void sum_heads_f32_cuda(const float *input, float *output, int bs, int s, int nh);
/* core/src/cuda_ffi.rs:458: dst[b, t, :] = src[b, :]; returns 0 / 1 (overflow) / 2 (launch) */
int broadcast_fill_f32_cuda(float *dst, const float *src, int dd, int n_slots, int n_batch);
/* core/src/cuda_ffi.rs:467 / 471: Frobenius clamp, no-op for max <= 0 or >= 1e30 */
void m_norm_clamp_f32_cuda(float *m, int d, float m_norm_max);
void m_norm_clamp_batch_f32_cuda(float *m, int d, int batch_size, float m_norm_max);
/* core/src/cuda_ffi.rs:478: norm_out[0] = |M k - v|_2 */
void dgd_delta_norm_cuda(const float *m, const float *k, const float *v, float *norm_out, int d);

/* ── Sliding-window attention (bf16 storage as uint16_t, f32 math) ──────────
 * q,k,v,out [batch, seq, heads*hd]; attn_weights [batch, heads, seq,
 * n_persistent + window].  Query t sees prefix keys [0, min(t+1, n_persistent))
 * (slot = key) and local keys [ls, t], ls = max(t+1-window, n_persistent)
 * (slot = n_persistent + key - ls); unused slots are written as 0. */
/* core/src/cuda_ffi.rs:26 */
void swa_forward_f32_cuda(const uint16_t *q, const uint16_t *k, const uint16_t *v, uint16_t *out,
                          uint16_t *attn_weights, int seq_len, int num_heads, int head_dim,
                          int window_size, int batch_size, int n_persistent);
/* core/src/cuda_ffi.rs:62.  d_q is overwritten; d_k and d_v are ACCUMULATED
 * (+=) into caller-zeroed buffers.  Differentiates through the stored weights. */
void swa_backward_f32_cuda(const uint16_t *q, const uint16_t *k, const uint16_t *v,
                           const uint16_t *attn_weights, const float *d_attn_out,
                           float *d_q, float *d_k, float *d_v, int seq_len, int num_heads, int head_dim,
                           int window_size, int batch_size, int n_persistent);

/* No counterpart in the reference (its backward, core/src/cuda_ffi.rs:62, reads the weight tensor the forward
 * stored): the same attention with the weight tensor left out.  The forward stores per query only
 * stats [batch, heads, seq, 2] fp32 = (max_j score * log2(e) / sqrt(hd), 1 / sum_j exp(...)); the backward rebuilds
 * each weight from q . k and those two numbers, rounded to bf16 as the stored tensor would hold it.
 * head_dim 64 or 32, window_size <= 512, no persistent prefix; other shapes are an error.  out, d_q, d_k, d_v as in
 * the pair above (d_k, d_v accumulated). */
void swa_forward_lse_bf16_rocm(const uint16_t *q, const uint16_t *k, const uint16_t *v, uint16_t *out, float *stats,
                               int seq_len, int num_heads, int head_dim, int window_size, int batch_size);
void swa_backward_lse_bf16_rocm(const uint16_t *q, const uint16_t *k, const uint16_t *v, const float *stats,
                                const float *d_attn_out, float *d_q, float *d_k, float *d_v, int seq_len,
                                int num_heads, int head_dim, int window_size, int batch_size);
/* The same backward with the three gradients written (not accumulated) as bf16 into columns of a wider row-major
 * matrix: g_q, g_k, g_v point at the first row's columns, ld is the row stride in elements.  No counterpart in the
 * reference: for a caller whose next step is a bf16 GEMM over those columns (the level step's projection gradients). */
void swa_backward_lse_bf16_cols_rocm(const uint16_t *q, const uint16_t *k, const uint16_t *v, const float *stats,
                                     const float *d_attn_out, uint16_t *g_q, uint16_t *g_k, uint16_t *g_v, long long ld,
                                     int seq_len, int num_heads, int head_dim, int window_size, int batch_size);

/* ── AdamW and gradient clipping; return hipError_t as unsigned, 0 = success ─ */
/* core/src/cuda_ffi.rs:674 */
unsigned adamw_update_cuda(float *w, const float *g, float *m, float *v, int n, float lr, float beta1,
                           float beta2, float eps, float bc1_inv, float bc2_inv, float weight_decay);
/* core/src/cuda_ffi.rs:686 / 693: ceil(n/256) partial sums, one per 256
 * elements; *out_num_blocks (host) receives that count */
unsigned grad_norm_sq_cuda(const float *g, float *partial_sums, int n, int *out_num_blocks);
unsigned dot_product_partial_f32_cuda(const float *a, const float *b, float *partial_sums, int n,
                                      int *out_num_blocks);
/* core/src/cuda_ffi.rs:700 */
unsigned grad_scale_cuda(float *g, float scale, int n);
/* core/src/cuda_ffi.rs:706: out_norm = sqrt(sum), out_scale = min(1, max/norm) on device */
unsigned reduce_partials_clip_cuda(const float *partial_sums, int total_partials, float max_grad_norm,
                                   float *out_norm, float *out_scale);
/* core/src/cuda_ffi.rs:714: g *= *scale_ptr unless it is >= 1 */
unsigned grad_scale_conditional_cuda(float *g, const float *scale_ptr, int n);
/* Additions: every tensor of a step in one launch.  The pointer / size /
 * bias-correction arrays are HOST arrays of `count` entries (device pointers
 * inside); replaces the per-tensor loop of core/src/gpu_optimizer.rs:403-515
 * and the partial-sum pipeline of core/src/gpu_stacked_optimizer.rs:193. */
unsigned adamw_update_multi_rocm(float *const *w, const float *const *g, float *const *m, float *const *v,
                                 const int *n, const float *bc1_inv, const float *bc2_inv, int count,
                                 float lr, float beta1, float beta2, float eps, float weight_decay);
unsigned grad_norm_clip_multi_rocm(float *const *g, const int *n, int count, float max_grad_norm,
                                   float *out_norm, float *out_scale);

/* ── CMS Conductor / Pulse and level dispatch (additions) ───────────────────
 * Host-side state machines that the reference keeps in Rust; here behind the
 * C ABI so that the level loop, the optimizer gating and the MAG combine are
 * one library. */
typedef struct nlh_conductor nlh_conductor;
typedef struct nlh_adamw nlh_adamw;

/* core/src/conductor.rs:47-55 Conductor::new (k levels, 1 <= k <= 8) */
nlh_conductor *nlh_conductor_new(int k, const long long *chunk_sizes);
void nlh_conductor_free(nlh_conductor *c);
/* core/src/conductor.rs:61 set_seq_len */
void nlh_conductor_set_seq_len(nlh_conductor *c, long long seq_len);
/* core/src/conductor.rs:136-144 pulse: level l is active iff step % chunk_sizes[l] == 0
 * or seq_len >= chunk_sizes[l] > 0.  active[k] receives 0/1; returns the
 * bitmask of core/src/gpu_forward.rs:2449 pulse_to_bitmask. */
unsigned nlh_conductor_pulse(const nlh_conductor *c, int *active);
/* core/src/conductor.rs:147 advance, :152 step */
void nlh_conductor_advance(nlh_conductor *c);
long long nlh_conductor_step(const nlh_conductor *c);
unsigned nlh_pulse_to_bitmask(const int *active, int k);
/* core/src/conductor.rs:105-128 restore: 0 ok, 1 config mismatch, 2 pulse mismatch */
int nlh_conductor_restore(nlh_conductor *c, int k, const long long *chunk_sizes, long long step,
                          long long stream_pulse_id);

/* ErrorBuffer of one frozen CMS level (core/src/conductor.rs:224-261): the outer-loop gradients a level
 * receives while it does not fire are summed and applied as one plain gradient step when it fires.
 * The accumulators are caller-owned device buffers, one per parameter tensor of the level (zeroed by
 * the caller), registered in a fixed order; `level_grads`, `params` and `single_step_grads` are host
 * arrays of device pointers in that order.
 *   accumulate       (:240-243): acc_i += grad_i for every tensor (one launch), steps_accumulated += 1
 *   apply_and_reset  (:246-252): if steps_accumulated > 0: param_i -= lr * acc_i, acc_i = 0, counter = 0
 *   health_check     (:256-261): *ratio = ||acc|| / ||single_step||; returns 1, or 0 (None) when the
 *                    single-step norm is below 1e-12, < 0 on error; synchronises the launch stream */
typedef struct nlh_error_buffer nlh_error_buffer;
nlh_error_buffer *nlh_error_buffer_new(void);
void nlh_error_buffer_free(nlh_error_buffer *b);
int nlh_error_buffer_add_tensor(nlh_error_buffer *b, float *accumulator, int n);
long long nlh_error_buffer_steps(const nlh_error_buffer *b);
void nlh_error_buffer_accumulate(nlh_error_buffer *b, const float *const *level_grads);
void nlh_error_buffer_apply_and_reset(nlh_error_buffer *b, float *const *params, float lr);
int nlh_error_buffer_health_check(const nlh_error_buffer *b, const float *const *single_step_grads, float *ratio);
/* ContextState (core/src/conductor.rs:156-221): the memories that persist across forward calls are
 * caller-owned device buffers.
 *   reset (:212-219): zero every buffer (per-level M, S and the self-referential memories) with one fill
 *         launch (no memset node, so the call may be captured); the Conductor's step is not touched
 *   seed_self_ref (:194-207): copy a level's m_*_init parameters into every chain of a
 *         [batch, 6, d*d] block of self-referential memories (order m_k, m_v, m_q, m_eta, m_alpha,
 *         m_mem): the five projection memories when m_k_init is non-null (all five are then required),
 *         m_mem when m_mem_init is non-null; a null pointer stands for the reference's empty vector */
void nlh_context_state_reset(float *const *buffers, const int *n, int count);
void nlh_context_state_seed_self_ref(float *mems, const float *m_k_init, const float *m_v_init, const float *m_q_init,
                                     const float *m_eta_init, const float *m_alpha_init, const float *m_mem_init,
                                     int batch, int d);
/* Frequency-aware AdamW (core/src/adamw.rs, core/src/gpu_optimizer.rs:403-515):
 * group -1 tensors update every step with the global step's bias correction;
 * group l tensors update only when level l's pulse is on, with that level's
 * own step counter.  w/g/m/v are device buffers owned by the caller. */
nlh_adamw *nlh_adamw_new(int k, float beta1, float beta2, float eps, float weight_decay);
void nlh_adamw_free(nlh_adamw *o);
int nlh_adamw_add_tensor(nlh_adamw *o, int group, float *w, float *g, float *m, float *v, int n);
void nlh_adamw_set_clamp(nlh_adamw *o, int tensor, float lo, float hi);
/* norm_scale: device buffer of 2 floats {pre-clip norm, applied scale}; may be
 * NULL when max_grad_norm <= 0.  Returns 0 on success. */
unsigned nlh_adamw_step(nlh_adamw *o, const int *active_levels, float lr, float max_grad_norm,
                        float *norm_scale);
unsigned nlh_adamw_swa_step(const nlh_adamw *o);
unsigned nlh_adamw_level_step(const nlh_adamw *o, int level);

/* Level combine + MAG sigmoid gate (core/src/gpu_forward.rs:1027-1070):
 * gate = sigmoid(c * sum_l y_l), gated = attn_out * gate, c = 1/sqrt(k) if k > 2.
 * y_levels: HOST array of k device pointers; y_combined may be NULL. */
void cms_combine_gate_rocm(const float *const *y_levels, int k, const float *attn_out,
                           float *y_combined, float *gate, float *gated, long long n);
/* core/src/gpu_backward.rs:263-283 */
void cms_gate_backward_rocm(const float *d_gated, const float *attn_out, const float *gate, int k,
                            float *d_attn, float *d_y_combined, long long n);
/* Frozen level (core/src/gpu_forward.rs:2906-2950): y = M_h q per head, token-major */
void memory_read_only_f32_rocm(const float *q_mem, const float *m, float *y, long long n_tokens, int nh,
                               int hd);
/* Backward of that read (core/src/opaque_adapters.rs:1030-1047, per head): d_q = M_h^T d_y; no gradient
 * reaches the frozen memory. */
void memory_read_only_backward_f32_rocm(const float *d_y, const float *m, float *d_q, long long n_tokens, int nh,
                                        int hd);

/* HOPE self-referential memory, chunkwise with frozen snapshots.  The reference runs it
 * on the CPU only (core/src/chunkwise_self_ref.rs:52-222 chunkwise_self_ref_step,
 * :336-620 chunkwise_self_ref_step_backward); these are the batched GPU forms.
 * Component order of every [6, d*d] block: m_k, m_v, m_q, m_eta, m_alpha, m_mem (:27-29).
 *   mems      [batch, 6, d*d]   in: initial memories, out: final memories
 *   embedded  [batch, seq_len, d]
 *   y, k/v/q_cache [batch, seq_len, d];  alpha/theta/alpha_mean/eta_mean_cache [batch, seq_len]
 *   frozen    [batch, num_chunks, 6, d*d], num_chunks = ceil(seq_len / chunk_size)
 * d = 16, 32, 64 run on the tiled kernels; every other d from 1 to 512 on general ones (the reference's own
 * tests use d = 4, core/src/chunkwise_self_ref.rs:662); larger d is an error. */
void selfref_chunkwise_forward_f32_rocm(float *mems, const float *embedded, float *y, float *k_cache,
                                        float *v_cache, float *q_cache, float *alpha_cache,
                                        float *theta_cache, float *alpha_mean_cache, float *eta_mean_cache,
                                        float *frozen, int seq_len, int d, int batch_size, int chunk_size,
                                        int self_generated_values);
/* d_embedded [batch, seq_len, d] and d_mems [batch, 6, d*d] (gradient w.r.t. the initial
 * memories, per chain) are overwritten. */
void selfref_chunkwise_backward_f32_rocm(const float *embedded, const float *d_y, const float *k_cache,
                                         const float *v_cache, const float *q_cache,
                                         const float *alpha_cache, const float *theta_cache,
                                         const float *alpha_mean_cache, const float *eta_mean_cache,
                                         const float *frozen, float *d_embedded, float *d_mems, int seq_len,
                                         int d, int batch_size, int chunk_size, int self_generated_values);

/* Frozen-M0 chunkwise Titans rule in matrix form on the matrix cores (same semantics as
 * titans_chunkwise_{forward,backward}_f32_cuda, core/src/cuda_ffi.rs:376/386, with
 * error_clip = 0 and no M-norm projection); no counterpart in the reference.
 * k/v/q: bf16 bit patterns [batch, seq_len, 64] (..._bf16_rocm) or float (..._mm_f32_rocm);
 * gates, states, y and all gradients are float.  d = 64, chunk_size in 1..64.
 * m_initial / s_initial [batch, d*d]; m/s_chunk_states [batch, num_chunks+1, d*d]. */
void titans_chunkwise_forward_bf16_rocm(const uint16_t *k_mem, const uint16_t *v_mem, const uint16_t *q_mem,
                                        const float *alpha, const float *theta, const float *eta,
                                        const float *m_initial, const float *s_initial,
                                        float *m_chunk_states, float *s_chunk_states, float *y,
                                        int seq_len, int d, int batch_size, int chunk_size);
void titans_chunkwise_forward_mm_f32_rocm(const float *k_mem, const float *v_mem, const float *q_mem,
                                          const float *alpha, const float *theta, const float *eta,
                                          const float *m_initial, const float *s_initial,
                                          float *m_chunk_states, float *s_chunk_states, float *y,
                                          int seq_len, int d, int batch_size, int chunk_size);
/* d_k/d_v/d_q [batch, seq_len, 64] and d_alpha/d_theta/d_eta [batch, seq_len] are overwritten;
 * d_m_initial / d_s_initial [d*d] are accumulated (+=) with the sum over the batch, like the
 * reference's chunkwise backward. */
void titans_chunkwise_backward_bf16_rocm(const uint16_t *k_mem, const uint16_t *v_mem, const uint16_t *q_mem,
                                         const float *alpha, const float *theta, const float *eta,
                                         const float *m_chunk_states, const float *s_chunk_states,
                                         const float *d_y, float *d_k_mem, float *d_v_mem, float *d_q_mem,
                                         float *d_alpha, float *d_theta, float *d_eta, float *d_m_initial,
                                         float *d_s_initial, int seq_len, int d, int batch_size,
                                         int chunk_size);
/* The bf16 pair above under the reference's production arguments (core/kernels/titans_chunkwise_forward.cu:89-176
 * with error_clip / m_norm_max as the json files under cli/configs ship them): the matrix form runs first and is kept when a
 * device-side test on its chunk-start states shows that neither the clip nor the projection can fire anywhere in
 * the call (then they are the identity and the results are the reference's); otherwise the sequential kernels,
 * which apply both per token, redo the call on the widened tokens.  One 4-byte copy to the host and a
 * synchronisation of the launch stream per call; while that stream is being captured the sequential kernels run.
 * The reference-named fp32 symbols {titans,delta}_chunkwise_{forward,backward}_f32_cuda do the same. */
void titans_chunkwise_forward_bf16_guarded_rocm(const uint16_t *k_mem, const uint16_t *v_mem, const uint16_t *q_mem,
                                                const float *alpha, const float *theta, const float *eta,
                                                const float *m_initial, const float *s_initial, float *m_chunk_states,
                                                float *s_chunk_states, float *y, int seq_len, int d, int batch_size,
                                                int chunk_size, float error_clip, float m_norm_max);
void titans_chunkwise_backward_bf16_guarded_rocm(const uint16_t *k_mem, const uint16_t *v_mem, const uint16_t *q_mem,
                                                 const float *alpha, const float *theta, const float *eta,
                                                 const float *m_chunk_states, const float *s_chunk_states, const float *d_y,
                                                 float *d_k_mem, float *d_v_mem, float *d_q_mem, float *d_alpha, float *d_theta,
                                                 float *d_eta, float *d_m_initial, float *d_s_initial, int seq_len, int d,
                                                 int batch_size, int chunk_size, float error_clip, float m_norm_max);
/* The same pair for a layer that keeps its tensors token-major (no counterpart in the reference, whose
 * gpu_memory_forward / gpu_memory_backward transpose between the layouts, core/src/gpu_forward.rs:1197 ff.):
 * chain c = (level, batch element, head), batch_size = levels * bs * heads; y_tokens [levels, bs, seq_len, heads*d]
 * is written directly; d_y_tokens has that shape (d_y_per_level != 0) or is ONE [bs, seq_len, heads*d] gradient
 * that every level reads.  k, v, q, the gates and the gradients stay head-major.  d = 64, chunk_size <= 64. */
void titans_chunkwise_forward_bf16_tokens_rocm(const uint16_t *k_mem, const uint16_t *v_mem, const uint16_t *q_mem,
                                               const float *alpha, const float *theta, const float *eta,
                                               const float *m_initial, const float *s_initial, float *m_chunk_states,
                                               float *s_chunk_states, float *y_tokens, int seq_len, int d,
                                               int batch_size, int chunk_size, int heads, int levels);
void titans_chunkwise_backward_bf16_tokens_rocm(const uint16_t *k_mem, const uint16_t *v_mem, const uint16_t *q_mem,
                                                const float *alpha, const float *theta, const float *eta,
                                                const float *m_chunk_states, const float *s_chunk_states,
                                                const float *d_y_tokens, float *d_k_mem, float *d_v_mem,
                                                float *d_q_mem, float *d_alpha, float *d_theta, float *d_eta,
                                                float *d_m_initial, float *d_s_initial, int seq_len, int d,
                                                int batch_size, int chunk_size, int heads, int levels,
                                                int d_y_per_level);
void titans_chunkwise_backward_mm_f32_rocm(const float *k_mem, const float *v_mem, const float *q_mem,
                                           const float *alpha, const float *theta, const float *eta,
                                           const float *m_chunk_states, const float *s_chunk_states,
                                           const float *d_y, float *d_k_mem, float *d_v_mem, float *d_q_mem,
                                           float *d_alpha, float *d_theta, float *d_eta, float *d_m_initial,
                                           float *d_s_initial, int seq_len, int d, int batch_size,
                                           int chunk_size);
/* Delta rule (no momentum state) in the same matrix form: semantics of
 * delta_chunkwise_{forward,backward}_f32_cuda (core/src/cuda_ffi.rs:356/365) with
 * error_clip = 0 and no M-norm projection.  d_m_initial [d*d] is accumulated (+=). */
void delta_chunkwise_forward_bf16_rocm(const uint16_t *k_mem, const uint16_t *v_mem, const uint16_t *q_mem,
                                       const float *alpha, const float *theta, const float *m_initial,
                                       float *m_chunk_states, float *y, int seq_len, int d, int batch_size,
                                       int chunk_size);
void delta_chunkwise_forward_mm_f32_rocm(const float *k_mem, const float *v_mem, const float *q_mem,
                                         const float *alpha, const float *theta, const float *m_initial,
                                         float *m_chunk_states, float *y, int seq_len, int d, int batch_size,
                                         int chunk_size);
void delta_chunkwise_backward_bf16_rocm(const uint16_t *k_mem, const uint16_t *v_mem, const uint16_t *q_mem,
                                        const float *alpha, const float *theta, const float *m_chunk_states,
                                        const float *d_y, float *d_k_mem, float *d_v_mem, float *d_q_mem,
                                        float *d_alpha, float *d_theta, float *d_m_initial, int seq_len, int d,
                                        int batch_size, int chunk_size);
void delta_chunkwise_backward_mm_f32_rocm(const float *k_mem, const float *v_mem, const float *q_mem,
                                          const float *alpha, const float *theta, const float *m_chunk_states,
                                          const float *d_y, float *d_k_mem, float *d_v_mem, float *d_q_mem,
                                          float *d_alpha, float *d_theta, float *d_m_initial, int seq_len, int d,
                                          int batch_size, int chunk_size);

/* core/src/cuda_ffi.rs:401: predictions[r] -= v[r], then rows with |.|_2 > error_clip are scaled to
 * error_clip (no clip for error_clip <= 0). */
void error_subtract_clip_f32_cuda(float *predictions, const float *v, int total_rows, int d, float error_clip);
/* core/src/cuda_ffi.rs:1000 / 973: k_mem and q_mem are L2-normalised IN PLACE (norm floor 1e-8),
 * the gates come from the normalised k and raw v (alpha = clamp(sigmoid), theta = clamp(softplus),
 * eta = sigmoid), then the full-trajectory recurrence runs; alpha/theta/eta/k_norms/q_norms
 * [batch*seq_len] are written for the backward. */
void titans_fused_forward_f32_cuda(float *k_mem, const float *v_mem, float *q_mem, const float *w_alpha,
                                   const float *b_alpha_ptr, const float *w_theta, const float *b_theta_ptr,
                                   const float *w_eta, const float *b_eta_ptr, float alpha_floor,
                                   float alpha_ceil, float theta_floor, float theta_ceil,
                                   const float *m_initial, const float *s_initial, float *m_states,
                                   float *s_states, float *y, float *alpha_out, float *theta_out,
                                   float *eta_out, float *k_norms_out, float *q_norms_out, int seq_len, int d,
                                   int batch_size, float error_clip, float m_norm_max);
void dgd_fused_forward_f32_cuda(float *k_mem, const float *v_mem, float *q_mem, const float *w_alpha,
                                const float *b_alpha_ptr, const float *w_theta, const float *b_theta_ptr,
                                float alpha_floor, float alpha_ceil, float theta_floor, float theta_ceil,
                                const float *m_initial, float *m_states, float *y, float *alpha_out,
                                float *theta_out, float *k_norms_out, float *q_norms_out, int seq_len, int d,
                                int batch_size, float error_clip);
/* core/src/cuda_ffi.rs:50: attention of the newest token (position cache_len-1) over a bf16 KV
 * cache [cache_len, heads*hd]; q, out [1, heads*hd]; no weights are kept. */
void swa_single_token_cuda(const uint16_t *q, const uint16_t *k_cache, const uint16_t *v_cache, uint16_t *out,
                           int cache_len, int num_heads, int head_dim, int window_size, int n_persistent);
/* Phase-2 kernels of the split chunkwise path (core/src/cuda_ffi.rs:407-453): the recurrence /
 * reverse sweep of chunk `chunk_idx` with the chunk's errors [batch, chunk_size, d] supplied by
 * the caller.  Forward: m_work / s_work [batch, d*d] are the running state (in/out); slot
 * chunk_idx of m/s_chunk_states [batch, num_chunks+1, d*d] receives the state at the chunk start
 * (and slot num_chunks the final state after the last chunk).  Backward: d_M / d_S [batch, d*d]
 * persist across chunks (in/out, per chain), d_M0 [batch, d*d] is written, m/s_recompute
 * [batch, chunk_size+1, d*d] are caller scratch for the replayed states.  d in {16, 32, 64}. */
void delta_phase2_forward_f32_cuda(const float *k_mem, const float *q_mem, const float *alpha,
                                   const float *theta, const float *errors, float *m_work,
                                   float *m_chunk_states, float *y, int seq_len, int d, int batch_size,
                                   int chunk_size, int chunk_idx, float m_norm_max);
void titans_phase2_forward_f32_cuda(const float *k_mem, const float *q_mem, const float *alpha,
                                    const float *theta, const float *eta, const float *errors,
                                    float *m_work, float *s_work, float *m_chunk_states,
                                    float *s_chunk_states, float *y, int seq_len, int d, int batch_size,
                                    int chunk_size, int chunk_idx, float m_norm_max);
void delta_phase2_backward_f32_cuda(const float *k_mem, const float *q_mem, const float *alpha,
                                    const float *theta, const float *errors, const float *m_chunk_states,
                                    const float *d_y, float *d_k_mem, float *d_v_mem, float *d_q_mem,
                                    float *d_alpha, float *d_theta, float *d_M, float *d_M0,
                                    float *m_recompute, int seq_len, int d, int batch_size, int chunk_size,
                                    int chunk_idx, float m_norm_max);
void titans_phase2_backward_f32_cuda(const float *k_mem, const float *q_mem, const float *alpha,
                                     const float *theta, const float *eta, const float *errors,
                                     const float *m_chunk_states, const float *s_chunk_states,
                                     const float *d_y, float *d_k_mem, float *d_v_mem, float *d_q_mem,
                                     float *d_alpha, float *d_theta, float *d_eta, float *d_M, float *d_S,
                                     float *d_M0, float *m_recompute, float *s_recompute, int seq_len, int d,
                                     int batch_size, int chunk_size, int chunk_idx, float m_norm_max);

/* ── one memory level's glue in one pass (no symbol in cuda_ffi.rs) ───────── */
/* Replaces, in gpu_memory_forward (core/src/gpu_forward.rs:1197 ff.), l2_normalize_rows x2, gate_compute x3,
 * transpose_heads x3, broadcast_heads x3 (and the f32 -> bf16 copies when heads_bf16 != 0).  k_mem and q_mem
 * [bs*s, nh*hd] are normalised in place; alpha = sigmoid, theta = softplus, eta = sigmoid of
 * w . [k | v] + b; k/v/q_heads are [bs*nh, s, hd] (bf16 bit patterns when heads_bf16, else float), the
 * *_heads gates [bs*nh, s]. */
void memory_inputs_fused_rocm(float *k_mem, const float *v_mem, float *q_mem, const float *w_alpha,
                              const float *b_alpha, const float *w_theta, const float *b_theta, const float *w_eta,
                              const float *b_eta, float *k_norms, float *q_norms, float *alpha, float *theta,
                              float *eta, void *k_heads, void *v_heads, void *q_heads, float *alpha_heads,
                              float *theta_heads, float *eta_heads, int bs, int s, int nh, int hd, float eps,
                              int heads_bf16);
/* Replaces, in gpu_memory_backward (core/src/gpu_backward.rs:2047 ff.), sum_heads x3, transpose_heads x3 and
 * l2_normalize_backward x2: from the rule's head-major gradients to the token-major ones that the gate and
 * projection gradients take.  k_norm / q_norm are the normalised rows, k_norms / q_norms their former norms. */
void memory_grads_fused_rocm(const float *d_k_heads, const float *d_v_heads, const float *d_q_heads,
                             const float *d_alpha_heads, const float *d_theta_heads, const float *d_eta_heads,
                             const float *k_norm, const float *q_norm, const float *k_norms, const float *q_norms,
                             float *d_k_in, float *d_v, float *d_q_in, float *d_alpha, float *d_theta, float *d_eta,
                             int bs, int s, int nh, int hd, float eps);

/* ── the layer step's glue with strided operands (no symbols in cuda_ffi.rs) ───────────────────────────
 * The reference's layer step (core/src/gpu_forward.rs:864-1071, gpu_backward.rs:212-435) runs its projections as
 * one cuBLAS call each and streams every [tokens, d] tensor through a dozen small kernels.  Here the projections
 * of x are split-bf16 GEMMs over packed operands; these entry points let several producers fill column slabs of
 * ONE operand, and read projection outputs in place as column ranges of a wider GEMM output (row stride ld). */
/* As split_pack_bf16_rocm with row strides: source rows src_ld floats apart; in row r of out (out_ld bf16 values
 * apart) source i, column c goes to i*d + c, its hi part at off_h1 + and off_h2 +, its lo part at off_l +.
 * off_h2 < 0 (here and in level_grads_packed_rocm): the hi part is written once. */
void split_pack_bf16_ld_rocm(const float *const *srcs, int count, long long src_ld, uint16_t *out, long long n, int d,
                             long long out_ld, long long off_h1, long long off_l, long long off_h2);
/* The packed fp32 weight rows [rows, d] -> wb [rows, 3d] = (Wh | Wl | Wh) per row, the right operand of the
 * forward projections against x packed as (xh | xh | xl), and wstack [3*rows_stack, d] = (Wh ; Wh ; Wl) of the
 * first rows_stack rows, the right operand of d_x = P . wstack for P packed as (H | L | H). */
void split_pack_weights_rocm(const float *pack, int rows, int rows_stack, int d, uint16_t *wb, uint16_t *wstack);
/* memory_inputs_fused_rocm on k_mem, v_mem, q_mem with row stride ld (floats); 16-byte accesses, so head_dim must
 * be a multiple of 4 and nh*hd <= 1024.  Sums run in another order than in memory_inputs_fused_rocm.
 * normalise_in_place == 0 leaves k_mem and q_mem as they came (the heads still get the normalised rows): a
 * backward that divides by k_norms / q_norms again (level_grads_packed_rocm, inputs_raw) saves the write. */
void level_inputs_fused_rocm(float *k_mem, const float *v_mem, float *q_mem, long long ld, const float *w_alpha,
                             const float *b_alpha, const float *w_theta, const float *b_theta, const float *w_eta,
                             const float *b_eta, float *k_norms, float *q_norms, float *alpha, float *theta, float *eta,
                             void *k_heads, void *v_heads, void *q_heads, float *alpha_heads, float *theta_heads,
                             float *eta_heads, int bs, int s, int nh, int hd, float eps, int heads_bf16,
                             int normalise_in_place);
/* memory_grads_fused_rocm + gate_backward_cuda + split_pack_bf16_rocm in one pass (gpu_backward.rs:2047-2115):
 * from the rule's head-major gradients to (a) the packed operand of the projection-gradient GEMMs, written into
 * p_out (row stride p_ld) with d_k_in at column 0, d_v at d, d_q_in at 2d of each of the three positions
 * off_h1 / off_l / off_h2, and (b) the gate projections' weight [2d] and bias [1] gradients, assigned.
 * k_norm, v_mem, q_norm: the level's normalised k, its v and normalised q, row stride ld (inputs_raw != 0: k and
 * q as projected, normalised here with k_norms / q_norms); alpha, theta, eta [bs*s]: the gate outputs. */
void level_grads_packed_rocm(const float *d_k_heads, const float *d_v_heads, const float *d_q_heads,
                             const float *d_alpha_heads, const float *d_theta_heads, const float *d_eta_heads,
                             const float *k_norm, const float *v_mem, const float *q_norm, long long ld,
                             const float *k_norms, const float *q_norms, const float *alpha, const float *theta,
                             const float *eta, uint16_t *p_out, long long p_ld, long long off_h1, long long off_l,
                             long long off_h2, float *d_w_alpha, float *d_b_alpha, float *d_w_theta, float *d_b_theta,
                             float *d_w_eta, float *d_b_eta, int bs, int s, int nh, int hd, float eps, int inputs_raw);
/* cms_combine_gate_rocm / cms_gate_backward_rocm with the attention output in bf16 (what the attention kernels
 * write) and no y_combined copy; n a multiple of 4.  gated (fp32) and gated_packed ([n / d, 3d] bf16: hi | hi | lo of
 * each row, the left operand of the output projection as a split-bf16 GEMM) may each be null. */
void cms_combine_gate_bf16_rocm(const float *const *y_levels, int k, const uint16_t *attn_out, float *gate, float *gated,
                                uint16_t *gated_packed, int d, long long n);
void cms_gate_backward_bf16_rocm(const float *d_gated, const uint16_t *attn_out, const float *gate, int k, float *d_attn,
                                 float *d_y_combined, long long n);

/* ── Titans rule with an MLP memory: packed state [W1 (dh x d) | b1 (dh) | W2 (d x dh) | b2 (d)] ── */
/* core/src/cuda_ffi.rs:854.  input_stride = elements between the chains' token tensors (seq_len * d),
 * m_stride = elements between the chains' trajectories ((seq_len + 1) * state_size); activation 0 GELU,
 * 1 SiLU, 2 ReLU. */
void titans_mlp_forward_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem, const float *alpha,
                                 const float *theta, const float *eta, const float *m_initial, const float *s_initial,
                                 float *m_states, float *s_states, float *y, int seq_len, int d, int d_hidden,
                                 int batch_size, int input_stride, int m_stride, int activation, float m_norm_max);
/* core/src/cuda_ffi.rs:887 (d_m_initial, d_s_initial [state_size] are summed over the batch into the
 * caller's zeroed buffers) */
void titans_mlp_backward_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem, const float *alpha,
                                  const float *theta, const float *eta, const float *m_states, const float *s_states,
                                  const float *d_y, float *d_k_mem, float *d_v_mem, float *d_q_mem, float *d_alpha,
                                  float *d_theta, float *d_eta, float *d_m_initial, float *d_s_initial, int seq_len,
                                  int d, int d_hidden, int batch_size, int input_stride, int m_stride, int activation,
                                  float m_norm_max);

/* ── MIRAS MLP memories (one chain): MONETA (l_p error, L_q / L2 retention), YAAD (Huber, local + L2) ── */
/* core/src/cuda_ffi.rs:785.  w*_states [(seq_len + 1), d_hidden * d]: the full trajectories. */
void mlp_forward_lp_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem, const float *alpha,
                             const float *theta, const float *w1_initial, const float *w2_initial, float *w1_states,
                             float *w2_states, float *y, int seq_len, int d, int d_hidden, float lp_p,
                             float sign_sharpness, float lambda_2, float lq_q);
/* core/src/cuda_ffi.rs:799 */
void mlp_forward_huber_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem, const float *alpha,
                                const float *theta, const float *w1_initial, const float *w2_initial,
                                const float *w1_boundary, const float *w2_boundary, float *w1_states, float *w2_states,
                                float *y, int seq_len, int d, int d_hidden, float huber_delta, float lambda_local,
                                float lambda_2);
/* core/src/cuda_ffi.rs:813 (q = 2 only; d_k_mem is added to and d_v_mem subtracted from: the caller zeroes them) */
void mlp_backward_lp_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem, const float *alpha,
                              const float *theta, const float *w1_states, const float *w2_states, const float *d_y,
                              float *d_k_mem, float *d_v_mem, float *d_q_mem, float *d_alpha, float *d_theta,
                              float *d_w1_initial, float *d_w2_initial, int seq_len, int d, int d_hidden, float lp_p,
                              float sign_sharpness, float lambda_2, float lq_q);
/* core/src/cuda_ffi.rs:829 */
void mlp_backward_huber_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem, const float *alpha,
                                 const float *theta, const float *w1_states, const float *w2_states,
                                 const float *w1_boundary, const float *w2_boundary, const float *d_y, float *d_k_mem,
                                 float *d_v_mem, float *d_q_mem, float *d_alpha, float *d_theta, float *d_w1_initial,
                                 float *d_w2_initial, int seq_len, int d, int d_hidden, float huber_delta,
                                 float lambda_local, float lambda_2);

/* ── SwiGLU MLP, device-to-device (the GEMMs go to rocBLAS on the library's stream) ── */
/* core/src/cuda_ffi.rs:925 */
void swiglu_forward_f32_cuda_dd(const float *x, const float *gate_proj, const float *up_proj, const float *down_proj,
                                float *y, float *gate_buf, float *up_buf, float *fused_buf, float *cache_buf,
                                int seq_len, int d_model, int intermediate);
/* core/src/cuda_ffi.rs:945 (output gradients are written, not accumulated) */
void swiglu_backward_f32_cuda_dd(const float *d_y, const float *x, const float *gate_proj, const float *up_proj,
                                 const float *down_proj, const float *fused_buf, const float *gate_buf,
                                 const float *up_buf, const float *cache_buf, float *d_x, float *d_gate_proj,
                                 float *d_up_proj, float *d_down_proj, int seq_len, int d_model, int intermediate);

/* ── around the memory path: normalisation, embedding, loss, TNT helpers, pooling, M3 helpers ── */
/* core/src/cuda_ffi.rs:487 */
void layer_norm_forward_cuda(const float *x, const float *gamma, const float *beta, float *out,
                             float *mean_cache, float *rstd_cache, int n, int d, float eps);
/* core/src/cuda_ffi.rs:495 (d_gamma, d_beta are accumulated: the caller zeroes them; d <= 2048) */
void layer_norm_backward_cuda(const float *d_out, const float *x, const float *gamma, const float *mean_cache,
                              const float *rstd_cache, float *d_x, float *d_gamma, float *d_beta, int n, int d);
/* core/src/cuda_ffi.rs:523 */
void embedding_gather_cuda(const float *w_embed, const int *input_ids, float *output, int seq_len, int d);
/* core/src/cuda_ffi.rs:532 (d_embed is accumulated) */
void embedding_scatter_add_cuda(const float *d_embedded, const int *input_ids, float *d_embed, int seq_len, int d);
/* core/src/cuda_ffi.rs:542: dst[col * rows + row] = src[row * cols + col] */
void transpose_copy_cuda(const float *src, float *dst, int rows, int cols);
/* core/src/cuda_ffi.rs:766 (loss_out[0] = sum of the rows' NLL; rows with a target outside [0, vocab) are skipped) */
void cross_entropy_forward_cuda(const float *logits, const int *target_ids, float *loss_out, int seq_len, int vocab);
/* core/src/cuda_ffi.rs:772 */
void cross_entropy_backward_cuda(const float *logits, const int *target_ids, float *d_logits, int seq_len, int vocab,
                                 float inv_count);
/* core/src/cuda_ffi.rs:616 */
void tnt_broadcast_m_f32_cuda(const float *m_src, float *m_dst, int n_local, int d);
/* core/src/cuda_ffi.rs:624 */
void tnt_shard_summary_mean_f32_cuda(const float *local_y, float *k_sum, float *v_sum, int shard_len, int d);
/* core/src/cuda_ffi.rs:633 */
void tnt_global_update_f32_cuda(float *global_m, const float *k_sum, const float *v_sum, int d, float alpha);
/* core/src/cuda_ffi.rs:642 (d_k_sum, d_v_sum are accumulated) */
void tnt_global_update_backward_f32_cuda(const float *d_m_new, const float *k_sum, const float *v_sum,
                                         float *d_m_old, float *d_k_sum, float *d_v_sum, int d, float alpha);
/* core/src/cuda_ffi.rs:654 (d_local_y is accumulated) */
void tnt_shard_summary_mean_backward_f32_cuda(const float *d_k_sum, const float *d_v_sum, float *d_local_y,
                                              int shard_len, int d);
/* core/src/cuda_ffi.rs:663 */
void tnt_combine_gradients_f32_cuda(const float *d_y_upstream, const float *d_y_global, float *d_y_combined, int n);
/* core/src/cuda_ffi.rs:1061, 1067, 1074 (d_x accumulated), 1081; tokens past the last full group of C are
 * not read and not written */
void mean_pool_1d_f32_cuda(const float *x, float *out, int bs, int s, int d, int C);
void repeat_upsample_1d_f32_cuda(const float *x, float *out, int bs, int s, int d, int C);
void mean_pool_1d_backward_f32_cuda(const float *d_out, float *d_x, int bs, int s, int d, int C);
void repeat_upsample_1d_backward_f32_cuda(const float *d_out, float *d_x, int bs, int s, int d, int C);
/* core/src/cuda_ffi.rs:722, 730, 740, 747, 753, 757; return 0 on success like the AdamW family */
unsigned m3_ema_update_cuda(float *m1, float *m2, float *v, const float *g, int n, float beta1, float beta2,
                            float beta3, int update_m2);
unsigned m3_apply_1d_cuda(float *w, const float *m1, const float *m2, const float *v, int n, float lr, float alpha,
                          float eps, float bc2);
unsigned m3_apply_2d_cuda(float *w, const float *o1, const float *o2, int n, float lr, float alpha);
unsigned frob_norm_sq_cuda(const float *x, float *partial_sums, int n, int *out_num_blocks);
unsigned scale_buf_cuda(float *x, float scale, int n);
unsigned m3_ns_poly_cuda(float *x, const float *y, const float *z, int n, float a, float b, float c);

/* ── host-slice dispatch: every pointer below is HOST memory ───────────────────────────────────
 * The bodies of the reference's `*_dispatch` functions for a device feature: one chain is staged on
 * the device (allocate, copy in, zero the outputs, launch with batch_size = 1, synchronise, copy out),
 * as core/src/dispatch.rs:1665-2085 does with its own DevBuf.  Argument order = the Rust function's.
 * These are what the rule structs and the opaque VJP blocks of the Wengert tape call on a CPU tape
 * (core/src/opaque_adapters.rs:306-400 Delta, 402-590 Titans, 593-629 Hebbian, 966-1010 SWA,
 * 1686-1725 DGD). */
/* core/src/dispatch.rs:746 */
void nlh_delta_forward_dispatch(const float *k_mem, const float *v_mem, const float *q_mem, const float *alpha,
                                const float *theta, const float *m_initial, float *m_states, float *y,
                                int seq_len, int d, float error_clip, float m_norm_max);
/* core/src/dispatch.rs:775 (gradients are overwritten) */
void nlh_delta_backward_dispatch(const float *k_mem, const float *v_mem, const float *q_mem, const float *alpha,
                                 const float *theta, const float *m_states, const float *d_y, float *d_k_mem,
                                 float *d_v_mem, float *d_q_mem, float *d_alpha, float *d_theta,
                                 float *d_m_initial, int seq_len, int d, float error_clip);
/* core/src/dispatch.rs:810 */
void nlh_titans_forward_dispatch(const float *k_mem, const float *v_mem, const float *q_mem, const float *alpha,
                                 const float *theta, const float *eta, const float *m_initial,
                                 const float *s_initial, float *m_states, float *s_states, float *y,
                                 int seq_len, int d, float error_clip, float m_norm_max);
/* core/src/dispatch.rs:842 */
void nlh_titans_backward_dispatch(const float *k_mem, const float *v_mem, const float *q_mem, const float *alpha,
                                  const float *theta, const float *eta, const float *m_states,
                                  const float *s_states, const float *d_y, float *d_k_mem, float *d_v_mem,
                                  float *d_q_mem, float *d_alpha, float *d_theta, float *d_eta,
                                  float *d_m_initial, float *d_s_initial, int seq_len, int d, float error_clip);
/* core/src/dispatch.rs:1083 (a finite positive m_norm_max is refused: the reference runs that case on the CPU) */
void nlh_hebbian_forward_dispatch(const float *k_mem, const float *v_mem, const float *q_mem, const float *alpha,
                                  const float *m_initial, float *m_states, float *y, int seq_len, int d,
                                  float m_norm_max);
/* core/src/dispatch.rs:1110 */
void nlh_hebbian_backward_dispatch(const float *k_mem, const float *v_mem, const float *q_mem, const float *alpha,
                                   const float *m_states, const float *d_y, float *d_k_mem, float *d_v_mem,
                                   float *d_q_mem, float *d_alpha, float *d_m_initial, int seq_len, int d);
/* core/src/dispatch.rs:1153 */
void nlh_dgd_forward_dispatch(const float *k_mem, const float *v_mem, const float *q_mem, const float *alpha,
                              const float *theta, const float *m_initial, float *m_states, float *y, int seq_len,
                              int d, float error_clip);
/* core/src/dispatch.rs:1182 */
void nlh_dgd_backward_dispatch(const float *k_mem, const float *v_mem, const float *q_mem, const float *alpha,
                               const float *theta, const float *m_states, const float *d_y, float *d_k_mem,
                               float *d_v_mem, float *d_q_mem, float *d_alpha, float *d_theta, float *d_m_initial,
                               int seq_len, int d, float error_clip);
/* core/src/dispatch.rs:378 (float on the host, bf16 on the device; one sequence, no persistent tokens) */
void nlh_swa_forward_dispatch(const float *q, const float *k, const float *v, float *out, float *attn_weights,
                              int seq_len, int num_heads, int head_dim, int window_size);
/* core/src/dispatch.rs:408 (the caller zeroes d_q, d_k, d_v as the reference asks: d_k, d_v are accumulated
 * into, d_q is overwritten) */
void nlh_swa_backward_dispatch(const float *q, const float *k, const float *v, const float *attn_weights,
                               const float *d_attn_out, float *d_q, float *d_k, float *d_v, int seq_len,
                               int num_heads, int head_dim, int window_size);

/* ── The level step of a CMS layer (no single counterpart symbol in core/src/cuda_ffi.rs: the reference
 * composes it on the host from cublasSgemm and the glue kernels) ─────────────────────────────────────
 * gpu_memory_forward (core/src/gpu_forward.rs:1197-1382) for `levels` Titans levels over the same tokens:
 * k, v, q = x W^T per level, k and q L2-normalised over the model width, the three gates
 * (sigmoid / softplus / sigmoid of [k | v] . w + b), head split.  One launch computes every projection on the
 * bf16 matrix cores (x and the weights rounded once to bf16, fp32 accumulation) and writes the rule kernels'
 * operands directly.  n = bs * seq_len tokens, d = heads * head_dim in {256, 512}, head_dim = 64.
 *   x [n, d]; w_extra [n_extra * d, d]: plain projections of x (the attention branch's q, k, v) whose results
 *   leave as bf16 [n, d] in extra_out[0 .. n_extra); w_levels [levels * 3 * d, d]: rows k, v, q of every level;
 *   gate_params: host array of 6 * levels device pointers (w_alpha [2d], b_alpha [1], w_theta, b_theta, w_eta,
 *   b_eta per level).  Outputs: x_bf16 [n, d] (x rounded to bf16, the backward's operand; may be null);
 *   k/v/q_heads bf16 [levels * bs * heads, seq_len, head_dim] (chain = (level, batch element, head));
 *   alpha/theta/eta_heads [levels * bs * heads, seq_len]; k_norms, q_norms, alpha, theta, eta [levels, n]. */
void level_project_forward_bf16_rocm(const float *x, const float *w_extra, int n_extra, uint16_t *const *extra_out,
                                     const float *w_levels, const float *const *gate_params, uint16_t *x_bf16,
                                     uint16_t *k_heads, uint16_t *v_heads, uint16_t *q_heads, float *alpha_heads,
                                     float *theta_heads, float *eta_heads, float *k_norms, float *q_norms, float *alpha,
                                     float *theta, float *eta, int bs, int seq_len, int heads, int head_dim, int levels,
                                     float eps);
/* The projections above, then the chunkwise Titans rule on all levels' chains at once
 * (titans_chunkwise_forward_bf16_tokens_rocm) from the carried context memories m_context, s_context
 * [levels * bs * heads, head_dim^2], which receive the final states (copy_final_m_batch, gpu_forward.rs:2824).
 * m/s_chunk_states [levels * bs * heads, num_chunks + 1, head_dim^2]; y_tokens [levels, bs, seq_len, d]. */
void titans_levels_forward_bf16_rocm(const float *x, const float *w_extra, int n_extra, uint16_t *const *extra_out,
                                     const float *w_levels, const float *const *gate_params, float *m_context,
                                     float *s_context, uint16_t *x_bf16, uint16_t *k_heads, uint16_t *v_heads,
                                     uint16_t *q_heads, float *alpha_heads, float *theta_heads, float *eta_heads,
                                     float *k_norms, float *q_norms, float *alpha, float *theta, float *eta,
                                     float *m_chunk_states, float *s_chunk_states, float *y_tokens, int bs, int seq_len,
                                     int heads, int head_dim, int levels, int chunk_size, float eps);
/* gpu_memory_backward + accumulate_projection_grads (core/src/gpu_backward.rs:459-640, 2047-2115) for the same
 * stack: rule backward from ONE upstream gradient d_y_tokens [bs, seq_len, d] that every level reads, head sums
 * and activation derivatives of the gates, backward of the two normalisations, then d_x [n, d] (overwritten) =
 * sum over all projections of g W, and d_w_extra [n_extra * d, d], d_w_levels [levels * 3 * d, d] (overwritten)
 * = g^T x, as bf16 GEMMs with fp32 accumulation; d_extra: host array of n_extra device pointers, the fp32
 * gradients [n, d] of the plain projections' outputs, or n_extra null pointers when the caller has already
 * written them as bf16 into columns e * d .. of the operand that level_grad_operand_rocm returns; d_gate_params:
 * host array of 6 * levels device pointers (overwritten).  As on the reference's GPU path nothing flows from the gates into k and v.
 * d_m_initial, d_s_initial [head_dim^2] are accumulated (+=, summed over all chains). */
void titans_levels_backward_bf16_rocm(const uint16_t *x_bf16, const float *w_extra, int n_extra, const float *const *d_extra,
                                      const float *w_levels, const uint16_t *k_heads, const uint16_t *v_heads,
                                      const uint16_t *q_heads, const float *alpha_heads, const float *theta_heads,
                                      const float *eta_heads, const float *k_norms, const float *q_norms, const float *alpha,
                                      const float *theta, const float *eta, const float *m_chunk_states,
                                      const float *s_chunk_states, const float *d_y_tokens, float *d_x, float *d_w_extra,
                                      float *d_w_levels, float *const *d_gate_params, float *d_m_initial, float *d_s_initial,
                                      int bs, int seq_len, int heads, int head_dim, int levels, int chunk_size, float eps);
/* The bf16 operand g [bs * seq_len, (n_extra + 3 * levels) * d] of the backward's two GEMMs, in the library's
 * scratch (stable until a larger call or nlh_release_workspace): projection e's output gradient belongs in columns
 * e * d .. e * d + d - 1.  A producer that can write bf16 with a row stride (swa_backward_lse_bf16_cols_rocm) fills
 * them in place and passes null pointers as d_extra.  *ld receives the row stride in elements.  Null on bad shapes. */
uint16_t *level_grad_operand_rocm(int bs, int seq_len, int heads, int head_dim, int levels, int n_extra, long long *ld);
/* cms_combine_gate_bf16_rocm with gated leaving as plain bf16 [n] (the output projection's operand). */
void cms_combine_gate_bf16x1_rocm(const float *const *y_levels, int k, const uint16_t *attn_out, float *gate,
                                  uint16_t *gated_bf16, long long n);
/* out [n, d_out] = a W^T and its backward d_a [n, d_in] = g W, d_w [d_out, d_in] = g^T a (either may be null)
 * for a bf16 activation a [n, d_in], fp32 weights W [d_out, d_in] and an fp32 upstream gradient g [n, d_out],
 * both rounded once to bf16; fp32 accumulation (the cublasSgemm call sites of the output projection,
 * gpu_forward.rs:1066-1071, gpu_backward.rs:212-260). */
void linear_forward_bf16_rocm(const uint16_t *a_bf16, const float *w, float *out, int n, int d_in, int d_out);
void linear_backward_bf16_rocm(const float *d_out_f32, const uint16_t *a_bf16, const float *w, float *d_a, float *d_w, int n,
                               int d_in, int d_out);

/* ── What the box sustains (no counterpart in the reference) ─────────────────────────────────────────
 * Probe kernels behind `bench.py --workload hbm_copy / mfma_peak`: a streaming kernel that reads `reads` and
 * writes `writes` streams of n floats (16-byte accesses; in [reads, n], out [writes, n]), and the matrix cores'
 * issue peak for kind 0 = v_mfma_f32_16x16x32_bf16, 1 = v_mfma_f32_16x16x4_f32, 2 = v_mfma_f32_32x32x16_bf16 (out: compute units *
 * waves_per_simd * 256 floats; returns matrix instructions per wave, or < 0). */
int nlh_probe_stream_rocm(const float *in, float *out, long long n, int reads, int writes);
int nlh_probe_mfma_rocm(int kind, int iters, int waves_per_simd, float *out);

/* ── Opaque VJP blocks of the Wengert tape ───────────────────────────────────────────────────────
 * core/src/tape.rs:141-150 OpaqueBackwardFn(d_outputs, saved, d_inputs) for the OpaqueKey values
 * below (numbered in the order of the enum at tape.rs:100-134), with the saved-buffer layouts of the
 * registry's adapters (core/src/opaque_adapters.rs:290-304 DeltaRule, :386-401 TitansLMM, :952-964
 * SWA, :1004-1008 frozen reads, :1680-1690 DGD).  All pointers are HOST memory (the tape is a CPU
 * structure): buffer i of a list has lens[i] floats.  The block's backward runs on the GPU and its
 * results are ADDED to d_inputs (the accumulation the tape performs after an adapter returns,
 * tape.rs:839-866, is part of the call; a d_inputs buffer longer than what the rule produces, as with
 * learned frequency gates, keeps its tail).  Returns 0, or non-zero after recording a message
 * (argument error 1, layout / unsupported configuration 2, runtime 3).  Built: the default block
 * configuration (L2 attentional bias, identity feature map, no Conv1D, linear memory, EMA momentum)
 * in the newest recording format; d must be a size the memory-rule kernels serve. */
enum {
    NLH_OPAQUE_DELTA_RULE = 0,
    NLH_OPAQUE_TITANS_LMM = 1,
    NLH_OPAQUE_DGD = 9,
    NLH_OPAQUE_SWA = 10,
    NLH_OPAQUE_FROZEN_DELTA_RULE = 11,
    NLH_OPAQUE_FROZEN_TITANS_LMM = 12
};
int nlh_opaque_backward(int key, const float *const *d_outputs, const long long *d_output_lens, int n_outputs,
                        const float *const *saved, const long long *saved_lens, int n_saved,
                        float *const *d_inputs, const long long *d_input_lens, int n_inputs);

#ifdef __cplusplus
}
#endif
#endif /* NL_HECATE_FFI_H */
