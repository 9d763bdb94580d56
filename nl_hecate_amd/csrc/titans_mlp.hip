// Titans rule with an MLP memory ("deep neural memory"): the memory is the packed buffer
// [W1 (dh x d) | b1 (dh) | W2 (d x dh) | b2 (d)], updated per token by a gradient step on
// 1/2 |MLP(k) - v|^2 with EMA momentum and retention, then read with q.
// Contracts of core/kernels/titans_mlp_forward.cu / titans_mlp_backward.cu
// (core/src/cuda_ffi.rs:854-925); arithmetic as core/src/titans_lmm.rs step_mlp / mlp_inner_backward.
//
// One workgroup of four waves per chain; the state lives in the trajectories the contract asks for
// (global memory: it does not fit on chip at production sizes), the vectors of a token in LDS.
// The products come in two shapes: rows (out[r] = A[r, :] . x: one wave per row, lanes along the row,
// DPP sum: every row is read as contiguous 256-byte pieces) and columns (out[c] = sum_r A[r, c] x[r]:
// one thread per column, consecutive threads on consecutive addresses).  Rank-one updates and the
// state-wide sums are grid-stride loops over the packed buffer.  As in the reference, the backward
// treats act'(pre) of the inner gradient as a constant and the norm projection as the identity.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>

#include "../../include/nl_hecate_ffi.h"
#include "lane_ops.h"
#include "rule_common.h"
#include "runtime.h"

namespace nlh {
namespace {

constexpr int kMlpThreads = 256, kMlpWaves = kMlpThreads / 64;

// titans_mlp_forward.cu:37-61, 97-111: 0 GELU (tanh form), 1 SiLU, 2 ReLU
__device__ __forceinline__ float mlp_act(float x, int act) {
    if (act == 0) {
        const float inner = 0.7978845608028654f * (x + 0.044715f * x * x * x);
        return 0.5f * x * (1.0f + tanhf(inner));
    }
    if (act == 1) return x * (1.0f / (1.0f + expf(-x)));
    return fmaxf(0.0f, x);
}
__device__ __forceinline__ float mlp_act_prime(float x, int act) {
    if (act == 0) {
        const float c = 0.7978845608028654f, a = 0.044715f;
        const float t = tanhf(c * (x + a * x * x * x));
        return 0.5f * (1.0f + t) + 0.5f * x * (1.0f - t * t) * (c * (1.0f + 3.0f * a * x * x));
    }
    if (act == 1) {
        const float sg = 1.0f / (1.0f + expf(-x));
        return sg + x * sg * (1.0f - sg);
    }
    return x > 0.0f ? 1.0f : 0.0f;
}

struct MlpDims {
    int d, dh;
    __device__ __host__ size_t w1n() const { return (size_t)dh * d; }
    __device__ __host__ size_t o_b1() const { return w1n(); }
    __device__ __host__ size_t o_w2() const { return w1n() + dh; }
    __device__ __host__ size_t o_b2() const { return 2 * w1n() + dh; }
    __device__ __host__ size_t n() const { return 2 * w1n() + dh + d; }
};

// out[r] = f(r, A[r, :] . x + (bias ? bias[r] : 0)) for r < nrows; x in LDS.  One wave per row.
template <typename F>
__device__ __forceinline__ void rows_product(const float *A, int nrows, int ncols, const float *x, const float *bias,
                                             F store) {
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    for (int r = wv; r < nrows; r += kMlpWaves) {
        const float *row = A + (size_t)r * ncols;
        float sum = 0.f;
        for (int j = lane; j < ncols; j += 64) sum += row[j] * x[j];
        sum = wave_allreduce(sum);
        if (lane == 0) store(r, sum + (bias ? bias[r] : 0.f));
    }
}
// out[c] = f(c, sum_r A[r, c] x[r]) for c < ncols; x in LDS.  One thread per column.
template <typename F>
__device__ __forceinline__ void cols_product(const float *A, int nrows, int ncols, const float *x, F store) {
    for (int c = threadIdx.x; c < ncols; c += kMlpThreads) {
        float sum = 0.f;
        for (int r = 0; r < nrows; r++) sum += A[(size_t)r * ncols + c] * x[r];
        store(c, sum);
    }
}
// workgroup-wide sum; red: kMlpWaves floats of LDS; ends with a barrier
__device__ __forceinline__ float block_sum(float x, float *red) {
    x = wave_allreduce(x);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = x;
    __syncthreads();
    float tot = 0.f;
#pragma unroll
    for (int w = 0; w < kMlpWaves; w++) tot += red[w];
    __syncthreads();
    return tot;
}

struct MlpFwdArgs {
    const float *k, *v, *q, *alpha, *theta, *eta, *m_initial, *s_initial;
    float *m_states, *s_states, *y;
    int seq_len, d, dh, input_stride, m_stride, act;
    float m_norm_max;
};

__global__ __launch_bounds__(kMlpThreads) void titans_mlp_fwd_kernel(MlpFwdArgs a) {
    extern __shared__ float lds[];
    const MlpDims D{a.d, a.dh};
    const int d = a.d, dh = a.dh, tid = threadIdx.x, b = blockIdx.x;
    float *x = lds, *pre = x + d, *hid = pre + dh, *err = hid + dh, *gpre = err + d, *red = gpre + dh;
    const size_t n = D.n();
    const float *kb = a.k + (size_t)b * a.input_stride, *vb = a.v + (size_t)b * a.input_stride;
    const float *qb = a.q + (size_t)b * a.input_stride;
    const float *alb = a.alpha + (size_t)b * a.seq_len, *thb = a.theta + (size_t)b * a.seq_len;
    const float *etb = a.eta + (size_t)b * a.seq_len;
    float *mb = a.m_states + (size_t)b * a.m_stride, *sb = a.s_states + (size_t)b * a.m_stride;
    float *yb = a.y + (size_t)b * a.input_stride;
    for (size_t i = tid; i < n; i += kMlpThreads) {
        mb[i] = a.m_initial[(size_t)b * n + i];
        sb[i] = a.s_initial[(size_t)b * n + i];
    }
    __syncthreads();
    for (int t = 0; t < a.seq_len; t++) {
        const float *mt = mb + (size_t)t * n, *st = sb + (size_t)t * n;
        float *mn = mb + (size_t)(t + 1) * n, *sn = sb + (size_t)(t + 1) * n;
        for (int i = tid; i < d; i += kMlpThreads) x[i] = kb[(size_t)t * d + i];
        __syncthreads();
        rows_product(mt, dh, d, x, mt + D.o_b1(), [&](int r, float s) { pre[r] = s; hid[r] = mlp_act(s, a.act); });
        __syncthreads();
        rows_product(mt + D.o_w2(), d, dh, hid, mt + D.o_b2(), [&](int r, float s) { err[r] = s - vb[(size_t)t * d + r]; });
        __syncthreads();
        cols_product(mt + D.o_w2(), d, dh, err, [&](int c, float s) { gpre[c] = s * mlp_act_prime(pre[c], a.act); });
        __syncthreads();
        const float ret = 1.0f - alb[t], th = thb[t], et = etb[t];
        float sq = 0.f;
        for (size_t i = tid; i < n; i += kMlpThreads) {
            float grad;
            if (i < D.o_b1()) grad = gpre[i / d] * x[i % d];
            else if (i < D.o_w2()) grad = gpre[i - D.o_b1()];
            else if (i < D.o_b2()) grad = err[(i - D.o_w2()) / dh] * hid[(i - D.o_w2()) % dh];
            else grad = err[i - D.o_b2()];
            const float s_new = et * st[i] - th * grad;
            const float m_new = ret * mt[i] + s_new;
            sn[i] = s_new;
            mn[i] = m_new;
            sq += m_new * m_new;
        }
        __syncthreads();
        if (mnorm_active(a.m_norm_max)) {   // m_norm_project.cuh:22-58
            const float fnorm = sqrtf(block_sum(sq, red));
            if (fnorm > a.m_norm_max) {
                const float scale = a.m_norm_max / fnorm;
                for (size_t i = tid; i < n; i += kMlpThreads) mn[i] *= scale;
            }
            __syncthreads();
        }
        for (int i = tid; i < d; i += kMlpThreads) x[i] = qb[(size_t)t * d + i];
        __syncthreads();
        rows_product(mn, dh, d, x, mn + D.o_b1(), [&](int r, float s) { hid[r] = mlp_act(s, a.act); });
        __syncthreads();
        rows_product(mn + D.o_w2(), d, dh, hid, mn + D.o_b2(), [&](int r, float s) { yb[(size_t)t * d + r] = s; });
        __syncthreads();
    }
}

struct MlpBwdArgs {
    const float *k, *v, *q, *alpha, *theta, *eta, *m_states, *s_states, *d_y;
    float *d_k, *d_v, *d_q, *d_alpha, *d_theta, *d_eta, *dM, *dS;   // dM, dS: [batch, state] workspace, left as the result
    int seq_len, d, dh, input_stride, m_stride, act;
};

__global__ __launch_bounds__(kMlpThreads) void titans_mlp_bwd_kernel(MlpBwdArgs a) {
    extern __shared__ float lds[];
    const MlpDims D{a.d, a.dh};
    const int d = a.d, dh = a.dh, tid = threadIdx.x, b = blockIdx.x;
    float *x = lds, *pre = x + d, *hid = pre + dh, *err = hid + dh, *derr = err + d, *gpre = derr + d;
    float *dhb = gpre + dh, *dyv = dhb + dh, *red = dyv + d;
    const size_t n = D.n(), o_b1 = D.o_b1(), o_w2 = D.o_w2(), o_b2 = D.o_b2();
    const size_t io = (size_t)b * a.input_stride, go = (size_t)b * a.seq_len;
    const float *mb = a.m_states + (size_t)b * a.m_stride, *sb = a.s_states + (size_t)b * a.m_stride;
    float *dM = a.dM + (size_t)b * n, *dS = a.dS + (size_t)b * n;
    for (size_t i = tid; i < n; i += kMlpThreads) { dM[i] = 0.f; dS[i] = 0.f; }
    __syncthreads();
    for (int t = a.seq_len - 1; t >= 0; t--) {
        const float *mt = mb + (size_t)t * n, *mn = mb + (size_t)(t + 1) * n, *st = sb + (size_t)t * n;
        const float th = a.theta[go + t], ret = 1.0f - a.alpha[go + t], et = a.eta[go + t];
        // ── read path y = MLP_{M'}(q): d_M' and d_q ──
        for (int i = tid; i < d; i += kMlpThreads) { x[i] = a.q[io + (size_t)t * d + i]; dyv[i] = a.d_y[io + (size_t)t * d + i]; }
        __syncthreads();
        rows_product(mn, dh, d, x, mn + o_b1, [&](int r, float s) { pre[r] = s; hid[r] = mlp_act(s, a.act); });
        __syncthreads();
        cols_product(mn + o_w2, d, dh, dyv, [&](int c, float s) { dhb[c] = s * mlp_act_prime(pre[c], a.act); });
        __syncthreads();
        for (size_t i = tid; i < n; i += kMlpThreads) {
            float add;
            if (i < o_b1) add = dhb[i / d] * x[i % d];
            else if (i < o_w2) add = dhb[i - o_b1];
            else if (i < o_b2) add = dyv[(i - o_w2) / dh] * hid[(i - o_w2) % dh];
            else add = dyv[i - o_b2];
            dM[i] += add;
        }
        cols_product(mn, dh, d, dhb, [&](int c, float s) { a.d_q[io + (size_t)t * d + c] = s; });
        __syncthreads();
        // ── M' = (1 - alpha) M + S', S' = eta S - theta grad: d_S += d_M', d_alpha, d_eta ──
        float da = 0.f, de = 0.f;
        for (size_t i = tid; i < n; i += kMlpThreads) {
            const float ds = dS[i] + dM[i];
            dS[i] = ds;
            da += mt[i] * dM[i];
            de += st[i] * ds;
        }
        da = block_sum(da, red);
        de = block_sum(de, red);
        if (tid == 0) { a.d_alpha[go + t] = -da; a.d_eta[go + t] = de; }
        // ── the inner gradient at M_t on (k, v) ──
        for (int i = tid; i < d; i += kMlpThreads) x[i] = a.k[io + (size_t)t * d + i];
        __syncthreads();
        rows_product(mt, dh, d, x, mt + o_b1, [&](int r, float s) { pre[r] = s; hid[r] = mlp_act(s, a.act); });
        __syncthreads();
        rows_product(mt + o_w2, d, dh, hid, mt + o_b2, [&](int r, float s) { err[r] = s - a.v[io + (size_t)t * d + r]; });
        __syncthreads();
        cols_product(mt + o_w2, d, dh, err, [&](int c, float s) { gpre[c] = s * mlp_act_prime(pre[c], a.act); });
        __syncthreads();
        float dt = 0.f;
        for (size_t i = tid; i < n; i += kMlpThreads) {
            float grad;
            if (i < o_b1) grad = gpre[i / d] * x[i % d];
            else if (i < o_w2) grad = gpre[i - o_b1];
            else if (i < o_b2) grad = err[(i - o_w2) / dh] * hid[(i - o_w2) % dh];
            else grad = err[i - o_b2];
            dt += grad * dS[i];
        }
        dt = block_sum(dt, red);
        if (tid == 0) a.d_theta[go + t] = -dt;
        // d_err = -theta (dS_W2 h + dS_b2);  d_h = -theta dS_W2^T e;  d_k = -theta dS_W1^T gpre
        rows_product(dS + o_w2, d, dh, hid, dS + o_b2, [&](int r, float s) { derr[r] = -th * s; });
        cols_product(dS + o_w2, d, dh, err, [&](int c, float s) { dhb[c] = -th * s; });
        cols_product(dS, dh, d, gpre, [&](int c, float s) { a.d_k[io + (size_t)t * d + c] = -th * s; });
        __syncthreads();
        // d_gpre = -theta (dS_W1 k + dS_b1); through gpre = gh * act'(pre): d_gh (kept in gpre's place after use)
        rows_product(dS, dh, d, x, dS + o_b1, [&](int r, float s) { red[kMlpWaves + r] = -th * s * mlp_act_prime(pre[r], a.act); });
        __syncthreads();
        float *dgh = red + kMlpWaves;   // [dh]
        rows_product(mt + o_w2, d, dh, dgh, nullptr, [&](int r, float s) {
            const float de_r = derr[r] + s;
            derr[r] = de_r;
            a.d_v[io + (size_t)t * d + r] = -de_r;
        });
        __syncthreads();
        cols_product(mt + o_w2, d, dh, derr, [&](int c, float s) { dhb[c] = (dhb[c] + s) * mlp_act_prime(pre[c], a.act); });
        __syncthreads();
        cols_product(mt, dh, d, dhb, [&](int c, float s) { a.d_k[io + (size_t)t * d + c] += s; });
        // ── d_M = (1 - alpha) d_M' + the three outer products; d_S *= eta ──
        for (size_t i = tid; i < n; i += kMlpThreads) {
            float add;
            if (i < o_b1) add = dhb[i / d] * x[i % d];
            else if (i < o_w2) add = dhb[i - o_b1];
            else if (i < o_b2) {
                const size_t r = (i - o_w2) / dh, c = (i - o_w2) % dh;
                add = derr[r] * hid[c] + err[r] * dgh[c];
            } else add = derr[i - o_b2];
            dM[i] = ret * dM[i] + add;
            dS[i] = et * dS[i];
        }
        __syncthreads();
    }
}

bool mlp_args_ok(const char *fn, int seq_len, int d, int dh, int batch, int act) {
    if (d <= 0 || dh <= 0) { fail("%s: d=%d, d_hidden=%d must be > 0.", fn, d, dh); return false; }
    if (seq_len < 0 || batch < 0) { fail("%s: seq_len=%d batch=%d must be >= 0.", fn, seq_len, batch); return false; }
    if (act < 0 || act > 2) { fail("%s: unknown activation %d (expected 0=GELU, 1=SiLU, 2=ReLU).", fn, act); return false; }
    return true;
}

}  // namespace
}  // namespace nlh

using namespace nlh;

extern "C" {

void titans_mlp_forward_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem, const float *alpha,
                                 const float *theta, const float *eta, const float *m_initial, const float *s_initial,
                                 float *m_states, float *s_states, float *y, int seq_len, int d, int d_hidden,
                                 int batch_size, int input_stride, int m_stride, int activation, float m_norm_max) {
    if (!mlp_args_ok("titans_mlp_forward_f32_cuda", seq_len, d, d_hidden, batch_size, activation) || batch_size == 0) return;
    const size_t lds = (size_t)(2 * d + 3 * d_hidden + kMlpWaves) * sizeof(float);
    if (lds > 64 * 1024) { fail("titans_mlp_forward_f32_cuda: d=%d d_hidden=%d need %zu bytes of LDS (limit 65536).", d, d_hidden, lds); return; }
    const MlpFwdArgs a{k_mem, v_mem, q_mem, alpha, theta, eta, m_initial, s_initial, m_states, s_states, y,
                       seq_len, d, d_hidden, input_stride, m_stride, activation, m_norm_max};
    hipLaunchKernelGGL(titans_mlp_fwd_kernel, dim3(batch_size), dim3(kMlpThreads), lds, stream(), a);
    check_launch("titans_mlp_fwd_kernel");
}

void titans_mlp_backward_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem, const float *alpha,
                                  const float *theta, const float *eta, const float *m_states, const float *s_states,
                                  const float *d_y, float *d_k_mem, float *d_v_mem, float *d_q_mem, float *d_alpha,
                                  float *d_theta, float *d_eta, float *d_m_initial, float *d_s_initial, int seq_len,
                                  int d, int d_hidden, int batch_size, int input_stride, int m_stride, int activation,
                                  float m_norm_max) {
    (void)m_norm_max;   // the projection is the identity in the backward (titans_mlp_backward.cu: no use either)
    if (!mlp_args_ok("titans_mlp_backward_f32_cuda", seq_len, d, d_hidden, batch_size, activation) || batch_size == 0) return;
    const size_t lds = (size_t)(4 * d + 5 * d_hidden + kMlpWaves) * sizeof(float);
    if (lds > 64 * 1024) { fail("titans_mlp_backward_f32_cuda: d=%d d_hidden=%d need %zu bytes of LDS (limit 65536).", d, d_hidden, lds); return; }
    const size_t n = MlpDims{d, d_hidden}.n();
    float *dM = scratch(6, (size_t)batch_size * n * sizeof(float));
    float *dS = scratch(7, (size_t)batch_size * n * sizeof(float));
    if (failed()) return;
    const MlpBwdArgs a{k_mem, v_mem, q_mem, alpha, theta, eta, m_states, s_states, d_y, d_k_mem, d_v_mem, d_q_mem,
                       d_alpha, d_theta, d_eta, dM, dS, seq_len, d, d_hidden, input_stride, m_stride, activation};
    hipLaunchKernelGGL(titans_mlp_bwd_kernel, dim3(batch_size), dim3(kMlpThreads), lds, stream(), a);
    check_launch("titans_mlp_bwd_kernel");
    // summed over the batch into the caller's (zeroed) buffers, in a fixed order
    accumulate_over_batch(dM, d_m_initial, batch_size, (int)n);
    accumulate_over_batch(dS, d_s_initial, batch_size, (int)n);
}

}  // extern "C"
