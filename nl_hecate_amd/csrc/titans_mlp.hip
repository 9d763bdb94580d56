// Memory rules whose memory is a two-layer MLP.
// (1) Titans rule with an MLP memory ("deep neural memory"): the packed buffer
//     [W1 (dh x d) | b1 (dh) | W2 (d x dh) | b2 (d)], updated per token by a gradient step on
//     1/2 |MLP(k) - v|^2 with EMA momentum and retention, then read with q.  Contracts of
//     core/kernels/titans_mlp_forward.cu / titans_mlp_backward.cu (core/src/cuda_ffi.rs:854-925);
//     arithmetic as core/src/titans_lmm.rs step_mlp / mlp_inner_backward.
// (2) The MIRAS pair MONETA (l_p error, L_q / L2 retention) and YAAD (Huber error, local + global L2
//     retention): W1, W2 without biases, SiLU.  Contracts of core/kernels/moneta_forward.cu /
//     moneta_backward.cu (core/src/cuda_ffi.rs:785-846).
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

// ── MIRAS MLP memories ───────────────────────────────────────────────────────
// error gradient g(e) and its derivative: moneta_forward.cu:40-66, moneta_backward.cu:60-82.
// mode 0: l_p with p1 = p, p2 = sharpness of the smooth sign; mode 1: Huber with p1 = delta.
__device__ __forceinline__ float miras_g(float e, int mode, float p1, float p2) {
    if (mode == 1) return fabsf(e) < p1 ? e : (e > 0.0f ? p1 : -p1);
    if (fabsf(p1 - 2.0f) < 1e-6f) return 2.0f * e;
    if (fabsf(p1 - 1.0f) < 1e-6f) return tanhf(p2 * e);
    return p1 * tanhf(p2 * e) * powf(e * e + 1e-6f, (p1 - 1.0f) * 0.5f);
}
__device__ __forceinline__ float miras_g_prime(float e, int mode, float p1, float p2) {
    if (mode == 1) return fabsf(e) < p1 ? 1.0f : 0.0f;
    if (fabsf(p1 - 2.0f) < 1e-6f) return 2.0f;
    const float t = tanhf(p2 * e), sech2 = 1.0f - t * t;
    if (fabsf(p1 - 1.0f) < 1e-6f) return p2 * sech2;
    const float e2 = e * e + 1e-6f;
    return p1 * (p2 * sech2 * powf(e2, (p1 - 1.0f) * 0.5f) + t * (p1 - 1.0f) * e * powf(e2, (p1 - 3.0f) * 0.5f));
}

struct MirasArgs {
    const float *k, *v, *q, *alpha, *theta, *w1_boundary, *w2_boundary;
    int seq_len, d, dh, mode;
    float p1, p2, lambda_2, lq_q;
};

// moneta_forward.cu:100-430.  a1 / a2: the un-normalised accumulators of the L_q retention (q != 2), else null.
__global__ __launch_bounds__(kMlpThreads) void miras_mlp_fwd_kernel(MirasArgs a, const float *w1_initial,
                                                                    const float *w2_initial, float *w1_states,
                                                                    float *w2_states, float *y, float *a1, float *a2) {
    extern __shared__ float lds[];
    const int d = a.d, dh = a.dh, tid = threadIdx.x;
    float *x = lds, *pre = x + d, *hid = pre + dh, *g = hid + dh, *gpre = g + d, *red = gpre + dh;
    const size_t n = (size_t)dh * d;
    const bool use_lq = a1 != nullptr;
    const float lam_loc = a.mode == 1 ? a.p2 : 0.0f;
    for (size_t i = tid; i < n; i += kMlpThreads) {
        w1_states[i] = w1_initial[i];
        w2_states[i] = w2_initial[i];
        if (use_lq) { a1[i] = w1_initial[i]; a2[i] = w2_initial[i]; }
    }
    __syncthreads();
    for (int t = 0; t < a.seq_len; t++) {
        const float *w1 = w1_states + (size_t)t * n, *w2 = w2_states + (size_t)t * n;
        float *w1n = w1_states + (size_t)(t + 1) * n, *w2n = w2_states + (size_t)(t + 1) * n;
        for (int i = tid; i < d; i += kMlpThreads) x[i] = a.k[(size_t)t * d + i];
        __syncthreads();
        rows_product(w1, dh, d, x, nullptr, [&](int r, float s) { pre[r] = s; hid[r] = mlp_act(s, 1); });
        __syncthreads();
        rows_product(w2, d, dh, hid, nullptr, [&](int r, float s) { g[r] = miras_g(s - a.v[(size_t)t * d + r], a.mode, a.p1, a.p2); });
        __syncthreads();
        cols_product(w2, d, dh, g, [&](int c, float s) { gpre[c] = s * mlp_act_prime(pre[c], 1); });
        __syncthreads();
        const float al = a.alpha[t], th = a.theta[t];
        float q1 = 0.f, q2 = 0.f;
        for (size_t i = tid; i < n; i += kMlpThreads) {
            const float u1 = w1[i], u2 = w2[i];
            float r1 = a.lambda_2 * 2.0f * u1, r2 = a.lambda_2 * 2.0f * u2;
            if (a.mode == 1) {
                r1 += lam_loc * 2.0f * (u1 - a.w1_boundary[i]);
                r2 += lam_loc * 2.0f * (u2 - a.w2_boundary[i]);
            }
            const float g1 = gpre[i / d] * x[i % d], g2 = g[i / dh] * hid[i % dh];
            if (use_lq) {
                const float n1 = al * a1[i] - th * (g1 + r1), n2 = al * a2[i] - th * (g2 + r2);
                a1[i] = n1; a2[i] = n2;
                q1 += powf(fabsf(n1), a.lq_q);
                q2 += powf(fabsf(n2), a.lq_q);
            } else {
                w1n[i] = al * u1 - th * (g1 + r1);
                w2n[i] = al * u2 - th * (g2 + r2);
            }
        }
        __syncthreads();
        if (use_lq) {   // moneta_forward.cu:330-395: W' = A |A|_q^{-(q-2)}
            const float nq1 = powf(block_sum(q1, red), 1.0f / a.lq_q), nq2 = powf(block_sum(q2, red), 1.0f / a.lq_q);
            const float s1 = nq1 > 1e-12f ? powf(nq1, -(a.lq_q - 2.0f)) : 1.0f;
            const float s2 = nq2 > 1e-12f ? powf(nq2, -(a.lq_q - 2.0f)) : 1.0f;
            for (size_t i = tid; i < n; i += kMlpThreads) { w1n[i] = a1[i] * s1; w2n[i] = a2[i] * s2; }
            __syncthreads();
        }
        for (int i = tid; i < d; i += kMlpThreads) x[i] = a.q[(size_t)t * d + i];
        __syncthreads();
        rows_product(w1n, dh, d, x, nullptr, [&](int r, float s) { hid[r] = mlp_act(s, 1); });
        __syncthreads();
        rows_product(w2n, d, dh, hid, nullptr, [&](int r, float s) { y[(size_t)t * d + r] = s; });
        __syncthreads();
    }
}

// moneta_backward.cu:96-520 (q = 2).  dW1 / dW2: workspace, copied to d_w*_initial at the end.
__global__ __launch_bounds__(kMlpThreads) void miras_mlp_bwd_kernel(MirasArgs a, const float *w1_states,
                                                                    const float *w2_states, const float *d_y,
                                                                    float *d_k, float *d_v, float *d_q, float *d_alpha,
                                                                    float *d_theta, float *d_w1_initial,
                                                                    float *d_w2_initial, float *dW1, float *dW2) {
    extern __shared__ float lds[];
    const int d = a.d, dh = a.dh, tid = threadIdx.x;
    float *x = lds, *pre = x + d, *hid = pre + dh, *err = hid + dh, *g = err + d, *dg = g + d, *gpre = dg + d;
    float *dhb = gpre + dh, *dgh = dhb + dh, *dyv = dgh + dh, *red = dyv + d;
    const size_t n = (size_t)dh * d;
    const float lam_loc = a.mode == 1 ? a.p2 : 0.0f;
    for (size_t i = tid; i < n; i += kMlpThreads) { dW1[i] = 0.f; dW2[i] = 0.f; }
    __syncthreads();
    for (int t = a.seq_len - 1; t >= 0; t--) {
        const float *w1 = w1_states + (size_t)t * n, *w2 = w2_states + (size_t)t * n;
        const float *w1n = w1_states + (size_t)(t + 1) * n, *w2n = w2_states + (size_t)(t + 1) * n;
        const float al = a.alpha[t], th = a.theta[t];
        // read path
        for (int i = tid; i < d; i += kMlpThreads) { x[i] = a.q[(size_t)t * d + i]; dyv[i] = d_y[(size_t)t * d + i]; }
        __syncthreads();
        rows_product(w1n, dh, d, x, nullptr, [&](int r, float s) { pre[r] = s; hid[r] = mlp_act(s, 1); });
        __syncthreads();
        cols_product(w2n, d, dh, dyv, [&](int c, float s) { dhb[c] = s * mlp_act_prime(pre[c], 1); });
        __syncthreads();
        for (size_t i = tid; i < n; i += kMlpThreads) {
            dW2[i] += dyv[i / dh] * hid[i % dh];
            dW1[i] += dhb[i / d] * x[i % d];
        }
        cols_product(w1n, dh, d, dhb, [&](int c, float s) { d_q[(size_t)t * d + c] = s; });
        __syncthreads();
        // inner gradient at (W1_t, W2_t) on (k, v)
        for (int i = tid; i < d; i += kMlpThreads) x[i] = a.k[(size_t)t * d + i];
        __syncthreads();
        rows_product(w1, dh, d, x, nullptr, [&](int r, float s) { pre[r] = s; hid[r] = mlp_act(s, 1); });
        __syncthreads();
        rows_product(w2, d, dh, hid, nullptr, [&](int r, float s) {
            const float e = s - a.v[(size_t)t * d + r];
            err[r] = e;
            g[r] = miras_g(e, a.mode, a.p1, a.p2);
        });
        __syncthreads();
        cols_product(w2, d, dh, g, [&](int c, float s) { gpre[c] = s * mlp_act_prime(pre[c], 1); });
        __syncthreads();
        float da = 0.f, dt = 0.f;
        for (size_t i = tid; i < n; i += kMlpThreads) {
            const float u1 = w1[i], u2 = w2[i], e1 = dW1[i], e2 = dW2[i];
            da += e1 * u1 + e2 * u2;
            float r1 = a.lambda_2 * 2.0f * u1, r2 = a.lambda_2 * 2.0f * u2;
            if (a.mode == 1) {
                r1 += lam_loc * 2.0f * (u1 - a.w1_boundary[i]);
                r2 += lam_loc * 2.0f * (u2 - a.w2_boundary[i]);
            }
            dt -= e1 * (gpre[i / d] * x[i % d] + r1) + e2 * (g[i / dh] * hid[i % dh] + r2);
        }
        da = block_sum(da, red);
        dt = block_sum(dt, red);
        if (tid == 0) { d_alpha[t] = da; d_theta[t] = dt; }
        rows_product(dW2, d, dh, hid, nullptr, [&](int r, float s) { dg[r] = -th * s; });
        cols_product(dW2, d, dh, g, [&](int c, float s) { dhb[c] = -th * s; });
        cols_product(dW1, dh, d, gpre, [&](int c, float s) { d_k[(size_t)t * d + c] += -th * s; });
        rows_product(dW1, dh, d, x, nullptr, [&](int r, float s) { dgh[r] = -th * s * mlp_act_prime(pre[r], 1); });
        __syncthreads();
        rows_product(w2, d, dh, dgh, nullptr, [&](int r, float s) {
            const float de = (dg[r] + s) * miras_g_prime(err[r], a.mode, a.p1, a.p2);
            dg[r] = de;   // now d_err
            d_v[(size_t)t * d + r] -= de;
        });
        __syncthreads();
        cols_product(w2, d, dh, dg, [&](int c, float s) { dhb[c] = (dhb[c] + s) * mlp_act_prime(pre[c], 1); });
        __syncthreads();
        cols_product(w1, dh, d, dhb, [&](int c, float s) { d_k[(size_t)t * d + c] += s; });
        const float coeff = al - th * (lam_loc + a.lambda_2) * 2.0f;
        for (size_t i = tid; i < n; i += kMlpThreads) {
            dW1[i] = coeff * dW1[i] + dhb[i / d] * x[i % d];
            dW2[i] = coeff * dW2[i] + dg[i / dh] * hid[i % dh] + g[i / dh] * dgh[i % dh];
        }
        __syncthreads();
    }
    for (size_t i = tid; i < n; i += kMlpThreads) { d_w1_initial[i] = dW1[i]; d_w2_initial[i] = dW2[i]; }
}

void miras_forward(const char *fn, MirasArgs a, const float *w1_initial, const float *w2_initial, float *w1_states,
                   float *w2_states, float *y) {
    const ErrorScope es;
    if (a.d <= 0 || a.dh <= 0) { fail("%s: d=%d, d_hidden=%d must be > 0.", fn, a.d, a.dh); return; }
    if (a.seq_len < 0) { fail("%s: seq_len=%d must be >= 0.", fn, a.seq_len); return; }
    const size_t lds = (size_t)(2 * a.d + 3 * a.dh + kMlpWaves) * sizeof(float);
    if (lds > 64 * 1024) { fail("%s: d=%d d_hidden=%d need %zu bytes of LDS (limit 65536).", fn, a.d, a.dh, lds); return; }
    float *a1 = nullptr, *a2 = nullptr;
    if (a.mode == 0 && fabsf(a.lq_q - 2.0f) >= 1e-6f) {
        const size_t bytes = (size_t)a.dh * a.d * sizeof(float);
        a1 = scratch(6, bytes);
        a2 = scratch(7, bytes);
        if (es.failed()) return;
    }
    hipLaunchKernelGGL(miras_mlp_fwd_kernel, dim3(1), dim3(kMlpThreads), lds, stream(), a, w1_initial, w2_initial,
                       w1_states, w2_states, y, a1, a2);
    check_launch("miras_mlp_fwd_kernel");
}

void miras_backward(const char *fn, MirasArgs a, const float *w1_states, const float *w2_states, const float *d_y,
                    float *d_k, float *d_v, float *d_q, float *d_alpha, float *d_theta, float *d_w1_initial,
                    float *d_w2_initial) {
    const ErrorScope es;
    if (a.d <= 0 || a.dh <= 0) { fail("%s: d=%d, d_hidden=%d must be > 0.", fn, a.d, a.dh); return; }
    if (a.seq_len < 0) { fail("%s: seq_len=%d must be >= 0.", fn, a.seq_len); return; }
    const size_t lds = (size_t)(5 * a.d + 5 * a.dh + kMlpWaves) * sizeof(float);
    if (lds > 64 * 1024) { fail("%s: d=%d d_hidden=%d need %zu bytes of LDS (limit 65536).", fn, a.d, a.dh, lds); return; }
    const size_t bytes = (size_t)a.dh * a.d * sizeof(float);
    float *dW1 = scratch(6, bytes), *dW2 = scratch(7, bytes);
    if (es.failed()) return;
    hipLaunchKernelGGL(miras_mlp_bwd_kernel, dim3(1), dim3(kMlpThreads), lds, stream(), a, w1_states, w2_states, d_y,
                       d_k, d_v, d_q, d_alpha, d_theta, d_w1_initial, d_w2_initial, dW1, dW2);
    check_launch("miras_mlp_bwd_kernel");
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
    const ErrorScope es;
    (void)m_norm_max;   // the projection is the identity in the backward (titans_mlp_backward.cu: no use either)
    if (!mlp_args_ok("titans_mlp_backward_f32_cuda", seq_len, d, d_hidden, batch_size, activation) || batch_size == 0) return;
    const size_t lds = (size_t)(4 * d + 5 * d_hidden + kMlpWaves) * sizeof(float);
    if (lds > 64 * 1024) { fail("titans_mlp_backward_f32_cuda: d=%d d_hidden=%d need %zu bytes of LDS (limit 65536).", d, d_hidden, lds); return; }
    const size_t n = MlpDims{d, d_hidden}.n();
    float *dM = scratch(6, (size_t)batch_size * n * sizeof(float));
    float *dS = scratch(7, (size_t)batch_size * n * sizeof(float));
    if (es.failed()) return;
    const MlpBwdArgs a{k_mem, v_mem, q_mem, alpha, theta, eta, m_states, s_states, d_y, d_k_mem, d_v_mem, d_q_mem,
                       d_alpha, d_theta, d_eta, dM, dS, seq_len, d, d_hidden, input_stride, m_stride, activation};
    hipLaunchKernelGGL(titans_mlp_bwd_kernel, dim3(batch_size), dim3(kMlpThreads), lds, stream(), a);
    check_launch("titans_mlp_bwd_kernel");
    // summed over the batch into the caller's (zeroed) buffers, in a fixed order
    accumulate_over_batch(dM, d_m_initial, batch_size, (int)n);
    accumulate_over_batch(dS, d_s_initial, batch_size, (int)n);
}

void mlp_forward_lp_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem, const float *alpha,
                             const float *theta, const float *w1_initial, const float *w2_initial, float *w1_states,
                             float *w2_states, float *y, int seq_len, int d, int d_hidden, float lp_p,
                             float sign_sharpness, float lambda_2, float lq_q) {
    const MirasArgs a{k_mem, v_mem, q_mem, alpha, theta, nullptr, nullptr, seq_len, d, d_hidden, 0,
                      lp_p, sign_sharpness, lambda_2, lq_q};
    miras_forward("mlp_forward_lp_f32_cuda", a, w1_initial, w2_initial, w1_states, w2_states, y);
}

void mlp_forward_huber_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem, const float *alpha,
                                const float *theta, const float *w1_initial, const float *w2_initial,
                                const float *w1_boundary, const float *w2_boundary, float *w1_states, float *w2_states,
                                float *y, int seq_len, int d, int d_hidden, float huber_delta, float lambda_local,
                                float lambda_2) {
    const MirasArgs a{k_mem, v_mem, q_mem, alpha, theta, w1_boundary, w2_boundary, seq_len, d, d_hidden, 1,
                      huber_delta, lambda_local, lambda_2, 2.0f};
    miras_forward("mlp_forward_huber_f32_cuda", a, w1_initial, w2_initial, w1_states, w2_states, y);
}

void mlp_backward_lp_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem, const float *alpha,
                              const float *theta, const float *w1_states, const float *w2_states, const float *d_y,
                              float *d_k_mem, float *d_v_mem, float *d_q_mem, float *d_alpha, float *d_theta,
                              float *d_w1_initial, float *d_w2_initial, int seq_len, int d, int d_hidden, float lp_p,
                              float sign_sharpness, float lambda_2, float lq_q) {
    if (fabsf(lq_q - 2.0f) > 1e-6f) {   // moneta_backward.cu:547-552
        fail("mlp_backward_lp_f32_cuda: lq_q=%.4f but only q=2.0 (L2 retention) is supported.", lq_q);
        return;
    }
    const MirasArgs a{k_mem, v_mem, q_mem, alpha, theta, nullptr, nullptr, seq_len, d, d_hidden, 0,
                      lp_p, sign_sharpness, lambda_2, 2.0f};
    miras_backward("mlp_backward_lp_f32_cuda", a, w1_states, w2_states, d_y, d_k_mem, d_v_mem, d_q_mem, d_alpha,
                   d_theta, d_w1_initial, d_w2_initial);
}

void mlp_backward_huber_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem, const float *alpha,
                                 const float *theta, const float *w1_states, const float *w2_states,
                                 const float *w1_boundary, const float *w2_boundary, const float *d_y, float *d_k_mem,
                                 float *d_v_mem, float *d_q_mem, float *d_alpha, float *d_theta, float *d_w1_initial,
                                 float *d_w2_initial, int seq_len, int d, int d_hidden, float huber_delta,
                                 float lambda_local, float lambda_2) {
    const MirasArgs a{k_mem, v_mem, q_mem, alpha, theta, w1_boundary, w2_boundary, seq_len, d, d_hidden, 1,
                      huber_delta, lambda_local, lambda_2, 2.0f};
    miras_backward("mlp_backward_huber_f32_cuda", a, w1_states, w2_states, d_y, d_k_mem, d_v_mem, d_q_mem, d_alpha,
                   d_theta, d_w1_initial, d_w2_initial);
}

}  // extern "C"
