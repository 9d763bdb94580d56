// Phase-2 kernels of the reference's split chunkwise path: the per-token
// recurrence (forward) and the reverse token sweep (backward) of ONE chunk, with
// the chunk's prediction errors supplied by the caller (computed there with a
// GEMM against the chunk-start M plus error_subtract_clip).
//   core/kernels/{titans,delta}_phase2_forward.cu, {titans,delta}_phase2_backward.cu
//
// One workgroup of 4*d threads per chain in the row-quad layout: lane (r, cq)
// holds columns [cq*d/4, (cq+1)*d/4) of row r of M, S and their adjoints.  The
// next token's k, q, error row and gates are loaded one token ahead.
#include <hip/hip_runtime.h>
#include <math.h>

#include "../../include/nl_hecate_ffi.h"
#include "lane_ops.h"
#include "quad_rows.h"
#include "runtime.h"

namespace nlh {
namespace {

// ||M||_F over the workgroup; every thread gets the value.  slot: [2][8] floats.
template <int NW>
__device__ __forceinline__ float block_sum(float x, float *slot, int wave, int lane) {
    x = wave_allreduce(x);
    if (lane == 0) slot[wave] = x;
    lds_barrier();
    float s = 0.f;
#pragma unroll
    for (int w = 0; w < NW; w++) s += slot[w];
    return s;
}

template <int D, bool HAS_S>
__global__ __launch_bounds__(4 * D) void phase2_fwd_kernel(
    const float *__restrict__ k_mem, const float *__restrict__ q_mem, const float *__restrict__ alpha,
    const float *__restrict__ theta, const float *__restrict__ eta, const float *__restrict__ errors,
    float *__restrict__ m_work, float *__restrict__ s_work, float *__restrict__ m_chunk_states,
    float *__restrict__ s_chunk_states, float *__restrict__ y, int seq_len, int chunk_size, int chunk_idx,
    float m_norm_max, int project) {
    constexpr int CP = D / 4, NW = (4 * D + 63) / 64, DD = D * D;
    __shared__ float slot[2][8];
    const int tid = threadIdx.x, r = tid >> 2, cq = tid & 3, c0 = cq * CP, wave = tid >> 6, lane = tid & 63;
    const size_t b = blockIdx.x;
    const int num_chunks = (seq_len + chunk_size - 1) / chunk_size;
    const int t_start = chunk_idx * chunk_size, C = min(chunk_size, seq_len - t_start);
    const size_t eo = r * D + c0;
    float M[CP], S[CP];
    lds_read<CP>(M, m_work + b * DD + eo);
    vec_store<CP>(m_chunk_states + (b * (num_chunks + 1) + chunk_idx) * DD + eo, M);
    if (HAS_S) {
        lds_read<CP>(S, s_work + b * DD + eo);
        vec_store<CP>(s_chunk_states + (b * (num_chunks + 1) + chunk_idx) * DD + eo, S);
    }
    const float *kb = k_mem + (b * seq_len + t_start) * D, *qb = q_mem + (b * seq_len + t_start) * D;
    const float *eb = errors + b * (size_t)chunk_size * D;
    const size_t g0 = b * seq_len + t_start;
    float kc[CP], qc[CP], e_r, al, th, et = 0.f;
    auto load = [&](int tl, float (&k_)[CP], float (&q_)[CP], float &e_, float &al_, float &th_, float &et_) {
        lds_read<CP>(k_, kb + (size_t)tl * D + c0);
        lds_read<CP>(q_, qb + (size_t)tl * D + c0);
        e_ = eb[(size_t)tl * D + r];
        al_ = alpha[g0 + tl]; th_ = theta[g0 + tl];
        if (HAS_S) et_ = eta[g0 + tl];
    };
    if (C > 0) load(0, kc, qc, e_r, al, th, et);
    for (int tl = 0; tl < C; tl++) {
        float kn[CP], qn[CP], en = 0.f, aln = 0.f, thn = 0.f, etn = 0.f;
        if (tl + 1 < C) load(tl + 1, kn, qn, en, aln, thn, etn);
        const float keep = 1.f - al, se = -th * e_r;
        float sq = 0.f;
#pragma unroll
        for (int i = 0; i < CP; i++) {
            if (HAS_S) {
                S[i] = fmaf(se, kc[i], et * S[i]);
                M[i] = fmaf(keep, M[i], S[i]);
            } else {
                M[i] = fmaf(se, kc[i], keep * M[i]);
            }
            sq = fmaf(M[i], M[i], sq);
        }
        if (project) {   // per-token Frobenius projection (core/kernels/m_norm_project.cuh)
            const float nrm = sqrtf(block_sum<NW>(sq, slot[tl & 1], wave, lane));
            if (nrm > m_norm_max) {
                const float sc = m_norm_max / nrm;
#pragma unroll
                for (int i = 0; i < CP; i++) M[i] *= sc;
            }
        }
        const float y_r = quad_allreduce(dotn<CP>(M, qc));
        if (cq == 0) y[(g0 + tl) * D + r] = y_r;
        if (tl + 1 < C) {
#pragma unroll
            for (int i = 0; i < CP; i++) { kc[i] = kn[i]; qc[i] = qn[i]; }
            e_r = en; al = aln; th = thn; et = etn;
        }
    }
    vec_store<CP>(m_work + b * DD + eo, M);
    if (HAS_S) vec_store<CP>(s_work + b * DD + eo, S);
    if (chunk_idx == num_chunks - 1) {
        vec_store<CP>(m_chunk_states + (b * (num_chunks + 1) + num_chunks) * DD + eo, M);
        if (HAS_S) vec_store<CP>(s_chunk_states + (b * (num_chunks + 1) + num_chunks) * DD + eo, S);
    }
}

// Backward of one chunk.  d_M / d_S [batch, d*d] persist across chunks (in/out), d_M0 is
// written; m_recompute / s_recompute [batch, chunk_size+1, d*d] receive the replayed states.
template <int D, bool HAS_S>
__global__ __launch_bounds__(4 * D) void phase2_bwd_kernel(
    const float *__restrict__ k_mem, const float *__restrict__ q_mem, const float *__restrict__ alpha,
    const float *__restrict__ theta, const float *__restrict__ eta, const float *__restrict__ errors,
    const float *__restrict__ m_chunk_states, const float *__restrict__ s_chunk_states,
    const float *__restrict__ d_y, float *__restrict__ d_k, float *__restrict__ d_v, float *__restrict__ d_q,
    float *__restrict__ d_alpha, float *__restrict__ d_theta, float *__restrict__ d_eta, float *__restrict__ d_M,
    float *__restrict__ d_S, float *__restrict__ d_M0, float *m_recompute, float *s_recompute, int seq_len,
    int chunk_size, int chunk_idx, float m_norm_max, int project) {
    constexpr int CP = D / 4, NW = (4 * D + 63) / 64, DD = D * D;
    __shared__ float slot[2][8];
    __shared__ __align__(16) float colp[2][2][NW][D];   // [parity][dq | dk][wave][column]
    __shared__ float scl[2][NW][4];                    // [parity][wave][d_alpha, d_eta, d_theta]
    const int tid = threadIdx.x, r = tid >> 2, cq = tid & 3, c0 = cq * CP, wave = tid >> 6, lane = tid & 63;
    const size_t b = blockIdx.x;
    const int num_chunks = (seq_len + chunk_size - 1) / chunk_size;
    const int t_start = chunk_idx * chunk_size, C = min(chunk_size, seq_len - t_start);
    const size_t eo = r * D + c0;
    float *mr = m_recompute + b * (size_t)(chunk_size + 1) * DD + eo;
    float *sr = HAS_S ? s_recompute + b * (size_t)(chunk_size + 1) * DD + eo : nullptr;
    const float *kb = k_mem + (b * seq_len + t_start) * D, *qb = q_mem + (b * seq_len + t_start) * D;
    const float *dyb = d_y + (b * seq_len + t_start) * D;
    const float *eb = errors + b * (size_t)chunk_size * D;
    const size_t g0 = b * seq_len + t_start;

    // replay the chunk's states from the boundary state with the given errors
    float M[CP], S[CP], M0[CP];
    lds_read<CP>(M, m_chunk_states + (b * (num_chunks + 1) + chunk_idx) * DD + eo);
#pragma unroll
    for (int i = 0; i < CP; i++) { M0[i] = M[i]; S[i] = 0.f; }
    vec_store<CP>(mr, M);
    if (HAS_S) {
        lds_read<CP>(S, s_chunk_states + (b * (num_chunks + 1) + chunk_idx) * DD + eo);
        vec_store<CP>(sr, S);
    }
    for (int tl = 0; tl < C; tl++) {
        float kc[CP];
        lds_read<CP>(kc, kb + (size_t)tl * D + c0);
        const float keep = 1.f - alpha[g0 + tl], se = -theta[g0 + tl] * eb[(size_t)tl * D + r];
        const float et = HAS_S ? eta[g0 + tl] : 0.f;
        float sq = 0.f;
#pragma unroll
        for (int i = 0; i < CP; i++) {
            if (HAS_S) {
                S[i] = fmaf(se, kc[i], et * S[i]);
                M[i] = fmaf(keep, M[i], S[i]);
            } else {
                M[i] = fmaf(se, kc[i], keep * M[i]);
            }
            sq = fmaf(M[i], M[i], sq);
        }
        if (project) {
            const float nrm = sqrtf(block_sum<NW>(sq, slot[tl & 1], wave, lane));
            if (nrm > m_norm_max) {
                const float sc = m_norm_max / nrm;
#pragma unroll
                for (int i = 0; i < CP; i++) M[i] *= sc;
            }
        }
        vec_store<CP>(mr + (size_t)(tl + 1) * DD, M);
        if (HAS_S) vec_store<CP>(sr + (size_t)(tl + 1) * DD, S);
    }

    // reverse sweep; every thread re-reads only what it wrote itself
    float dM[CP], dS[CP], dM0[CP];
    lds_read<CP>(dM, d_M + b * DD + eo);
#pragma unroll
    for (int i = 0; i < CP; i++) { dM0[i] = 0.f; dS[i] = 0.f; }
    if (HAS_S) lds_read<CP>(dS, d_S + b * DD + eo);
    const int rho = lane >> 4, coff = c0 + (CP / 2) * (rho >> 1) + (CP / 4) * (rho & 1);
    const bool cwriter = ((lane & 15) >> 2) == 0;
    for (int tl = C - 1; tl >= 0; tl--) {
        const int pb = tl & 1;
        float kc[CP], qc[CP], mn[CP], mt[CP], st[CP];
        lds_read<CP>(kc, kb + (size_t)tl * D + c0);
        lds_read<CP>(qc, qb + (size_t)tl * D + c0);
        lds_read<CP>(mn, mr + (size_t)(tl + 1) * DD);
        lds_read<CP>(mt, mr + (size_t)tl * DD);
        if (HAS_S) lds_read<CP>(st, sr + (size_t)tl * DD);
        const float dy_r = dyb[(size_t)tl * D + r], e_r = eb[(size_t)tl * D + r];
        const float al = alpha[g0 + tl], th = theta[g0 + tl], et = HAS_S ? eta[g0 + tl] : 0.f;
        float colv[CP], out[CP / 4], pa = 0.f, pe = 0.f;
#pragma unroll
        for (int i = 0; i < CP; i++) {
            dM[i] = fmaf(dy_r, qc[i], dM[i]);          // d_M += dy q^T
            colv[i] = mn[i] * dy_r;                    // d_q = M_{t+1}^T dy
            if (HAS_S) dS[i] += dM[i];
            pa = fmaf(mt[i], dM[i], pa);               // d_alpha = -<M_t, d_M>
            if (HAS_S) pe = fmaf(st[i], dS[i], pe);    // d_eta = <S_t, d_S>
        }
        rows_reduce_scatter<CP>(colv, out);
        if (cwriter) {
#pragma unroll
            for (int i = 0; i < CP / 4; i++) colp[pb][0][wave][coff + i] = out[i];
        }
        const float (&G)[CP] = HAS_S ? dS : dM;        // adjoint of the rank-1 term
        const float w_r = quad_allreduce(dotn<CP>(G, kc));
        const float derr = -th * w_r;                  // d_err = -theta G k
        float pt = 0.25f * e_r * w_r;                  // d_theta = -e^T G k (each row counted once)
#pragma unroll
        for (int i = 0; i < CP; i++) colv[i] = fmaf(-th * G[i], e_r, M0[i] * derr);   // d_k
        rows_reduce_scatter<CP>(colv, out);
        if (cwriter) {
#pragma unroll
            for (int i = 0; i < CP / 4; i++) colp[pb][1][wave][coff + i] = out[i];
        }
        pa = wave_allreduce(pa); pe = wave_allreduce(pe); pt = wave_allreduce(pt);
        if (lane == 0) { scl[pb][wave][0] = pa; scl[pb][wave][1] = pe; scl[pb][wave][2] = pt; }
        if (cq == 0) d_v[(g0 + tl) * D + r] = -derr;
        const float keep = 1.f - al;
#pragma unroll
        for (int i = 0; i < CP; i++) {
            dM0[i] = fmaf(derr, kc[i], dM0[i]);
            dM[i] *= keep;
            if (HAS_S) dS[i] *= et;
        }
        lds_barrier();
        if (tid < D) {
            float xq = 0.f, xk = 0.f;
#pragma unroll
            for (int w = 0; w < NW; w++) { xq += colp[pb][0][w][tid]; xk += colp[pb][1][w][tid]; }
            d_q[(g0 + tl) * D + tid] = xq;
            d_k[(g0 + tl) * D + tid] = xk;
        } else if (tid == D) {
            float xa = 0.f, xe = 0.f, xt = 0.f;
#pragma unroll
            for (int w = 0; w < NW; w++) { xa += scl[pb][w][0]; xe += scl[pb][w][1]; xt += scl[pb][w][2]; }
            d_alpha[g0 + tl] = -xa;
            d_theta[g0 + tl] = -xt;
            if (HAS_S) d_eta[g0 + tl] = xe;
        }
    }
    // the error path lands on the chunk-start matrix
#pragma unroll
    for (int i = 0; i < CP; i++) dM[i] += dM0[i];
    vec_store<CP>(d_M + b * DD + eo, dM);
    vec_store<CP>(d_M0 + b * DD + eo, dM0);
    if (HAS_S) vec_store<CP>(d_S + b * DD + eo, dS);
}

bool check_p2(const char *fn, int seq_len, int d, int batch, int chunk_size, int chunk_idx) {
    if (seq_len <= 0 || batch <= 0 || chunk_size <= 0) {
        fail("%s: seq_len, batch_size and chunk_size must be positive", fn);
        return false;
    }
    if (d != 16 && d != 32 && d != 64) { fail("%s: d=%d unsupported (16, 32, 64)", fn, d); return false; }
    const int nc = (seq_len + chunk_size - 1) / chunk_size;
    if (chunk_idx < 0 || chunk_idx >= nc) { fail("%s: chunk_idx=%d outside [0, %d)", fn, chunk_idx, nc); return false; }
    return true;
}
inline int project_on(float m_norm_max) { return m_norm_max > 0.f && m_norm_max < 1e30f; }

}  // namespace
}  // namespace nlh

using namespace nlh;

#define NLH_P2_DISPATCH(KERN, HAS, ...)                                                                      \
    do {                                                                                                     \
        if (d == 16) hipLaunchKernelGGL((KERN<16, HAS>), dim3(batch_size), dim3(64), 0, stream(), __VA_ARGS__);  \
        else if (d == 32) hipLaunchKernelGGL((KERN<32, HAS>), dim3(batch_size), dim3(128), 0, stream(), __VA_ARGS__); \
        else hipLaunchKernelGGL((KERN<64, HAS>), dim3(batch_size), dim3(256), 0, stream(), __VA_ARGS__);     \
        check_launch(#KERN);                                                                                 \
    } while (0)

extern "C" void titans_phase2_forward_f32_cuda(const float *k_mem, const float *q_mem, const float *alpha,
                                               const float *theta, const float *eta, const float *errors,
                                               float *m_work, float *s_work, float *m_chunk_states,
                                               float *s_chunk_states, float *y, int seq_len, int d, int batch_size,
                                               int chunk_size, int chunk_idx, float m_norm_max) {
    if (!check_p2("titans_phase2_forward_f32_cuda", seq_len, d, batch_size, chunk_size, chunk_idx)) return;
    NLH_P2_DISPATCH(phase2_fwd_kernel, true, k_mem, q_mem, alpha, theta, eta, errors, m_work, s_work,
                    m_chunk_states, s_chunk_states, y, seq_len, chunk_size, chunk_idx, m_norm_max,
                    project_on(m_norm_max));
}

extern "C" void delta_phase2_forward_f32_cuda(const float *k_mem, const float *q_mem, const float *alpha,
                                              const float *theta, const float *errors, float *m_work,
                                              float *m_chunk_states, float *y, int seq_len, int d, int batch_size,
                                              int chunk_size, int chunk_idx, float m_norm_max) {
    if (!check_p2("delta_phase2_forward_f32_cuda", seq_len, d, batch_size, chunk_size, chunk_idx)) return;
    NLH_P2_DISPATCH(phase2_fwd_kernel, false, k_mem, q_mem, alpha, theta, (const float *)nullptr, errors, m_work,
                    (float *)nullptr, m_chunk_states, (float *)nullptr, y, seq_len, chunk_size, chunk_idx,
                    m_norm_max, project_on(m_norm_max));
}

extern "C" void titans_phase2_backward_f32_cuda(const float *k_mem, const float *q_mem, const float *alpha,
                                                const float *theta, const float *eta, const float *errors,
                                                const float *m_chunk_states, const float *s_chunk_states,
                                                const float *d_y, float *d_k_mem, float *d_v_mem, float *d_q_mem,
                                                float *d_alpha, float *d_theta, float *d_eta, float *d_M,
                                                float *d_S, float *d_M0, float *m_recompute, float *s_recompute,
                                                int seq_len, int d, int batch_size, int chunk_size, int chunk_idx,
                                                float m_norm_max) {
    if (!check_p2("titans_phase2_backward_f32_cuda", seq_len, d, batch_size, chunk_size, chunk_idx)) return;
    NLH_P2_DISPATCH(phase2_bwd_kernel, true, k_mem, q_mem, alpha, theta, eta, errors, m_chunk_states,
                    s_chunk_states, d_y, d_k_mem, d_v_mem, d_q_mem, d_alpha, d_theta, d_eta, d_M, d_S, d_M0,
                    m_recompute, s_recompute, seq_len, chunk_size, chunk_idx, m_norm_max, project_on(m_norm_max));
}

extern "C" void delta_phase2_backward_f32_cuda(const float *k_mem, const float *q_mem, const float *alpha,
                                               const float *theta, const float *errors,
                                               const float *m_chunk_states, const float *d_y, float *d_k_mem,
                                               float *d_v_mem, float *d_q_mem, float *d_alpha, float *d_theta,
                                               float *d_M, float *d_M0, float *m_recompute, int seq_len, int d,
                                               int batch_size, int chunk_size, int chunk_idx, float m_norm_max) {
    if (!check_p2("delta_phase2_backward_f32_cuda", seq_len, d, batch_size, chunk_size, chunk_idx)) return;
    NLH_P2_DISPATCH(phase2_bwd_kernel, false, k_mem, q_mem, alpha, theta, (const float *)nullptr, errors,
                    m_chunk_states, (const float *)nullptr, d_y, d_k_mem, d_v_mem, d_q_mem, d_alpha, d_theta,
                    (float *)nullptr, d_M, (float *)nullptr, d_M0, m_recompute, (float *)nullptr, seq_len,
                    chunk_size, chunk_idx, m_norm_max, project_on(m_norm_max));
}
