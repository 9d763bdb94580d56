// HOPE self-referential memory, chunkwise with frozen snapshots: six d x d
// memories per chain (k, v, q, eta, alpha, mem) that generate their own keys,
// values, queries and gates.  The reference has this on the CPU only
// (core/src/chunkwise_self_ref.rs:52-222 forward, :236-620 backward); here one
// workgroup owns one chain.
//
// Thread layout for head size D: 4*D threads, lane (r, cq) = (tid / 4, tid % 4)
// holds columns [cq*D/4, (cq+1)*D/4) of row r of every matrix.  A matrix-vector
// product is a per-lane dot over D/4 columns plus a sum over the quad (two DPP
// adds); vectors travel between the row-indexed and the column-indexed form
// through LDS, one barrier per token.
//
// Forward: the update equations as written.  Backward: inside a chunk every
// memory is M_c,t = F_c G_t + H_t with F_c the chunk-start snapshot and G, H
// shared by the six memories:
//     G_0 = I, G_{t+1} = (1-a_t) G_t - th_t u_t k_t^T      u = k - v (self-generated
//     H_0 = 0, H_{t+1} = (1-a_t) H_t + th_t v_t k_t^T       values: H == 0) or u = k
// so the reverse sweep carries dG, dH (and the six dF) instead of six dM and six
// dF, and only G_t, H_t have to be replayed per token.
#include <hip/hip_runtime.h>
#include <math.h>

#include "../../include/nl_hecate_ffi.h"
#include "lane_ops.h"
#include "quad_rows.h"
#include "runtime.h"

namespace nlh {
namespace {

constexpr int kTB = 16;  // tokens staged in LDS at a time

// core/src/tensor.rs:202-207, 221-227
__device__ __forceinline__ float sr_sigmoid(float x) {
    if (x >= 15.f) return 1.f;
    if (x <= -15.f) return 0.f;
    return 1.f / (1.f + expf(-x));
}
__device__ __forceinline__ float sr_softplus(float x) {
    if (x >= 15.f) return x;
    if (x <= -15.f) return 0.f;
    return logf(1.f + expf(x));
}

// ── forward ────────────────────────────────────────────────────────────────
// core/src/chunkwise_self_ref.rs:95-218.  mems [B,6,D*D] is updated in place;
// frozen [B,nc,6,D*D] receives the chunk-start snapshots; the per-token caches
// are what the backward consumes.
template <int D, bool SG>
__global__ __launch_bounds__(4 * D) void selfref_fwd_kernel(
    float *__restrict__ mems, const float *__restrict__ emb, float *__restrict__ y,
    float *__restrict__ k_cache, float *__restrict__ v_cache, float *__restrict__ q_cache,
    float *__restrict__ alpha_cache, float *__restrict__ theta_cache,
    float *__restrict__ amean_cache, float *__restrict__ emean_cache, float *__restrict__ frozen,
    int s, int C, int nc) {
    constexpr int CP = D / 4, NT = 4 * D, NW = (NT + 63) / 64, DD = D * D;
    __shared__ __align__(16) float xt[2][kTB][D];
    __shared__ __align__(16) float vec[2][3][D];
    __shared__ __align__(16) float gpart[2][8];

    const int tid = threadIdx.x, r = tid >> 2, cq = tid & 3, wave = tid >> 6, lane = tid & 63;
    const size_t b = blockIdx.x;
    float *mb = mems + b * 6 * DD + r * D + cq * CP;
    const float *xb = emb + b * (size_t)s * D;
    float *fb = frozen + b * (size_t)nc * 6 * DD + r * D + cq * CP;

    float M[6][CP], F[6][CP];
#pragma unroll
    for (int c = 0; c < 6; c++) {
        lds_read<CP>(M[c], mb + c * DD);
#pragma unroll
        for (int i = 0; i < CP; i++) F[c][i] = 0.f;
    }

    // x tiles: one float4 per thread per tile of kTB tokens
    const int xtt = tid / (D / 4), xj = (tid % (D / 4)) * 4;
    auto load_x = [&](int tile) -> float4 {
        const int t = tile * kTB + xtt;
        return t < s ? *reinterpret_cast<const float4 *>(xb + (size_t)t * D + xj) : make_float4(0, 0, 0, 0);
    };
    const int ntiles = (s + kTB - 1) / kTB;
    *reinterpret_cast<float4 *>(&xt[0][xtt][xj]) = load_x(0);
    __syncthreads();

    for (int tile = 0; tile < ntiles; tile++) {
        const int xb_cur = tile & 1;
        float4 xnext = make_float4(0, 0, 0, 0);
        if (tile + 1 < ntiles) xnext = load_x(tile + 1);
        const int nt = min(kTB, s - tile * kTB);
        for (int tt = 0; tt < nt; tt++) {
            const int t = tile * kTB + tt, pb = tt & 1;
            if (t % C == 0) {
                const int ci = t / C;
#pragma unroll
                for (int c = 0; c < 6; c++) {
#pragma unroll
                    for (int i = 0; i < CP; i++) F[c][i] = M[c][i];
                    vec_store<CP>(fb + ((size_t)ci * 6 + c) * DD, F[c]);
                }
            }
            float xc[CP];
            lds_read<CP>(xc, &xt[xb_cur][tt][cq * CP]);
            float pr[5];
#pragma unroll
            for (int c = 0; c < 5; c++) pr[c] = quad_allreduce(dotn<CP>(M[c], xc));
            const float k_r = pr[0], v_r = pr[1], q_r = pr[2];
            // eta_raw in even-cq lanes, alpha_raw in odd-cq lanes: one reduction for both sums
            const float gsum = rows_allreduce((cq & 1) ? pr[4] : pr[3]);
            if (lane < 2) gpart[pb][wave * 2 + lane] = gsum;
            if (cq < 3) {
                const float val = cq == 0 ? k_r : cq == 1 ? v_r : q_r;
                vec[pb][cq][r] = val;
                float *dst = cq == 0 ? k_cache : cq == 1 ? v_cache : q_cache;
                dst[(b * s + t) * D + r] = val;
            }
            lds_barrier();
            float em = 0.f, am = 0.f;
#pragma unroll
            for (int w = 0; w < NW; w++) { em += gpart[pb][2 * w]; am += gpart[pb][2 * w + 1]; }
            em *= 1.f / D; am *= 1.f / D;
            const float alpha = sr_sigmoid(am), theta = sr_softplus(em);
            if (tid == 0) {
                alpha_cache[b * s + t] = alpha; theta_cache[b * s + t] = theta;
                amean_cache[b * s + t] = am; emean_cache[b * s + t] = em;
            }
            float kc[CP], uc[CP], qc[CP];
            lds_read<CP>(kc, &vec[pb][0][cq * CP]);
            lds_read<CP>(qc, &vec[pb][2][cq * CP]);
            if (SG) {
                lds_read<CP>(uc, &vec[pb][1][cq * CP]);
#pragma unroll
                for (int i = 0; i < CP; i++) uc[i] = kc[i] - uc[i];
            }
            const float y_r = quad_allreduce(dotn<CP>(M[5], qc));  // read before the update (:138)
            if (cq == 3) y[(b * s + t) * D + r] = y_r;
            const float keep = 1.f - alpha;
#pragma unroll
            for (int c = 0; c < 6; c++) {
                // self-generated target F_c v: the error is F_c (k - v)  (:155-166, :200)
                float e = quad_allreduce(SG ? dotn<CP>(F[c], uc) : dotn<CP>(F[c], kc));
                if (!SG) e -= v_r;
                const float se = theta * e;
#pragma unroll
                for (int i = 0; i < CP; i++) M[c][i] = fmaf(-se, kc[i], keep * M[c][i]);
            }
        }
        if (tile + 1 < ntiles) {
            *reinterpret_cast<float4 *>(&xt[xb_cur ^ 1][xtt][xj]) = xnext;
            __syncthreads();
        }
    }
#pragma unroll
    for (int c = 0; c < 6; c++) vec_store<CP>(mb + c * DD, M[c]);
}

// ── backward ───────────────────────────────────────────────────────────────
// Staged tile arrays, [kTB][D] floats each.
enum { A_K = 0, A_V, A_Q, A_X, A_DY, A_G, A_P, A_DQ, A_DP, A_DG, A_DH, A_COUNT };

template <int D, bool SG>
__global__ __launch_bounds__(4 * D) void selfref_bwd_kernel(
    const float *__restrict__ emb, const float *__restrict__ d_y, const float *__restrict__ k_cache,
    const float *__restrict__ v_cache, const float *__restrict__ q_cache,
    const float *__restrict__ alpha_cache, const float *__restrict__ theta_cache,
    const float *__restrict__ amean_cache, const float *__restrict__ emean_cache,
    const float *__restrict__ frozen, float *__restrict__ d_emb, float *__restrict__ d_mems,
    float *gtraj, float *htraj, float *rp, int s, int C, int nc) {
    constexpr int CP = D / 4, NT = 4 * D, NW = (NT + 63) / 64, DD = D * D, V4 = D / 4, LD = D + 4;
    constexpr int TILE_F = A_COUNT * kTB * D, BND_F = 3 * D * LD;
    constexpr int RAW_F = TILE_F > BND_F ? TILE_F : BND_F;
    __shared__ __align__(16) float raw[RAW_F];
    __shared__ __align__(16) float wv[2][2][D];
    __shared__ __align__(16) float zp[2][2][NW][D];
    __shared__ __align__(16) float sp[2][NW][2];
    __shared__ __align__(16) float sc[4][kTB];
    __shared__ __align__(16) float av[2][D];
#define T_(a, tt, i) raw[((a) * kTB + (tt)) * D + (i)]

    const int tid = threadIdx.x, r = tid >> 2, cq = tid & 3, wave = tid >> 6, lane = tid & 63;
    const int c0 = cq * CP;
    const size_t b = blockIdx.x;
    const size_t tok0 = b * (size_t)s;
    float *gt_b = gtraj + b * (size_t)C * DD;
    float *ht_b = SG ? nullptr : htraj + b * (size_t)C * DD;
    float *rp_b = rp + tok0 * 4 * D;
    const int stt = tid / V4, sj = (tid % V4) * 4;  // staging slot: token, column

    float dF[4][CP], accE[CP], accA[CP], dG[CP], dH[CP];
#pragma unroll
    for (int i = 0; i < CP; i++) {
        dF[0][i] = dF[1][i] = dF[2][i] = dF[3][i] = 0.f;
        accE[i] = accA[i] = dG[i] = dH[i] = 0.f;
    }

    for (int ci = nc - 1; ci >= 0; ci--) {
        const int t0 = ci * C, L = min(C, s - t0);
        const float *fz = frozen + (b * nc + ci) * (size_t)6 * DD;
        // transposed register copies of F_k, F_v, F_q, F_mem and the column sums of F_eta, F_alpha
        float FTk[CP], FTv[CP], FTq[CP], FTm[CP], csE = 0.f, csA = 0.f;
#pragma unroll
        for (int i = 0; i < CP; i++) {
            const size_t o = (size_t)(c0 + i) * D + r;
            FTk[i] = fz[0 * DD + o]; FTv[i] = fz[1 * DD + o]; FTq[i] = fz[2 * DD + o];
            FTm[i] = fz[5 * DD + o];
            csE += fz[3 * DD + o]; csA += fz[4 * DD + o];
        }
        csE = quad_allreduce(csE); csA = quad_allreduce(csA);

        // ---- replay G_t, H_t over the chunk; products g = G x, p = G q, dp = F_mem^T dy, dq ----
        float G[CP], H[CP];
#pragma unroll
        for (int i = 0; i < CP; i++) { G[i] = (c0 + i == r) ? 1.f : 0.f; H[i] = 0.f; }
        const int ntile = (L + kTB - 1) / kTB;
        for (int tile = 0; tile < ntile; tile++) {
            const int tb = t0 + tile * kTB, nt = min(kTB, t0 + L - tb);
            __syncthreads();
            if (stt < nt) {
                const size_t o = (tok0 + tb + stt) * D + sj;
                *reinterpret_cast<float4 *>(&T_(A_K, stt, sj)) = *reinterpret_cast<const float4 *>(k_cache + o);
                *reinterpret_cast<float4 *>(&T_(A_V, stt, sj)) = *reinterpret_cast<const float4 *>(v_cache + o);
                *reinterpret_cast<float4 *>(&T_(A_Q, stt, sj)) = *reinterpret_cast<const float4 *>(q_cache + o);
                *reinterpret_cast<float4 *>(&T_(A_X, stt, sj)) = *reinterpret_cast<const float4 *>(emb + o);
                *reinterpret_cast<float4 *>(&T_(A_DY, stt, sj)) = *reinterpret_cast<const float4 *>(d_y + o);
            }
            if (tid < nt) { sc[0][tid] = alpha_cache[tok0 + tb + tid]; sc[1][tid] = theta_cache[tok0 + tb + tid]; }
            __syncthreads();
            for (int tt = 0; tt < nt; tt++) {
                const int li = tb + tt - t0;
                vec_store<CP>(gt_b + (size_t)li * DD + r * D + c0, G);
                if (!SG) vec_store<CP>(ht_b + (size_t)li * DD + r * D + c0, H);
                float xc[CP], qc[CP], dyc[CP], kc[CP];
                lds_read<CP>(xc, &T_(A_X, tt, c0));
                lds_read<CP>(qc, &T_(A_Q, tt, c0));
                lds_read<CP>(dyc, &T_(A_DY, tt, c0));
                lds_read<CP>(kc, &T_(A_K, tt, c0));
                const float g = quad_allreduce(dotn<CP>(G, xc));
                const float p = quad_allreduce(dotn<CP>(G, qc));
                const float dp = quad_allreduce(dotn<CP>(FTm, dyc));
                if (cq < 3) {
                    const float val = cq == 0 ? g : cq == 1 ? p : dp;
                    const int slot = cq == 2 ? 3 : cq;
                    rp_b[((size_t)(tb + tt) * 4 + slot) * D + r] = val;
                    if (cq == 2) T_(A_DP, tt, r) = dp;
                }
                const float k_r = T_(A_K, tt, r), v_r = T_(A_V, tt, r);
                const float u_r = SG ? k_r - v_r : k_r;
                const float keep = 1.f - sc[0][tt], th = sc[1][tt];
                const float su = th * u_r, sv = th * v_r;
#pragma unroll
                for (int i = 0; i < CP; i++) {
                    G[i] = fmaf(-su, kc[i], keep * G[i]);
                    if (!SG) H[i] = fmaf(sv, kc[i], keep * H[i]);
                }
            }
            __syncthreads();
            // dq_t = G_t^T dp_t + H_t^T dy_t: one float4 of columns per thread, rows from memory
            if (stt < nt) {
                const int li = tb + stt - t0;
                const float4 *gp = reinterpret_cast<const float4 *>(gt_b + (size_t)li * DD) + (sj >> 2);
                const float4 *hp = SG ? nullptr : reinterpret_cast<const float4 *>(ht_b + (size_t)li * DD) + (sj >> 2);
                float4 acc = make_float4(0, 0, 0, 0);
#pragma unroll 8
                for (int m = 0; m < D; m++) {
                    const float4 g4 = gp[m * V4];
                    const float a = T_(A_DP, stt, m);
                    acc.x = fmaf(g4.x, a, acc.x); acc.y = fmaf(g4.y, a, acc.y);
                    acc.z = fmaf(g4.z, a, acc.z); acc.w = fmaf(g4.w, a, acc.w);
                    if (!SG) {
                        const float4 h4 = hp[m * V4];
                        const float a2 = T_(A_DY, stt, m);
                        acc.x = fmaf(h4.x, a2, acc.x); acc.y = fmaf(h4.y, a2, acc.y);
                        acc.z = fmaf(h4.z, a2, acc.z); acc.w = fmaf(h4.w, a2, acc.w);
                    }
                }
                *reinterpret_cast<float4 *>(rp_b + ((size_t)(tb + stt) * 4 + 2) * D + sj) = acc;
            }
        }

        // ---- chunk boundary: gradients of F'_c = F_c G_L + H_L flow into dG_L, dH_L, dF_c ----
        __syncthreads();
        if (ci < nc - 1) {
            float *Fs = raw, *Bm = raw + D * LD, *GLT = raw + 2 * D * LD;
#pragma unroll
            for (int i = 0; i < CP; i++) GLT[(c0 + i) * LD + r] = G[i];
            if (r == 0) { vec_store<CP>(&av[0][c0], accE); vec_store<CP>(&av[1][c0], accA); }
            // rows of dF_eta, dF_alpha are all equal (accE, accA): rank-1 terms
#pragma unroll
            for (int i = 0; i < CP; i++) {
                dG[i] = csE * accE[i] + csA * accA[i];
                dH[i] = accE[i] + accA[i];
            }
#pragma unroll
            for (int comp = 0; comp < 4; comp++) {
                const int c = comp < 3 ? comp : 5;
                __syncthreads();
                for (int e = tid; e < DD / 4; e += NT) {
                    const int m = e / V4, j = (e % V4) * 4;
                    *reinterpret_cast<float4 *>(Fs + m * LD + j) = *reinterpret_cast<const float4 *>(fz + (size_t)c * DD + m * D + j);
                }
                vec_store<CP>(Bm + r * LD + c0, dF[comp]);
                __syncthreads();
                float nf[CP];
#pragma unroll
                for (int i = 0; i < CP; i++) { nf[i] = 0.f; if (!SG) dH[i] += dF[comp][i]; }
#pragma unroll 4
                for (int m = 0; m < D; m++) {
                    float b1[CP], b2[CP];
                    lds_read<CP>(b1, Bm + m * LD + c0);
                    lds_read<CP>(b2, GLT + m * LD + c0);
                    const float a1 = Fs[m * LD + r], a2 = Bm[r * LD + m];
#pragma unroll
                    for (int i = 0; i < CP; i++) { dG[i] = fmaf(a1, b1[i], dG[i]); nf[i] = fmaf(a2, b2[i], nf[i]); }
                }
#pragma unroll
                for (int i = 0; i < CP; i++) dF[comp][i] = nf[i];
            }
            {   // accE <- G_L accE, accA <- G_L accA (column-indexed)
                float nE[CP], nA[CP];
#pragma unroll
                for (int i = 0; i < CP; i++) nE[i] = nA[i] = 0.f;
#pragma unroll 4
                for (int m = 0; m < D; m++) {
                    float b2[CP];
                    lds_read<CP>(b2, GLT + m * LD + c0);
                    const float aE = av[0][m], aA = av[1][m];
#pragma unroll
                    for (int i = 0; i < CP; i++) { nE[i] = fmaf(aE, b2[i], nE[i]); nA[i] = fmaf(aA, b2[i], nA[i]); }
                }
#pragma unroll
                for (int i = 0; i < CP; i++) { accE[i] = nE[i]; accA[i] = nA[i]; }
            }
            __syncthreads();
        }

        // ---- reverse sweep over the chunk ----
        for (int tile = ntile - 1; tile >= 0; tile--) {
            const int tb = t0 + tile * kTB, nt = min(kTB, t0 + L - tb);
            if (stt < nt) {
                const size_t o = (tok0 + tb + stt) * D + sj;
                const float *rpt = rp_b + (size_t)(tb + stt) * 4 * D + sj;
                *reinterpret_cast<float4 *>(&T_(A_K, stt, sj)) = *reinterpret_cast<const float4 *>(k_cache + o);
                *reinterpret_cast<float4 *>(&T_(A_V, stt, sj)) = *reinterpret_cast<const float4 *>(v_cache + o);
                *reinterpret_cast<float4 *>(&T_(A_Q, stt, sj)) = *reinterpret_cast<const float4 *>(q_cache + o);
                *reinterpret_cast<float4 *>(&T_(A_X, stt, sj)) = *reinterpret_cast<const float4 *>(emb + o);
                *reinterpret_cast<float4 *>(&T_(A_DY, stt, sj)) = *reinterpret_cast<const float4 *>(d_y + o);
                *reinterpret_cast<float4 *>(&T_(A_G, stt, sj)) = *reinterpret_cast<const float4 *>(rpt);
                *reinterpret_cast<float4 *>(&T_(A_P, stt, sj)) = *reinterpret_cast<const float4 *>(rpt + D);
                *reinterpret_cast<float4 *>(&T_(A_DQ, stt, sj)) = *reinterpret_cast<const float4 *>(rpt + 2 * D);
                *reinterpret_cast<float4 *>(&T_(A_DP, stt, sj)) = *reinterpret_cast<const float4 *>(rpt + 3 * D);
            }
            if (tid < nt) {
                const size_t o = tok0 + tb + tid;
                sc[0][tid] = alpha_cache[o]; sc[1][tid] = theta_cache[o];
                const float sa = sr_sigmoid(amean_cache[o]);
                sc[2][tid] = sa * (1.f - sa) * (1.f / D);           // sigmoid'(mean) / d
                sc[3][tid] = sr_sigmoid(emean_cache[o]) * (1.f / D);  // softplus'(mean) / d
            }
            float Gt[CP], Ht[CP];
            {
                const int li = tb + nt - 1 - t0;
                lds_read<CP>(Gt, gt_b + (size_t)li * DD + r * D + c0);
                if (!SG) lds_read<CP>(Ht, ht_b + (size_t)li * DD + r * D + c0);
            }
            __syncthreads();
            for (int tt = nt - 1; tt >= 0; tt--) {
                const int pb = tt & 1, li = tb + tt - t0;
                float Gn[CP], Hn[CP];
                if (tt > 0) {
                    lds_read<CP>(Gn, gt_b + (size_t)(li - 1) * DD + r * D + c0);
                    if (!SG) lds_read<CP>(Hn, ht_b + (size_t)(li - 1) * DD + r * D + c0);
                }
                const float al = sc[0][tt], th = sc[1][tt];
                const float k_r = T_(A_K, tt, r), v_r = T_(A_V, tt, r);
                const float u_r = SG ? k_r - v_r : k_r;
                float kc[CP];
                lds_read<CP>(kc, &T_(A_K, tt, c0));
                const float w = quad_allreduce(dotn<CP>(dG, kc));
                float wh = 0.f;
                float alp = dotn<CP>(Gt, dG), thp = 0.25f * u_r * w;
                float zv[CP], zo[CP / 4];
#pragma unroll
                for (int i = 0; i < CP; i++) zv[i] = dG[i] * u_r;
                rows_reduce_scatter<CP>(zv, zo);
                const int rho = lane >> 4, zoff = c0 + (CP / 2) * (rho >> 1) + (CP / 4) * (rho & 1);
                const bool zwriter = ((lane & 15) >> 2) == 0;
                if (zwriter) {
#pragma unroll
                    for (int i = 0; i < CP / 4; i++) zp[pb][0][wave][zoff + i] = zo[i];
                }
                if (!SG) {
                    wh = quad_allreduce(dotn<CP>(dH, kc));
                    alp += dotn<CP>(Ht, dH);
                    thp -= 0.25f * v_r * wh;
#pragma unroll
                    for (int i = 0; i < CP; i++) zv[i] = dH[i] * v_r;
                    rows_reduce_scatter<CP>(zv, zo);
                    if (zwriter) {
#pragma unroll
                        for (int i = 0; i < CP / 4; i++) zp[pb][1][wave][zoff + i] = zo[i];
                    }
                }
                alp = wave_allreduce(alp);
                thp = wave_allreduce(thp);
                if (lane == 0) { sp[pb][wave][0] = alp; sp[pb][wave][1] = thp; }
                if (cq == 0) wv[pb][0][r] = w;
                if (!SG && cq == 1) wv[pb][1][r] = wh;
                lds_barrier();

                float dal = 0.f, dth = 0.f;
#pragma unroll
                for (int x = 0; x < NW; x++) { dal -= sp[pb][x][0]; dth -= sp[pb][x][1]; }
                const float da = dal * sc[2][tt], de = dth * sc[3][tt];
                float zc[CP], wc[CP], z_r = 0.f, zh_r = 0.f;
                lds_read<CP>(zc, &zp[pb][0][0][c0]);
                z_r = zp[pb][0][0][r];
#pragma unroll
                for (int x = 1; x < NW; x++) {
                    float tmp[CP];
                    lds_read<CP>(tmp, &zp[pb][0][x][c0]);
#pragma unroll
                    for (int i = 0; i < CP; i++) zc[i] += tmp[i];
                    z_r += zp[pb][0][x][r];
                }
                lds_read<CP>(wc, &wv[pb][0][c0]);
                float dkc[CP], dvc[CP];
#pragma unroll
                for (int i = 0; i < CP; i++) {
                    const float du = -th * wc[i];
                    dkc[i] = fmaf(-th, zc[i], du);
                    dvc[i] = -du;
                }
                const float du_r = -th * w;
                float dk_r = fmaf(-th, z_r, du_r), dv_r = -du_r;
                if (!SG) {
                    float zhc[CP], whc[CP];
                    lds_read<CP>(zhc, &zp[pb][1][0][c0]);
                    zh_r = zp[pb][1][0][r];
#pragma unroll
                    for (int x = 1; x < NW; x++) {
                        float tmp[CP];
                        lds_read<CP>(tmp, &zp[pb][1][x][c0]);
#pragma unroll
                        for (int i = 0; i < CP; i++) zhc[i] += tmp[i];
                        zh_r += zp[pb][1][x][r];
                    }
                    lds_read<CP>(whc, &wv[pb][1][c0]);
#pragma unroll
                    for (int i = 0; i < CP; i++) { dkc[i] = fmaf(th, zhc[i], dkc[i]); dvc[i] = th * whc[i]; }
                    dk_r = fmaf(th, zh_r, dk_r);
                    dv_r = th * wh;
                }
                float dqc[CP];
                lds_read<CP>(dqc, &T_(A_DQ, tt, c0));
                const float dq_r = T_(A_DQ, tt, r), dy_r = T_(A_DY, tt, r), dp_r = T_(A_DP, tt, r);
                float dgp = dotn<CP>(FTk, dkc);
#pragma unroll
                for (int i = 0; i < CP; i++) dgp = fmaf(FTv[i], dvc[i], fmaf(FTq[i], dqc[i], dgp));
                const float dg = quad_allreduce(dgp) + de * csE + da * csA;
                const float dh = dk_r + dv_r + dq_r + de + da;
                float xc[CP], qc[CP], gc[CP], pc[CP];
                lds_read<CP>(xc, &T_(A_X, tt, c0));
                lds_read<CP>(qc, &T_(A_Q, tt, c0));
                lds_read<CP>(gc, &T_(A_G, tt, c0));
                lds_read<CP>(pc, &T_(A_P, tt, c0));
                const float keep = 1.f - al;
#pragma unroll
                for (int i = 0; i < CP; i++) {
                    dG[i] = fmaf(dg, xc[i], fmaf(dp_r, qc[i], keep * dG[i]));
                    if (!SG) dH[i] = fmaf(dh, xc[i], fmaf(dy_r, qc[i], keep * dH[i]));
                    dF[0][i] = fmaf(dk_r, gc[i], dF[0][i]);
                    dF[1][i] = fmaf(dv_r, gc[i], dF[1][i]);
                    dF[2][i] = fmaf(dq_r, gc[i], dF[2][i]);
                    dF[3][i] = fmaf(dy_r, pc[i], dF[3][i]);
                    accE[i] = fmaf(de, gc[i], accE[i]);
                    accA[i] = fmaf(da, gc[i], accA[i]);
                }
                if (cq == 0) T_(A_DG, tt, r) = dg;
                if (!SG && cq == 1) T_(A_DH, tt, r) = dh;
                if (tt > 0) {
#pragma unroll
                    for (int i = 0; i < CP; i++) { Gt[i] = Gn[i]; if (!SG) Ht[i] = Hn[i]; }
                }
            }
            __syncthreads();
            // d_x_t = G_t^T dg_t + H_t^T dh_t
            if (stt < nt) {
                const int li = tb + stt - t0;
                const float4 *gp = reinterpret_cast<const float4 *>(gt_b + (size_t)li * DD) + (sj >> 2);
                const float4 *hp = SG ? nullptr : reinterpret_cast<const float4 *>(ht_b + (size_t)li * DD) + (sj >> 2);
                float4 acc = make_float4(0, 0, 0, 0);
#pragma unroll 8
                for (int m = 0; m < D; m++) {
                    const float4 g4 = gp[m * V4];
                    const float a = T_(A_DG, stt, m);
                    acc.x = fmaf(g4.x, a, acc.x); acc.y = fmaf(g4.y, a, acc.y);
                    acc.z = fmaf(g4.z, a, acc.z); acc.w = fmaf(g4.w, a, acc.w);
                    if (!SG) {
                        const float4 h4 = hp[m * V4];
                        const float a2 = T_(A_DH, stt, m);
                        acc.x = fmaf(h4.x, a2, acc.x); acc.y = fmaf(h4.y, a2, acc.y);
                        acc.z = fmaf(h4.z, a2, acc.z); acc.w = fmaf(h4.w, a2, acc.w);
                    }
                }
                *reinterpret_cast<float4 *>(d_emb + (tok0 + tb + stt) * D + sj) = acc;
            }
            __syncthreads();
        }
    }
    // gradients of the initial memories; rows of d_M_eta / d_M_alpha are all equal
    float *dmb = d_mems + b * 6 * DD + r * D + c0;
    vec_store<CP>(dmb + 0 * DD, dF[0]);
    vec_store<CP>(dmb + 1 * DD, dF[1]);
    vec_store<CP>(dmb + 2 * DD, dF[2]);
    vec_store<CP>(dmb + 3 * DD, accE);
    vec_store<CP>(dmb + 4 * DD, accA);
    vec_store<CP>(dmb + 5 * DD, dF[3]);
#undef T_
}

template <int D>
void launch_fwd(bool sg, int batch, float *mems, const float *emb, float *y, float *kc, float *vc, float *qc,
                float *al, float *th, float *am, float *em, float *frozen, int s, int C, int nc) {
    if (sg)
        hipLaunchKernelGGL((selfref_fwd_kernel<D, true>), dim3(batch), dim3(4 * D), 0, stream(), mems, emb, y, kc,
                           vc, qc, al, th, am, em, frozen, s, C, nc);
    else
        hipLaunchKernelGGL((selfref_fwd_kernel<D, false>), dim3(batch), dim3(4 * D), 0, stream(), mems, emb, y, kc,
                           vc, qc, al, th, am, em, frozen, s, C, nc);
    check_launch("selfref_fwd_kernel");
}

template <int D>
void launch_bwd(bool sg, int batch, const float *emb, const float *dy, const float *kc, const float *vc,
                const float *qc, const float *al, const float *th, const float *am, const float *em,
                const float *frozen, float *d_emb, float *d_mems, float *gtraj, float *htraj, float *rp, int s,
                int C, int nc) {
    KernelTimer kt("selfref_bwd_kernel");
    if (sg)
        hipLaunchKernelGGL((selfref_bwd_kernel<D, true>), dim3(batch), dim3(4 * D), 0, stream(), emb, dy, kc, vc,
                           qc, al, th, am, em, frozen, d_emb, d_mems, gtraj, htraj, rp, s, C, nc);
    else
        hipLaunchKernelGGL((selfref_bwd_kernel<D, false>), dim3(batch), dim3(4 * D), 0, stream(), emb, dy, kc, vc,
                           qc, al, th, am, em, frozen, d_emb, d_mems, gtraj, htraj, rp, s, C, nc);
    check_launch("selfref_bwd_kernel");
}

bool check_args(const char *fn, int seq_len, int d, int batch, int chunk_size) {
    if (seq_len <= 0 || batch <= 0) { fail("%s: seq_len and batch_size must be positive", fn); return false; }
    if (chunk_size < 1) { fail("%s: chunk_size must be >= 1", fn); return false; }
    if (d != 16 && d != 32 && d != 64) { fail("%s: d=%d unsupported (16, 32, 64)", fn, d); return false; }
    return true;
}

}  // namespace
}  // namespace nlh

using namespace nlh;

extern "C" void selfref_chunkwise_forward_f32_rocm(float *mems, const float *embedded, float *y, float *k_cache,
                                                   float *v_cache, float *q_cache, float *alpha_cache,
                                                   float *theta_cache, float *alpha_mean_cache,
                                                   float *eta_mean_cache, float *frozen, int seq_len, int d,
                                                   int batch_size, int chunk_size, int self_generated_values) {
    if (!check_args("selfref_chunkwise_forward_f32_rocm", seq_len, d, batch_size, chunk_size)) return;
    const int C = chunk_size > seq_len ? seq_len : chunk_size;
    const int nc = (seq_len + chunk_size - 1) / chunk_size;
    const bool sg = self_generated_values != 0;
#define NLH_FWD(DV) launch_fwd<DV>(sg, batch_size, mems, embedded, y, k_cache, v_cache, q_cache, alpha_cache, \
                                   theta_cache, alpha_mean_cache, eta_mean_cache, frozen, seq_len, C, nc)
    if (d == 16) NLH_FWD(16); else if (d == 32) NLH_FWD(32); else NLH_FWD(64);
#undef NLH_FWD
}

extern "C" void selfref_chunkwise_backward_f32_rocm(const float *embedded, const float *d_y, const float *k_cache,
                                                    const float *v_cache, const float *q_cache,
                                                    const float *alpha_cache, const float *theta_cache,
                                                    const float *alpha_mean_cache, const float *eta_mean_cache,
                                                    const float *frozen, float *d_embedded, float *d_mems,
                                                    int seq_len, int d, int batch_size, int chunk_size,
                                                    int self_generated_values) {
    if (!check_args("selfref_chunkwise_backward_f32_rocm", seq_len, d, batch_size, chunk_size)) return;
    const int C = chunk_size > seq_len ? seq_len : chunk_size;
    const int nc = (seq_len + chunk_size - 1) / chunk_size;
    const bool sg = self_generated_values != 0;
    const size_t dd = (size_t)d * d;
    const size_t traj_bytes = (size_t)batch_size * C * dd * sizeof(float);
    if (traj_bytes > ((size_t)32 << 30)) {
        fail("selfref_chunkwise_backward_f32_rocm: chunk trajectory of %zu bytes exceeds the 32 GiB scratch limit",
             traj_bytes);
        return;
    }
    float *gtraj = scratch(0, traj_bytes);
    float *htraj = sg ? nullptr : scratch(1, traj_bytes);
    float *rp = scratch(2, (size_t)batch_size * seq_len * 4 * d * sizeof(float));
    if (failed()) return;
#define NLH_BWD(DV) launch_bwd<DV>(sg, batch_size, embedded, d_y, k_cache, v_cache, q_cache, alpha_cache, \
                                   theta_cache, alpha_mean_cache, eta_mean_cache, frozen, d_embedded, d_mems, \
                                   gtraj, htraj, rp, seq_len, C, nc)
    if (d == 16) NLH_BWD(16); else if (d == 32) NLH_BWD(32); else NLH_BWD(64);
#undef NLH_BWD
}
