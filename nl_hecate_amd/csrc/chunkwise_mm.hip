// Frozen-M0 chunkwise Titans / Delta rule in matrix form on the fp32 matrix
// cores (v_mfma_f32_16x16x4_f32), head size 64, chunks of up to 64 tokens.
//
// Semantics are those of core/kernels/titans_chunkwise_forward.cu and
// titans_chunkwise_backward.cu (errors of a chunk taken against the chunk-start
// M0; S and M then evolve per token; y_t reads M after token t's update) with
// error_clip and the M-norm projection off.  Because e_t = M0 k_t - v_t does not
// depend on the evolving state, the token recurrence inside a chunk is linear
// with scalar coefficients and unrolls into dense products.  With
//   r[j,t]  = prod_{i=j+1..t} (1-alpha_i)        bb[j,t] = prod_{i=j+1..t} eta_i
//   c[t,j]  = sum_{m=j..t} r[m,t] bb[j,m]        (weight of token j's rank-1 term in M_t)
//   a_t = prod_{i<=t}(1-alpha_i),  h_t = prod_{i<=t} eta_i,  beta_t = sum_{m<=t} r[m,t] h_m
// the state after token t is
//   M_t = a_t M0 + beta_t S0 - sum_{j<=t} theta_j c[t,j] e_j k_j^T
//   S_t = h_t S0           - sum_{j<=t} theta_j bb[j,t] e_j k_j^T
// so  Y = a.(Q M0^T) + beta.(Q S0^T) + (W . (Q K^T)) E,   W[t,j] = -theta_j c[t,j] (j <= t),
// and the end-of-chunk state is an affine map of (M0, S0) whose matrices depend
// on the chunk's K, V and gates only:
//   M' = M0 (a_L I + K^T diag(wM) K) + beta_L S0 - (V.wM)^T K,   wM_j = -theta_j c[L-1,j]
//   S' = M0 (        K^T diag(wS) K) + h_L    S0 - (V.wS)^T K,   wS_j = -theta_j bb[j,L-1]
// Three passes: (1) per chunk, in parallel, the four 64x64 matrices of that map;
// (2) a short sequential scan over chunks (two 32x64x64 products per step and
// row block) that writes the chunk-start states; (3) per chunk, in parallel, Y.
// The backward has the same shape: the adjoint scan uses the same (symmetric)
// matrices, and everything else is chunk-local.
//
// Delta rule = the same formulas with eta = 0 and S0 = 0.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/nl_hecate_ffi.h"
#include "chunkwise_chain.h"
#include "chunkwise_grads.h"
#include "chunkwise_guard.h"
#include "mm_coef.h"
#include "mm_tiles.h"
#include "rule_common.h"
#include "runtime.h"

namespace nlh {
namespace {

using namespace mmt;

// Per-chunk scratch written by the local passes and read by the scans:
//   loc  [chain][chunk][4][64*64]: T_a, T_b, C_1, C_2      locs [chain][chunk][4]: a_L, beta_L, h_L
constexpr size_t kLocMats = 4;

// ── pass 1 (forward) / shared with the backward: chunk-local matrices ───────
// T_a = a_L I + K^T diag(wM) K,  T_b = K^T diag(wS) K  (both symmetric);
// forward also C_1 = -(V.wM)^T K, C_2 = -(V.wS)^T K.
#define NLH_STRIP_ORIGIN() \
    const int w = threadIdx.x >> 6, m0 = 16 * (w >> 1), n0 = 32 * (w & 1), nh = w & 1; \
    (void)nh

template <class TIn>
__global__ __launch_bounds__(kThr) void cw_local_fwd_kernel(const TIn *__restrict__ k, const TIn *__restrict__ v,
                                                            const float *__restrict__ alpha,
                                                            const float *__restrict__ theta,
                                                            const float *__restrict__ eta, float *__restrict__ loc,
                                                            float *__restrict__ locs, int s, int C, int nc,
                                                            int has_s) {
    __shared__ float Ks[MAT], Vs[MAT];
    __shared__ Coef cf;
    __shared__ float wM[CW], wS[CW];
    const int chain = blockIdx.x / nc, ci = blockIdx.x % nc, t0 = ci * C, L = min(C, s - t0);
    const size_t tok = (size_t)chain * s + t0;
    {
        Tile<TIn> tk, tv;
        fetch(tk, k + tok * HD, L);
        fetch(tv, v + tok * HD, L);
        const Gates gt = fetch_gates(alpha + tok, theta + tok, eta + tok, L, has_s != 0);
        load_gates(cf, gt);
        coefficients(cf, gt, L, nullptr, nullptr, nullptr);
        commit(Ks, tk);
        commit(Vs, tv);
    }
    __syncthreads();
    if (threadIdx.x < CW) {
        wM[threadIdx.x] = -cf.th[threadIdx.x] * cf.cl[threadIdx.x];
        wS[threadIdx.x] = -cf.th[threadIdx.x] * cf.bl[threadIdx.x];
    }
    const float aL = cf.a[L - 1], betaL = cf.beta[L - 1], hL = cf.h[L - 1];
    if (threadIdx.x == 0) {
        float *sc = locs + ((size_t)chain * nc + ci) * 4;
        sc[0] = aL; sc[1] = betaL; sc[2] = hL; sc[3] = 0.f;
    }
    __syncthreads();
    NLH_STRIP_ORIGIN();
    float *out = loc + ((size_t)chain * nc + ci) * kLocMats * HD * HD;
    auto bK = [&](int kk, int n) { return Ks[kk * LDM + n0 + n]; };
#pragma unroll 1
    for (int o = 0; o < 4; o++) {
        const float *Am = o < 2 ? Ks : Vs;
        const float *wv = (o & 1) ? wS : wM;
        Strip acc = zero_strip();
        mma(acc, [&](int m, int kk) { return Am[kk * LDM + m0 + m] * wv[kk]; }, bK);
        for_c(acc, [&](int r, int c, float &x) {
            const int row = m0 + r, col = n0 + c;
            float y = o < 2 ? x : -x;
            if (o == 0 && row == col) y += aL;
            out[(size_t)o * HD * HD + row * HD + col] = y;
        });
    }
}

// ── pass 2: scan over chunks, one workgroup per (chain, 32-row block) ────────
// FWD:  X1' = X1 T_a + s1 X2 + C_1,  X2' = X1 T_b + s2 X2 + C_2,  (s1, s2) = (beta_L, h_L)
//       states[chain][c+1] = f(states[chain][c]), slot 0 = initial state
// BWD:  X1' = X1 T_a + X2 T_b + C_1, X2' = s1 X1 + s2 X2 + C_2
//       states[chain][c] = g(states[chain][c+1]), slot nc = 0
// Eight strips per step: (product 0/1) x (16-row half) x (32-column half).
template <bool FWD>
__global__ __launch_bounds__(kThr) void cw_scan_kernel(const float *__restrict__ init1,
                                                       const float *__restrict__ init2,
                                                       const float *__restrict__ loc,
                                                       const float *__restrict__ locs, float *__restrict__ st1,
                                                       float *__restrict__ st2, int nc, int has_s) {
    __shared__ float X1[32 * LDM], X2[32 * LDM], Ta[MAT], Tb[MAT], part[4][16 * 33];
    const int chain = blockIdx.x >> 1, r0 = 32 * (blockIdx.x & 1);
    const int w = threadIdx.x >> 6, which = w >> 2, m0 = 16 * ((w >> 1) & 1), n0 = 32 * (w & 1), pidx = w & 3;
    float *s1p = st1 + (size_t)chain * (nc + 1) * HD * HD, *s2p = st2 ? st2 + (size_t)chain * (nc + 1) * HD * HD : nullptr;
    for (int e = threadIdx.x; e < 32 * 64; e += kThr) {
        const int rr = e >> 6, cc = e & 63;
        float x1 = 0.f, x2 = 0.f;
        if (FWD) {
            x1 = init1[(size_t)chain * HD * HD + (r0 + rr) * HD + cc];
            if (has_s) x2 = init2[(size_t)chain * HD * HD + (r0 + rr) * HD + cc];
        }
        X1[rr * LDM + cc] = x1; X2[rr * LDM + cc] = x2;
        const size_t slot = FWD ? 0 : nc;
        s1p[slot * HD * HD + (r0 + rr) * HD + cc] = x1;
        if (s2p) s2p[slot * HD * HD + (r0 + rr) * HD + cc] = x2;
    }
    // Operands of step+1 (two 64x64 matrices, this wave's strip of the additive term, the two
    // scalars) are fetched into registers while step runs, so a step costs no HBM round trip.
    Tile<float> ta, tb;
    Strip cnext = zero_strip(), cadd;
    float scn = 0.f, s1, s2;   // lanes 4 j + 1, 2 of scn: the two scalars of the next step
    auto prefetch = [&](int step) {
        const int ci = FWD ? step : nc - 1 - step;
        const float *lc = loc + ((size_t)chain * nc + ci) * kLocMats * HD * HD;
        const float *sc = locs + ((size_t)chain * nc + ci) * 4;
        fetch(ta, lc, 64);
        fetch(tb, lc + HD * HD, 64);
        // a vector load (lane-dependent address) on purpose: a scalar load would share a counter with the LDS reads of
        // the step's product, which would then wait for it to come back from memory
        scn = sc[threadIdx.x & 3];
        const float *Cm = lc + (FWD ? 2 + which : (which ? 3 : 2)) * HD * HD;
        for_c(cnext, [&](int r, int c, float &x) { x = Cm[(r0 + m0 + r) * HD + n0 + c]; });
    };
    prefetch(0);
    for (int step = 0; step < nc; step++) {
        const int ci = FWD ? step : nc - 1 - step;
        __syncthreads();  // previous step's readers of Ta/Tb and writers of X1/X2 are done
        commit(Ta, ta);
        commit(Tb, tb);
        s1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, scn), 1));
        s2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, scn), 2));
        cadd = cnext;
        __syncthreads();
        if (step + 1 < nc) prefetch(step + 1);
        Strip acc = zero_strip(), out = zero_strip();
        const float *T = which ? Tb : Ta;
        const float *Xs = (FWD || !which) ? X1 : X2;
        mma(acc, [&](int m, int kk) { return Xs[(m0 + m) * LDM + kk]; },
            [&](int kk, int n) { return T[kk * LDM + n0 + n]; });
        if (FWD) {
            const float sx = which ? s2 : s1;
            for_c(out, [&](int r, int c, float &x) { x = sx * X2[(m0 + r) * LDM + n0 + c]; });
#pragma unroll
            for (int i = 0; i < 4; i++) { out.t[0][i] += acc.t[0][i] + cadd.t[0][i]; out.t[1][i] += acc.t[1][i] + cadd.t[1][i]; }
        } else if (which) {
            for_c(acc, [&](int r, int c, float &x) { part[pidx][r * 33 + c] = x; });
            for_c(out, [&](int r, int c, float &x) {
                x = s1 * X1[(m0 + r) * LDM + n0 + c] + s2 * X2[(m0 + r) * LDM + n0 + c];
            });
#pragma unroll
            for (int i = 0; i < 4; i++) { out.t[0][i] += cadd.t[0][i]; out.t[1][i] += cadd.t[1][i]; }
        }
        __syncthreads();  // all reads of the old X1/X2 are done; partial products are in LDS
        if (!FWD && !which) {
            for_c(out, [&](int r, int c, float &x) { x = part[pidx][r * 33 + c]; });
#pragma unroll
            for (int i = 0; i < 4; i++) { out.t[0][i] += acc.t[0][i] + cadd.t[0][i]; out.t[1][i] += acc.t[1][i] + cadd.t[1][i]; }
        }
        float *Xd = which ? X2 : X1;
        float *gd = which ? s2p : s1p;
        const size_t slot = FWD ? ci + 1 : ci;
        for_c(out, [&](int r, int c, float &x) {
            Xd[(m0 + r) * LDM + n0 + c] = x;
            if (gd) gd[slot * HD * HD + (r0 + m0 + r) * HD + n0 + c] = x;
        });
    }
}

// ── pass 3 (forward): outputs of one chunk ──────────────────────────────────
// TRACK: also leaves the ChainTracks of chunkwise_chain.h behind (per-token squared error norms per half of the
// memory rows, eight partial sums of squares of the chunk-start states per chunk).
template <class TIn, bool TRACK>
__global__ __launch_bounds__(kThr) void cw_out_fwd_kernel(const TIn *__restrict__ k, const TIn *__restrict__ v,
                                                          const TIn *__restrict__ q,
                                                          const float *__restrict__ alpha,
                                                          const float *__restrict__ theta,
                                                          const float *__restrict__ eta,
                                                          const float *__restrict__ m_states,
                                                          const float *__restrict__ s_states,
                                                          float *__restrict__ y, int s, int C, int nc, int has_s,
                                                          int ntask, ChainTracks tr) {
    extern __shared__ float smem[];
    float *Ks = smem, *Qs = Ks + MAT, *Es = Qs + MAT, *Ms = Es + MAT, *Ss = Ms + MAT, *Cc = Ss + MAT;
    __shared__ Coef cf;
    NLH_STRIP_ORIGIN();
    // Persistent over chunk tasks: the tiles and gates of the next task are fetched into
    // registers while the current one computes, so no task waits for HBM.
    Tile<TIn> tk, tq, tv;
    Tile<float> tm, ts;
    Gates gt;
    auto fetch_task = [&](int task) {
        const int chain = task / nc, ci = task % nc, t0 = ci * C, L = min(C, s - t0);
        const size_t tok = (size_t)chain * s + t0;
        gt = fetch_gates(alpha + tok, theta + tok, eta + tok, L, has_s != 0);
        fetch(tk, k + tok * HD, L);
        fetch(tq, q + tok * HD, L);
        fetch(tv, v + tok * HD, L);
        fetch(tm, m_states + ((size_t)chain * (nc + 1) + ci) * HD * HD, 64);
        if (has_s) fetch(ts, s_states + ((size_t)chain * (nc + 1) + ci) * HD * HD, 64);
    };
    // contiguous task range per workgroup: consecutive chunks of a chain share pages and cache lines
    const int per = (ntask + (int)gridDim.x - 1) / (int)gridDim.x, task_lo = blockIdx.x * per,
              task_hi = min(ntask, task_lo + per);
    if (task_lo < task_hi) fetch_task(task_lo);
    for (int task = task_lo; task < task_hi; task++) {
    const int chain = task / nc, ci = task % nc, t0 = ci * C, L = min(C, s - t0);
    const size_t tok = (size_t)chain * s + t0;
    load_gates(cf, gt);
    coefficients(cf, gt, L, Cc, nullptr, nullptr);
    commit(Ks, tk);
    commit(Qs, tq);
    commit(Es, tv);
    commit(Ms, tm);
    if (has_s) commit(Ss, ts);
    if (TRACK) {   // this wave's share of the sums of squares of the chunk-start states, from the staged registers
        float msq = 0.f, ssq = 0.f;
#pragma unroll
        for (int it = 0; it < 2; it++) {
            msq += tm.x[it].x * tm.x[it].x + tm.x[it].y * tm.x[it].y + tm.x[it].z * tm.x[it].z + tm.x[it].w * tm.x[it].w;
            if (has_s) ssq += ts.x[it].x * ts.x[it].x + ts.x[it].y * ts.x[it].y + ts.x[it].z * ts.x[it].z + ts.x[it].w * ts.x[it].w;
        }
        msq = wave_allreduce(msq);
        ssq = wave_allreduce(ssq);
        if ((threadIdx.x & 63) == 0)
            *reinterpret_cast<float2 *>(tr.nrm + (((size_t)chain * nc + ci) * 8 + w) * 2) = make_float2(msq, ssq);
    }
    __syncthreads();
    if (task + 1 < task_hi) fetch_task(task + 1);
    {
        // E[t][i] = sum_k K[t][k] M0[i][k] - V[t][i]   (in place over V: strips are disjoint per wave)
        Strip e = zero_strip(), p = zero_strip();
        mma(e, [&](int m, int kk) { return Ks[(m0 + m) * LDM + kk]; },
            [&](int kk, int n) { return Ms[(n0 + n) * LDM + kk]; });
        // P[t][j] = sum_k Q[t][k] K[j][k];  Pw = W.P over the coefficient matrix, W[t][j] = -theta_j c[t][j]
        mma(p, [&](int m, int kk) { return Qs[(m0 + m) * LDM + kk]; },
            [&](int kk, int n) { return Ks[(n0 + n) * LDM + kk]; });
        for_c(e, [&](int r, int c, float &x) { float *d = Es + (m0 + r) * LDM + n0 + c; x -= *d; *d = x; });
        for_c(p, [&](int r, int c, float &x) { float *d = Cc + (m0 + r) * LDM + n0 + c; *d = -cf.th[n0 + c] * *d * x; });
        if (TRACK) {   // squared error norm of the strip's 16 tokens over its 32 memory rows
            for_c(e, [&](int, int, float &x) { x *= x; });
            strip_row_sums(e);
            if (row_writer()) {
                float *eo = tr.e2 + (((size_t)chain * 2 + nh) * nc + ci) * CW + m0;
#pragma unroll
                for (int i = 0; i < 4; i++) eo[row_of(i)] = e.t[0][i];
            }
        }
    }
    __syncthreads();
    const float *Pw = Cc;
    Strip y0 = zero_strip(), y1 = zero_strip(), y2 = zero_strip();
    mma(y0, [&](int m, int kk) { return Qs[(m0 + m) * LDM + kk]; },
        [&](int kk, int n) { return Ms[(n0 + n) * LDM + kk]; });
    if (has_s)
        mma(y1, [&](int m, int kk) { return Qs[(m0 + m) * LDM + kk]; },
            [&](int kk, int n) { return Ss[(n0 + n) * LDM + kk]; });
    mma(y2, [&](int m, int kk) { return Pw[(m0 + m) * LDM + kk]; },
        [&](int kk, int n) { return Es[kk * LDM + n0 + n]; });
#pragma unroll
    for (int tl = 0; tl < 2; tl++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int row = m0 + row_of(i), col = n0 + 16 * tl + (threadIdx.x & 15);
            if (row < L)
                y[(tok + row) * HD + col] = cf.a[row] * y0.t[tl][i] + cf.beta[row] * y1.t[tl][i] + y2.t[tl][i];
        }
    __syncthreads();   // LDS is rewritten by the next task
    }
}

// ── backward, chunk-local pass: what the adjoint scan needs ─────────────────
//   T_a, T_b as in the forward (the chunk map is right-multiplication by symmetric matrices)
//   C_1 = G0  = (a.dY)^T Q + dE_loc^T K,   dE_loc[j] = -theta_j sum_{t>=j} c[t,j] (q_t.k_j) dy_t
//   C_2 = GS0 = (beta.dY)^T Q
template <class TIn>
__global__ __launch_bounds__(kThr) void cw_local_bwd_kernel(const TIn *__restrict__ k, const TIn *__restrict__ q,
                                                            const float *__restrict__ d_y,
                                                            const float *__restrict__ alpha,
                                                            const float *__restrict__ theta,
                                                            const float *__restrict__ eta, float *__restrict__ loc,
                                                            float *__restrict__ locs, int s, int C, int nc,
                                                            int has_s, int ntask) {
    extern __shared__ float smem[];
    float *Ks = smem, *Qs = Ks + MAT, *Ds = Qs + MAT, *Cc = Ds + MAT, *El = Cc + MAT;
    __shared__ Coef cf;
    __shared__ float wM[CW], wS[CW];
    NLH_STRIP_ORIGIN();
    Tile<TIn> tk, tq;
    Tile<float> td;
    Gates gt;
    auto fetch_task = [&](int task) {
        const int chain = task / nc, ci = task % nc, t0 = ci * C, L = min(C, s - t0);
        const size_t tok = (size_t)chain * s + t0;
        gt = fetch_gates(alpha + tok, theta + tok, eta + tok, L, has_s != 0);
        fetch(tk, k + tok * HD, L);
        fetch(tq, q + tok * HD, L);
        fetch(td, d_y + tok * HD, L);
    };
    // contiguous task range per workgroup: consecutive chunks of a chain share pages and cache lines
    const int per = (ntask + (int)gridDim.x - 1) / (int)gridDim.x, task_lo = blockIdx.x * per,
              task_hi = min(ntask, task_lo + per);
    if (task_lo < task_hi) fetch_task(task_lo);
    for (int task = task_lo; task < task_hi; task++) {
    const int chain = task / nc, ci = task % nc, t0 = ci * C, L = min(C, s - t0);
    load_gates(cf, gt);
    coefficients(cf, gt, L, Cc, nullptr, nullptr);
    commit(Ks, tk);
    commit(Qs, tq);
    commit(Ds, td);
    __syncthreads();
    if (task + 1 < task_hi) fetch_task(task + 1);
    if (threadIdx.x < CW) {
        wM[threadIdx.x] = -cf.th[threadIdx.x] * cf.cl[threadIdx.x];
        wS[threadIdx.x] = -cf.th[threadIdx.x] * cf.bl[threadIdx.x];
    }
    const float aL = cf.a[L - 1], betaL = cf.beta[L - 1], hL = cf.h[L - 1];
    if (threadIdx.x == 0) {
        float *sc = locs + ((size_t)chain * nc + ci) * 4;
        sc[0] = aL; sc[1] = betaL; sc[2] = hL; sc[3] = 0.f;
    }
    __syncthreads();
    float *out = loc + ((size_t)chain * nc + ci) * kLocMats * HD * HD;
    auto bK = [&](int kk, int n) { return Ks[kk * LDM + n0 + n]; };
#pragma unroll 1
    for (int o = 0; o < 2; o++) {
        const float *wv = o ? wS : wM;
        Strip acc = zero_strip();
        mma(acc, [&](int m, int kk) { return Ks[kk * LDM + m0 + m] * wv[kk]; }, bK);
        for_c(acc, [&](int r, int c, float &x) {
            const int row = m0 + r, col = n0 + c;
            out[(size_t)o * HD * HD + row * HD + col] = x + ((o == 0 && row == col) ? aL : 0.f);
        });
    }
    {   // Cc <- c[t][j] * (q_t . k_j), in place (own strip only)
        Strip p = zero_strip();
        mma(p, [&](int m, int kk) { return Qs[(m0 + m) * LDM + kk]; },
            [&](int kk, int n) { return Ks[(n0 + n) * LDM + kk]; });
        for_c(p, [&](int r, int c, float &x) { Cc[(m0 + r) * LDM + n0 + c] *= x; });
    }
    __syncthreads();
    {   // dE_loc[j][i] = -theta_j sum_t Cc[t][j] dY[t][i]
        Strip e = zero_strip();
        mma(e, [&](int m, int kk) { return Cc[kk * LDM + m0 + m]; },
            [&](int kk, int n) { return Ds[kk * LDM + n0 + n]; });
        for_c(e, [&](int r, int c, float &x) { El[(m0 + r) * LDM + n0 + c] = -cf.th[m0 + r] * x; });
    }
    __syncthreads();
    Strip g0 = zero_strip(), gs = zero_strip();
    mma(g0, [&](int m, int kk) { return cf.a[kk] * Ds[kk * LDM + m0 + m]; },
        [&](int kk, int n) { return Qs[kk * LDM + n0 + n]; });
    mma(g0, [&](int m, int kk) { return El[kk * LDM + m0 + m]; }, bK);
    if (has_s)
        mma(gs, [&](int m, int kk) { return cf.beta[kk] * Ds[kk * LDM + m0 + m]; },
            [&](int kk, int n) { return Qs[kk * LDM + n0 + n]; });
    for_c(g0, [&](int r, int c, float &x) { out[(size_t)2 * HD * HD + (m0 + r) * HD + n0 + c] = x; });
    for_c(gs, [&](int r, int c, float &x) { out[(size_t)3 * HD * HD + (m0 + r) * HD + n0 + c] = x; });
    __syncthreads();   // LDS is rewritten by the next task
    }
}
constexpr size_t kLocalBwdLds = 5 * MAT * sizeof(float);

// ── backward, main per-chunk pass: dQ, dK, dV, dtheta; exports for the gate pass ──
//   pvec [chain][token][4] = p0, ps, -theta g1, -theta g2   xs [chain][chunk][j][t] = -theta_j (dy_t.e_j)(q_t.k_j)
//   scal [chunk][4] = <M0, dMo>, <S0, dMo>, <S0, dSo> (dMo, dSo: adjoints of the chunk's end state)
template <class TIn, bool TRACK>
__global__ __launch_bounds__(kThr) void cw_grads_bwd_kernel(
    const TIn *__restrict__ k, const TIn *__restrict__ v, const TIn *__restrict__ q, const float *__restrict__ d_y,
    const float *__restrict__ alpha, const float *__restrict__ theta, const float *__restrict__ eta,
    const float *__restrict__ m_states, const float *__restrict__ s_states, const float *__restrict__ dm_states,
    const float *__restrict__ ds_states, float *__restrict__ d_k, float *__restrict__ d_v, float *__restrict__ d_q,
    float *__restrict__ d_theta, float *__restrict__ pvec, float *__restrict__ xs, float *__restrict__ scal, int s, int C,
    int nc, int has_s, int ntask, ChainTracks tr) {
    extern __shared__ float smem[];
    float *Ks = smem, *Qs = Ks + MAT, *Ds = Qs + MAT, *Es = Ds + MAT, *Ms = Es + MAT, *B5 = Ms + MAT,
          *B6 = B5 + MAT, *B7 = B6 + MAT, *B8 = B7 + MAT;
    __shared__ Coef cf;
    __shared__ float part[5][2][CW];   // p0, ps, dtheta, g1, g2: one partial per column half
    __shared__ float dots[3][8];       // partial <M0, dMo>, <S0, dMo>, <S0, dSo> per wave (the gate pass's scalars)
    float *Ss = B5, *Cc = B6;
    NLH_STRIP_ORIGIN();
    Tile<TIn> tk, tq, tv;
    Tile<float> td, tm, ts;
    Gates gt;
    auto fetch_task = [&](int task) {
        const int chain = task / nc, ci = task % nc, t0 = ci * C, L = min(C, s - t0);
        const size_t tok = (size_t)chain * s + t0;
        const size_t st0 = ((size_t)chain * (nc + 1) + ci) * HD * HD;
        gt = fetch_gates(alpha + tok, theta + tok, eta + tok, L, has_s != 0);
        fetch(tk, k + tok * HD, L);
        fetch(tq, q + tok * HD, L);
        fetch(tv, v + tok * HD, L);
        fetch(td, d_y + tok * HD, L);
        fetch(tm, m_states + st0, 64);
        if (has_s) fetch(ts, s_states + st0, 64);
    };
    // one task per workgroup: with the task loop the compiler keeps the LDS addresses of every
    // phase live across the loop and spills
    {
    const int task = blockIdx.x;
    (void)ntask;
    const int chain = task / nc, ci = task % nc, t0 = ci * C, L = min(C, s - t0);
    const size_t tok = (size_t)chain * s + t0;
    const size_t st1 = ((size_t)chain * (nc + 1) + ci + 1) * HD * HD;
    fetch_task(task);
    load_gates(cf, gt);
    coefficients(cf, gt, L, Cc, nullptr, nullptr);
    commit(Ks, tk);
    commit(Qs, tq);
    commit(Es, tv);
    commit(Ds, td);
    commit(Ms, tm);
    if (has_s) commit(Ss, ts);
    if (TRACK) {   // as in cw_out_fwd_kernel: the chunk-start states' sums of squares, then the error norms below
        float msq = 0.f, ssq = 0.f;
#pragma unroll
        for (int it = 0; it < 2; it++) {
            msq += tm.x[it].x * tm.x[it].x + tm.x[it].y * tm.x[it].y + tm.x[it].z * tm.x[it].z + tm.x[it].w * tm.x[it].w;
            if (has_s) ssq += ts.x[it].x * ts.x[it].x + ts.x[it].y * ts.x[it].y + ts.x[it].z * ts.x[it].z + ts.x[it].w * ts.x[it].w;
        }
        msq = wave_allreduce(msq);
        ssq = wave_allreduce(ssq);
        if ((threadIdx.x & 63) == 0)
            *reinterpret_cast<float2 *>(tr.nrm + (((size_t)chain * nc + ci) * 8 + w) * 2) = make_float2(msq, ssq);
    }
    __syncthreads();
    auto publish = [&](int which, Strip &x) {   // row sums of x -> part[which][column half][row]
        strip_row_sums(x);
        if (row_writer()) {
#pragma unroll
            for (int i = 0; i < 4; i++) part[which][nh][m0 + row_of(i)] = x.t[0][i];
        }
    };
    Strip p = zero_strip(), dq = zero_strip();
    {
        Strip e = zero_strip(), ym = zero_strip(), ys = zero_strip(), r0 = zero_strip(), r1 = zero_strip();
        mma(e, [&](int m, int kk) { return Ks[(m0 + m) * LDM + kk]; },
            [&](int kk, int n) { return Ms[(n0 + n) * LDM + kk]; });
        mma(p, [&](int m, int kk) { return Qs[(m0 + m) * LDM + kk]; },
            [&](int kk, int n) { return Ks[(n0 + n) * LDM + kk]; });
        mma(ym, [&](int m, int kk) { return Ds[(m0 + m) * LDM + kk]; },
            [&](int kk, int n) { return Ms[kk * LDM + n0 + n]; });
        if (has_s)
            mma(ys, [&](int m, int kk) { return Ds[(m0 + m) * LDM + kk]; },
                [&](int kk, int n) { return Ss[kk * LDM + n0 + n]; });
        for_c(e, [&](int r, int c, float &x) { float *d = Es + (m0 + r) * LDM + n0 + c; x -= *d; *d = x; });
        if (TRACK) {
            for_c(e, [&](int, int, float &x) { x *= x; });
            strip_row_sums(e);
            if (row_writer()) {
                float *eo = tr.e2 + (((size_t)chain * 2 + nh) * nc + ci) * CW + m0;
#pragma unroll
                for (int i = 0; i < 4; i++) eo[row_of(i)] = e.t[0][i];
            }
        }
#pragma unroll
        for (int tl = 0; tl < 2; tl++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int row = m0 + row_of(i), col = n0 + 16 * tl + (threadIdx.x & 15);
                const float qv = Qs[row * LDM + col];
                r0.t[tl][i] = ym.t[tl][i] * qv;
                r1.t[tl][i] = ys.t[tl][i] * qv;
                dq.t[tl][i] = cf.a[row] * ym.t[tl][i] + cf.beta[row] * ys.t[tl][i];
            }
        publish(0, r0);
        publish(1, r1);
    }
    __syncthreads();   // E complete; S0 no longer needed
    Tile<float> tdm, tds;   // adjoint states: in flight during the next two phases
    fetch(tdm, dm_states + st1, 64);
    if (has_s) fetch(tds, ds_states + st1, 64);
    float *CP = B5, *CR = B7;
    {
        Strip r = zero_strip();
        mma(r, [&](int m, int kk) { return Ds[(m0 + m) * LDM + kk]; },
            [&](int kk, int n) { return Es[(n0 + n) * LDM + kk]; });
        float *xo = xs + ((size_t)chain * nc + ci) * CW * CW;
#pragma unroll
        for (int tl = 0; tl < 2; tl++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int row = m0 + row_of(i), col = n0 + 16 * tl + (threadIdx.x & 15);
                const float c = Cc[row * LDM + col], pv = p.t[tl][i], rv = r.t[tl][i];
                xo[col * CW + row] = -cf.th[col] * rv * pv;   // [j][t], scaled for the gate pass
                CP[row * LDM + col] = c * pv;
                CR[row * LDM + col] = c * rv;
            }
    }
    __syncthreads();   // CP, CR complete; Cc no longer needed
    mma(dq, [&](int m, int kk) { return -cf.th[kk] * CR[(m0 + m) * LDM + kk]; },
        [&](int kk, int n) { return Ks[kk * LDM + n0 + n]; });
    for_c(dq, [&](int r, int c, float &x) {
        if (m0 + r < L) d_q[(tok + m0 + r) * HD + n0 + c] = x;
    });
    float *dMs = B6, *dSs = B8;
    commit(dMs, tdm);
    if (has_s) commit(dSs, tds);
    {   // from the staged registers; M0 is still in LDS (this thread's own eight elements), S0 is not
        const float x0 = wave_allreduce(tile_dot_lds(Ms, tdm));
        const float x1 = has_s ? wave_allreduce(tile_dot(ts, tdm)) : 0.f;
        const float x2 = has_s ? wave_allreduce(tile_dot(ts, tds)) : 0.f;
        if ((threadIdx.x & 63) == 0) { dots[0][w] = x0; dots[1][w] = x1; dots[2][w] = x2; }
    }
    __syncthreads();
    if (threadIdx.x < 3) {
        const float *pp = dots[threadIdx.x];
        scal[((size_t)chain * nc + ci) * 4 + threadIdx.x] = ((pp[0] + pp[1]) + (pp[2] + pp[3])) + ((pp[4] + pp[5]) + (pp[6] + pp[7]));
    }
    {
        // Dk[j][i] = sum_t CP[t][j] dY[t][i] + cl_j (K dMo^T)[j][i] + bl_j (K dSo^T)[j][i]
        Strip dk = zero_strip(), t1 = zero_strip(), t2 = zero_strip(), rt = zero_strip();
        mma(dk, [&](int m, int kk) { return CP[kk * LDM + m0 + m]; },
            [&](int kk, int n) { return Ds[kk * LDM + n0 + n]; });
        mma(t1, [&](int m, int kk) { return Ks[(m0 + m) * LDM + kk]; },
            [&](int kk, int n) { return dMs[(n0 + n) * LDM + kk]; });
        if (has_s)
            mma(t2, [&](int m, int kk) { return Ks[(m0 + m) * LDM + kk]; },
                [&](int kk, int n) { return dSs[(n0 + n) * LDM + kk]; });
#pragma unroll
        for (int tl = 0; tl < 2; tl++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int row = m0 + row_of(i), col = n0 + 16 * tl + (threadIdx.x & 15);
                float x = dk.t[tl][i] + cf.cl[row] * t1.t[tl][i] + cf.bl[row] * t2.t[tl][i];
                rt.t[tl][i] = Es[row * LDM + col] * x;
                x *= -cf.th[row];                                 // dE = -theta_j Dk
                dk.t[tl][i] = x;
                if (row < L) d_v[(tok + row) * HD + col] = -x;    // dV = -dE
            }
        publish(2, rt);
        __syncthreads();   // every wave is done reading CP
        for_c(dk, [&](int r, int c, float &x) { CP[(m0 + r) * LDM + n0 + c] = x; });
    }
    __syncthreads();
    {
        const float *dE = B5;
        // DTe[j][n] = sum_t CR[t][j] Q[t][n] + cl_j (E dMo)[j][n] + bl_j (E dSo)[j][n]
        Strip dt = zero_strip(), t3 = zero_strip(), t4 = zero_strip(), em = zero_strip(), r3 = zero_strip(),
              r4 = zero_strip();
        mma(dt, [&](int m, int kk) { return CR[kk * LDM + m0 + m]; },
            [&](int kk, int n) { return Qs[kk * LDM + n0 + n]; });
        mma(t3, [&](int m, int kk) { return Es[(m0 + m) * LDM + kk]; },
            [&](int kk, int n) { return dMs[kk * LDM + n0 + n]; });
        if (has_s)
            mma(t4, [&](int m, int kk) { return Es[(m0 + m) * LDM + kk]; },
                [&](int kk, int n) { return dSs[kk * LDM + n0 + n]; });
        mma(em, [&](int m, int kk) { return dE[(m0 + m) * LDM + kk]; },
            [&](int kk, int n) { return Ms[kk * LDM + n0 + n]; });
#pragma unroll
        for (int tl = 0; tl < 2; tl++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int row = m0 + row_of(i), col = n0 + 16 * tl + (threadIdx.x & 15);
                const float kv = Ks[row * LDM + col];
                r3.t[tl][i] = t3.t[tl][i] * kv;
                r4.t[tl][i] = t4.t[tl][i] * kv;
                const float dte = dt.t[tl][i] + cf.cl[row] * t3.t[tl][i] + cf.bl[row] * t4.t[tl][i];
                if (row < L) d_k[(tok + row) * HD + col] = -cf.th[row] * dte + em.t[tl][i];
            }
        publish(3, r3);
        publish(4, r4);
    }
    __syncthreads();
    if (threadIdx.x < L) {
        const int t = threadIdx.x;
        d_theta[tok + t] = -(part[2][0][t] + part[2][1][t]);
        float *pv = pvec + (tok + t) * 4;
        pv[0] = part[0][0][t] + part[0][1][t];
        pv[1] = part[1][0][t] + part[1][1][t];
        pv[2] = -cf.th[t] * (part[3][0][t] + part[3][1][t]);
        pv[3] = -cf.th[t] * (part[4][0][t] + part[4][1][t]);
    }
    }
}
constexpr size_t kGradsBwdLds = 9 * MAT * sizeof(float);

// Sum over chains of st[chain][slot 0][.]: stage 1 sums `per` chains per block row into
// tmp[which][rows][4096]; stage 2 adds the rows to dst (+=).  blockIdx.z = which: the M adjoint (0) and the S
// adjoint (1) share the two launches.
__global__ void cw_add_rows_kernel(const float *__restrict__ tmp, float *__restrict__ dst0, float *__restrict__ dst1,
                                   int rows) {
    float *dst = blockIdx.z ? dst1 : dst0;
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    float x = 0.f;
    for (int r = 0; r < rows; r++) x += tmp[((size_t)blockIdx.z * rows + r) * HD * HD + e];
    dst[e] += x;
}

constexpr size_t kOutFwdLds = 6 * MAT * sizeof(float);

// One workgroup per compute unit for the kernels whose LDS footprint allows no more.
int persistent_grid(int ntask) {
    const int cus = compute_units();
    return ntask < cus ? ntask : cus;
}

struct Scratch {
    float *loc, *locs;
};
Scratch local_scratch(int batch, int nc) {
    Scratch sc;
    sc.loc = scratch(3, (size_t)batch * nc * kLocMats * HD * HD * sizeof(float));
    sc.locs = scratch(4, (size_t)batch * nc * 4 * sizeof(float));
    return sc;
}

bool check_mm_args(const char *fn, int seq_len, int d, int batch, int chunk_size) {
    if (seq_len <= 0 || batch <= 0) { fail("%s: seq_len and batch_size must be positive", fn); return false; }
    if (d != HD) { fail("%s: d=%d unsupported (the matrix-core path is built for d=64)", fn, d); return false; }
    if (chunk_size < 1 || chunk_size > CW) {
        fail("%s: chunk_size=%d unsupported (1..64)", fn, chunk_size);
        return false;
    }
    return true;
}

template <class TIn>
void forward_mm(const char *fn, const TIn *k, const TIn *v, const TIn *q, const float *alpha, const float *theta,
                const float *eta, const float *m_initial, const float *s_initial, float *m_states, float *s_states,
                float *y, int seq_len, int d, int batch, int chunk_size, bool has_s, const ChainTracks *tracks = nullptr) {
    const ErrorScope es;
    if (!check_mm_args(fn, seq_len, d, batch, chunk_size)) return;
    const int nc = ceil_div(seq_len, chunk_size);
    Scratch sc = local_scratch(batch, nc);
    if (es.failed()) return;
    static bool attr_set = false;
    if (!attr_set) {
        const size_t lds = kOutFwdLds;
        check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(cw_out_fwd_kernel<float, false>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds), "dynamic LDS size");
        check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(cw_out_fwd_kernel<float, true>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds), "dynamic LDS size");
        check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(cw_out_fwd_kernel<uint16_t, false>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds), "dynamic LDS size");
        check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(cw_out_fwd_kernel<uint16_t, true>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds), "dynamic LDS size");
        attr_set = true;
    }
    hipLaunchKernelGGL((cw_local_fwd_kernel<TIn>), dim3(batch * nc), dim3(kThr), 0, stream(), k, v, alpha, theta,
                       eta, sc.loc, sc.locs, seq_len, chunk_size, nc, (int)has_s);
    check_launch("cw_local_fwd_kernel");
    hipLaunchKernelGGL((cw_scan_kernel<true>), dim3(batch * 2), dim3(kThr), 0, stream(), m_initial, s_initial,
                       sc.loc, sc.locs, m_states, has_s ? s_states : nullptr, nc, (int)has_s);
    check_launch("cw_scan_kernel");
    if (tracks)
        hipLaunchKernelGGL((cw_out_fwd_kernel<TIn, true>), dim3(persistent_grid(batch * nc)), dim3(kThr), kOutFwdLds,
                           stream(), k, v, q, alpha, theta, eta, m_states, s_states, y, seq_len, chunk_size, nc,
                           (int)has_s, batch * nc, *tracks);
    else
        hipLaunchKernelGGL((cw_out_fwd_kernel<TIn, false>), dim3(persistent_grid(batch * nc)), dim3(kThr), kOutFwdLds,
                           stream(), k, v, q, alpha, theta, eta, m_states, s_states, y, seq_len, chunk_size, nc,
                           (int)has_s, batch * nc, ChainTracks{nullptr, nullptr});
    check_launch("cw_out_fwd_kernel");
}

template <class K>
void set_lds(K kernel, size_t bytes) {
    check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  (int)bytes), "dynamic LDS size");
}

// guard: the gradient pass also leaves the ChainTracks behind, and the call ends with the test of
// the reference's couplings on them BEFORE anything is added to d_m_initial / d_s_initial; false: a coupling may have
// fired, the caller runs the sequential kernels, which overwrite every other output.
struct BackwardGuard { float error_clip, m_norm_max; };
template <class TIn>
bool backward_mm(const char *fn, const TIn *k, const TIn *v, const TIn *q, const float *alpha, const float *theta,
                 const float *eta, const float *m_states, const float *s_states, const float *d_y, float *d_k,
                 float *d_v, float *d_q, float *d_alpha, float *d_theta, float *d_eta, float *d_m_initial,
                 float *d_s_initial, int seq_len, int d, int batch, int chunk_size, bool has_s,
                 const HeadRows *dy_rows = nullptr, const GradOut16 *out16 = nullptr, const BackwardGuard *guard = nullptr) {
    const ErrorScope es;
    if (!check_mm_args(fn, seq_len, d, batch, chunk_size)) return true;
    if (out16 && sizeof(TIn) != 2) { fail("%s: bf16 gradient slabs are served for bf16 tokens only.", fn); return true; }
    if (dy_rows && sizeof(TIn) != 2) { fail("%s: token-major d_y is served for bf16 tokens only.", fn); return true; }
    if (guard && (out16 || dy_rows)) { fail("%s: the in-pass test is served for head-major fp32 gradients only.", fn); return true; }
    ChainTracks tracks{nullptr, nullptr};
    if (guard) tracks = chain_tracks(seq_len, batch, chunk_size);
    const int nc = ceil_div(seq_len, chunk_size);
    Scratch sc{nullptr, nullptr};
    if constexpr (sizeof(TIn) == 4) sc = local_scratch(batch, nc);
    // adjoint snapshots: fp32 [batch][nc + 1][d*d] on the fp32 path; on the bf16 path the same slots hold bf16
    // snapshots followed by the fp32 gradient of the initial state [batch][d*d]
    const size_t n_snap = (size_t)batch * (nc + 1) * HD * HD, n_first = (size_t)batch * HD * HD;
    const size_t st_bytes = sizeof(TIn) == 2 ? n_snap * sizeof(uint16_t) + n_first * sizeof(float) : n_snap * sizeof(float);
    float *dm_states = scratch(5, st_bytes);
    float *ds_states = scratch(6, st_bytes);
    float *xs = scratch(7, (size_t)batch * nc * CW * CW * sizeof(float));
    float *pvec = scratch(8, (size_t)batch * seq_len * 4 * sizeof(float));
    float *scal = scratch(9, (size_t)batch * nc * 4 * sizeof(float));
    if (es.failed()) return true;
    static bool attr_set = false;
    if (!attr_set) {
        set_lds(cw_local_bwd_kernel<float>, kLocalBwdLds);
        set_lds(cw_local_bwd_kernel<uint16_t>, kLocalBwdLds);
        set_lds(cw_grads_bwd_kernel<float, false>, kGradsBwdLds);
        set_lds(cw_grads_bwd_kernel<float, true>, kGradsBwdLds);
        set_lds(cw_grads_bwd_kernel<uint16_t, false>, kGradsBwdLds);
        attr_set = true;
    }
    if constexpr (sizeof(TIn) == 2) {
        // bf16 tokens: coefficient pre-pass, adjoint scan and per-chunk gradients on the bf16 matrix cores
        const size_t nchunks = (size_t)batch * nc;
        float *tab_b = scratch(13, nchunks * chunkwise_grads_table_floats() * sizeof(float));
        float *vecs = scratch(14, nchunks * chunkwise_grads_vec_floats() * sizeof(float));
        if (es.failed()) return true;
        chunkwise_backward_coefficients(alpha, theta, eta, tab_b, vecs, seq_len, batch, chunk_size, has_s);
        uint16_t *dm_snap = reinterpret_cast<uint16_t *>(dm_states), *ds_snap = reinterpret_cast<uint16_t *>(ds_states);
        chunkwise_adjoint_bf16(k, q, d_y, tab_b, vecs, dm_snap, ds_snap, reinterpret_cast<float *>(dm_snap + n_snap),
                               reinterpret_cast<float *>(ds_snap + n_snap), seq_len, batch, chunk_size, has_s, dy_rows);
        chunkwise_grads_bf16(k, v, q, d_y, m_states, s_states, dm_snap, ds_snap, d_k, d_v, d_q, d_theta, pvec, xs,
                             scal, tab_b, vecs, seq_len, batch, chunk_size, has_s,
                             persistent_grid(batch * nc), dy_rows, out16, guard ? &tracks : nullptr);
    } else {
        hipLaunchKernelGGL((cw_local_bwd_kernel<TIn>), dim3(persistent_grid(batch * nc)), dim3(kThr), kLocalBwdLds,
                           stream(), k, q, d_y, alpha, theta, eta, sc.loc, sc.locs, seq_len, chunk_size, nc,
                           (int)has_s, batch * nc);
        check_launch("cw_local_bwd_kernel");
        hipLaunchKernelGGL((cw_scan_kernel<false>), dim3(batch * 2), dim3(kThr), 0, stream(), nullptr, nullptr,
                           sc.loc, sc.locs, dm_states, ds_states, nc, (int)has_s);
        check_launch("cw_scan_kernel");
        KernelTimer kt("cw_grads_bwd_kernel");
        if (guard)
            hipLaunchKernelGGL((cw_grads_bwd_kernel<float, true>), dim3(batch * nc), dim3(kThr), kGradsBwdLds, stream(),
                               reinterpret_cast<const float *>(k), reinterpret_cast<const float *>(v),
                               reinterpret_cast<const float *>(q), d_y, alpha, theta, eta, m_states, s_states, dm_states,
                               ds_states, d_k, d_v, d_q, d_theta, pvec, xs, scal, seq_len, chunk_size, nc, (int)has_s, batch * nc,
                               tracks);
        else
            hipLaunchKernelGGL((cw_grads_bwd_kernel<TIn, false>), dim3(batch * nc), dim3(kThr), kGradsBwdLds, stream(), k, v,
                               q, d_y, alpha, theta, eta, m_states, s_states, dm_states, ds_states, d_k, d_v, d_q, d_theta,
                               pvec, xs, scal, seq_len, chunk_size, nc, (int)has_s, batch * nc, ChainTracks{nullptr, nullptr});
        check_launch("cw_grads_bwd_kernel");
    }
    const bool packed = sizeof(TIn) == 2;   // where the gradient of the initial state sits (see above)
    const size_t chain_stride = packed ? (size_t)HD * HD : (size_t)(nc + 1) * HD * HD;
    const float *dm_first = packed ? reinterpret_cast<const float *>(reinterpret_cast<const uint16_t *>(dm_states) + n_snap)
                                   : dm_states;
    const float *ds_first = packed ? reinterpret_cast<const float *>(reinterpret_cast<const uint16_t *>(ds_states) + n_snap)
                                   : ds_states;
    const int per = 8, rows = ceil_div(batch, per);
    const int nsum = has_s && d_s_initial ? 2 : 1;
    float *tmp = scratch(10, (size_t)nsum * rows * HD * HD * sizeof(float));
    if (es.failed()) return true;
    // d_alpha, d_eta, and in the same launch the first stage of the deterministic sum of d_m_initial, d_s_initial
    chunkwise_gate_gradients(alpha, eta, pvec, xs, scal, d_alpha, d_eta, seq_len, batch, chunk_size, has_s, dm_first,
                             ds_first, chain_stride, per, nsum, tmp);
    if (guard && couplings_may_fire_tracked(k, alpha, theta, eta, tracks, has_s, seq_len, batch, chunk_size, guard->error_clip,
                                            guard->m_norm_max))
        return false;
    KernelTimer kt("cw_add_rows_kernel");
    hipLaunchKernelGGL(cw_add_rows_kernel, dim3(HD * HD / 256, 1, nsum), dim3(256), 0, stream(), tmp, d_m_initial,
                       d_s_initial, rows);
    check_launch("cw_add_rows_kernel");
    return true;
}

}  // namespace

void chunkwise_forward_mm_f32_tracked(const char *fn, const float *k, const float *v, const float *q, const float *alpha,
                                      const float *theta, const float *eta, const float *m_initial, const float *s_initial,
                                      float *m_states, float *s_states, float *y, int seq_len, int d, int batch,
                                      int chunk_size, bool has_s, const ChainTracks &tracks) {
    forward_mm<float>(fn, k, v, q, alpha, theta, eta, m_initial, s_initial, m_states, s_states, y, seq_len, d, batch,
                      chunk_size, has_s, &tracks);
}

bool chunkwise_backward_bf16_guarded(const char *fn, const uint16_t *k, const uint16_t *v, const uint16_t *q, const float *alpha,
                                     const float *theta, const float *eta, const float *m_states, const float *s_states,
                                     const float *d_y, float *d_k, float *d_v, float *d_q, float *d_alpha, float *d_theta,
                                     float *d_eta, float *d_m_initial, float *d_s_initial, int seq_len, int d, int batch,
                                     int chunk_size, bool has_s, float error_clip, float m_norm_max) {
    const BackwardGuard g{error_clip, m_norm_max};
    return backward_mm<uint16_t>(fn, k, v, q, alpha, theta, eta, m_states, s_states, d_y, d_k, d_v, d_q, d_alpha, d_theta, d_eta,
                                 d_m_initial, d_s_initial, seq_len, d, batch, chunk_size, has_s, nullptr, nullptr, &g);
}

bool chunkwise_backward_mm_f32_guarded(const char *fn, const float *k, const float *v, const float *q, const float *alpha,
                                       const float *theta, const float *eta, const float *m_states, const float *s_states,
                                       const float *d_y, float *d_k, float *d_v, float *d_q, float *d_alpha, float *d_theta,
                                       float *d_eta, float *d_m_initial, float *d_s_initial, int seq_len, int d, int batch,
                                       int chunk_size, bool has_s, float error_clip, float m_norm_max) {
    const BackwardGuard g{error_clip, m_norm_max};
    return backward_mm<float>(fn, k, v, q, alpha, theta, eta, m_states, s_states, d_y, d_k, d_v, d_q, d_alpha, d_theta, d_eta,
                              d_m_initial, d_s_initial, seq_len, d, batch, chunk_size, has_s, nullptr, nullptr, &g);
}

}  // namespace nlh

using namespace nlh;

extern "C" void titans_chunkwise_forward_bf16_rocm(const uint16_t *k_mem, const uint16_t *v_mem,
                                                   const uint16_t *q_mem, const float *alpha, const float *theta,
                                                   const float *eta, const float *m_initial,
                                                   const float *s_initial, float *m_chunk_states,
                                                   float *s_chunk_states, float *y, int seq_len, int d,
                                                   int batch_size, int chunk_size) {
    if (chunkwise_chain_forward_bf16("titans_chunkwise_forward_bf16_rocm", k_mem, v_mem, q_mem, alpha, theta, eta,
                                     m_initial, s_initial, m_chunk_states, s_chunk_states, y, seq_len, d, batch_size,
                                     chunk_size, true))
        return;
    forward_mm<uint16_t>("titans_chunkwise_forward_bf16_rocm", k_mem, v_mem, q_mem, alpha, theta, eta, m_initial,
                         s_initial, m_chunk_states, s_chunk_states, y, seq_len, d, batch_size, chunk_size, true);
}

extern "C" void titans_chunkwise_forward_mm_f32_rocm(const float *k_mem, const float *v_mem, const float *q_mem,
                                                     const float *alpha, const float *theta, const float *eta,
                                                     const float *m_initial, const float *s_initial,
                                                     float *m_chunk_states, float *s_chunk_states, float *y,
                                                     int seq_len, int d, int batch_size, int chunk_size) {
    forward_mm<float>("titans_chunkwise_forward_mm_f32_rocm", k_mem, v_mem, q_mem, alpha, theta, eta, m_initial,
                      s_initial, m_chunk_states, s_chunk_states, y, seq_len, d, batch_size, chunk_size, true);
}

extern "C" void titans_chunkwise_backward_bf16_rocm(const uint16_t *k_mem, const uint16_t *v_mem,
                                                    const uint16_t *q_mem, const float *alpha, const float *theta,
                                                    const float *eta, const float *m_chunk_states,
                                                    const float *s_chunk_states, const float *d_y, float *d_k_mem,
                                                    float *d_v_mem, float *d_q_mem, float *d_alpha, float *d_theta,
                                                    float *d_eta, float *d_m_initial, float *d_s_initial,
                                                    int seq_len, int d, int batch_size, int chunk_size) {
    backward_mm<uint16_t>("titans_chunkwise_backward_bf16_rocm", k_mem, v_mem, q_mem, alpha, theta, eta,
                          m_chunk_states, s_chunk_states, d_y, d_k_mem, d_v_mem, d_q_mem, d_alpha, d_theta, d_eta,
                          d_m_initial, d_s_initial, seq_len, d, batch_size, chunk_size, true);
}

// The same rule for a layer that keeps its tensors token-major: chain c = (level, batch element, head) with
// batch_size = levels * bs * heads chains; y_tokens [levels, bs, seq_len, heads * d] is written directly, and
// d_y_tokens is [levels, ...] of that shape (d_y_per_level != 0) or ONE [bs, seq_len, heads * d] gradient that
// every level reads.  The head-major k, v, q, gates and the gradients keep the layout of the entry points above.
static bool token_rows_ok(const char *fn, int d, int batch_size, int chunk_size, int heads, int levels) {
    if (d != HD || chunk_size < 1 || chunk_size > CW) {
        fail("%s: needs d=%d == %d and chunk_size=%d in [1, %d].", fn, d, HD, chunk_size, CW);
        return false;
    }
    if (heads < 1 || levels < 1 || batch_size % (heads * levels)) {
        fail("%s: batch_size=%d must be a multiple of heads=%d * levels=%d.", fn, batch_size, heads, levels);
        return false;
    }
    return true;
}

extern "C" void titans_chunkwise_forward_bf16_tokens_rocm(const uint16_t *k_mem, const uint16_t *v_mem,
                                                          const uint16_t *q_mem, const float *alpha,
                                                          const float *theta, const float *eta,
                                                          const float *m_initial, const float *s_initial,
                                                          float *m_chunk_states, float *s_chunk_states,
                                                          float *y_tokens, int seq_len, int d, int batch_size,
                                                          int chunk_size, int heads, int levels) {
    const char *fn = "titans_chunkwise_forward_bf16_tokens_rocm";
    if (seq_len <= 0 || batch_size <= 0) return;
    if (!token_rows_ok(fn, d, batch_size, chunk_size, heads, levels)) return;
    const HeadRows yr = token_major_rows(seq_len, HD, heads, batch_size / levels, true);
    chunkwise_chain_forward_bf16(fn, k_mem, v_mem, q_mem, alpha, theta, eta, m_initial, s_initial, m_chunk_states,
                                 s_chunk_states, y_tokens, seq_len, d, batch_size, chunk_size, true, &yr);
}

extern "C" void titans_chunkwise_backward_bf16_tokens_rocm(
    const uint16_t *k_mem, const uint16_t *v_mem, const uint16_t *q_mem, const float *alpha, const float *theta,
    const float *eta, const float *m_chunk_states, const float *s_chunk_states, const float *d_y_tokens,
    float *d_k_mem, float *d_v_mem, float *d_q_mem, float *d_alpha, float *d_theta, float *d_eta,
    float *d_m_initial, float *d_s_initial, int seq_len, int d, int batch_size, int chunk_size, int heads, int levels,
    int d_y_per_level) {
    const char *fn = "titans_chunkwise_backward_bf16_tokens_rocm";
    if (seq_len <= 0 || batch_size <= 0) return;
    if (!token_rows_ok(fn, d, batch_size, chunk_size, heads, levels)) return;
    const HeadRows dyr = token_major_rows(seq_len, HD, heads, batch_size / levels, d_y_per_level != 0);
    backward_mm<uint16_t>(fn, k_mem, v_mem, q_mem, alpha, theta, eta, m_chunk_states, s_chunk_states, d_y_tokens,
                          d_k_mem, d_v_mem, d_q_mem, d_alpha, d_theta, d_eta, d_m_initial, d_s_initial, seq_len, d,
                          batch_size, chunk_size, true, &dyr);
}

void nlh::titans_chunkwise_backward_bf16_tokens_g16(
    const uint16_t *k_mem, const uint16_t *v_mem, const uint16_t *q_mem, const float *alpha, const float *theta,
    const float *eta, const float *m_chunk_states, const float *s_chunk_states, const float *d_y_tokens,
    const GradOut16 &out, float *d_alpha, float *d_theta, float *d_eta, float *d_m_initial, float *d_s_initial, int seq_len,
    int d, int batch_size, int chunk_size, int heads, int levels, int d_y_per_level) {
    const char *fn = "titans_chunkwise_backward_bf16_tokens_g16";
    if (seq_len <= 0 || batch_size <= 0) return;
    if (!token_rows_ok(fn, d, batch_size, chunk_size, heads, levels)) return;
    const HeadRows dyr = token_major_rows(seq_len, HD, heads, batch_size / levels, d_y_per_level != 0);
    backward_mm<uint16_t>(fn, k_mem, v_mem, q_mem, alpha, theta, eta, m_chunk_states, s_chunk_states, d_y_tokens,
                          nullptr, nullptr, nullptr, d_alpha, d_theta, d_eta, d_m_initial, d_s_initial, seq_len, d,
                          batch_size, chunk_size, true, &dyr, &out);
}

extern "C" void titans_chunkwise_backward_mm_f32_rocm(const float *k_mem, const float *v_mem, const float *q_mem,
                                                      const float *alpha, const float *theta, const float *eta,
                                                      const float *m_chunk_states, const float *s_chunk_states,
                                                      const float *d_y, float *d_k_mem, float *d_v_mem,
                                                      float *d_q_mem, float *d_alpha, float *d_theta, float *d_eta,
                                                      float *d_m_initial, float *d_s_initial, int seq_len, int d,
                                                      int batch_size, int chunk_size) {
    backward_mm<float>("titans_chunkwise_backward_mm_f32_rocm", k_mem, v_mem, q_mem, alpha, theta, eta,
                       m_chunk_states, s_chunk_states, d_y, d_k_mem, d_v_mem, d_q_mem, d_alpha, d_theta, d_eta,
                       d_m_initial, d_s_initial, seq_len, d, batch_size, chunk_size, true);
}

// Delta rule (no momentum state): the same passes with eta = 0 and no S traffic.
extern "C" void delta_chunkwise_forward_bf16_rocm(const uint16_t *k_mem, const uint16_t *v_mem,
                                                  const uint16_t *q_mem, const float *alpha, const float *theta,
                                                  const float *m_initial, float *m_chunk_states, float *y,
                                                  int seq_len, int d, int batch_size, int chunk_size) {
    if (chunkwise_chain_forward_bf16("delta_chunkwise_forward_bf16_rocm", k_mem, v_mem, q_mem, alpha, theta, nullptr,
                                     m_initial, nullptr, m_chunk_states, nullptr, y, seq_len, d, batch_size,
                                     chunk_size, false))
        return;
    forward_mm<uint16_t>("delta_chunkwise_forward_bf16_rocm", k_mem, v_mem, q_mem, alpha, theta, nullptr, m_initial,
                         nullptr, m_chunk_states, nullptr, y, seq_len, d, batch_size, chunk_size, false);
}

extern "C" void delta_chunkwise_forward_mm_f32_rocm(const float *k_mem, const float *v_mem, const float *q_mem,
                                                    const float *alpha, const float *theta, const float *m_initial,
                                                    float *m_chunk_states, float *y, int seq_len, int d,
                                                    int batch_size, int chunk_size) {
    forward_mm<float>("delta_chunkwise_forward_mm_f32_rocm", k_mem, v_mem, q_mem, alpha, theta, nullptr, m_initial,
                      nullptr, m_chunk_states, nullptr, y, seq_len, d, batch_size, chunk_size, false);
}

extern "C" void delta_chunkwise_backward_bf16_rocm(const uint16_t *k_mem, const uint16_t *v_mem,
                                                   const uint16_t *q_mem, const float *alpha, const float *theta,
                                                   const float *m_chunk_states, const float *d_y, float *d_k_mem,
                                                   float *d_v_mem, float *d_q_mem, float *d_alpha, float *d_theta,
                                                   float *d_m_initial, int seq_len, int d, int batch_size,
                                                   int chunk_size) {
    backward_mm<uint16_t>("delta_chunkwise_backward_bf16_rocm", k_mem, v_mem, q_mem, alpha, theta, nullptr,
                          m_chunk_states, nullptr, d_y, d_k_mem, d_v_mem, d_q_mem, d_alpha, d_theta, nullptr,
                          d_m_initial, nullptr, seq_len, d, batch_size, chunk_size, false);
}

extern "C" void delta_chunkwise_backward_mm_f32_rocm(const float *k_mem, const float *v_mem, const float *q_mem,
                                                     const float *alpha, const float *theta,
                                                     const float *m_chunk_states, const float *d_y, float *d_k_mem,
                                                     float *d_v_mem, float *d_q_mem, float *d_alpha, float *d_theta,
                                                     float *d_m_initial, int seq_len, int d, int batch_size,
                                                     int chunk_size) {
    backward_mm<float>("delta_chunkwise_backward_mm_f32_rocm", k_mem, v_mem, q_mem, alpha, theta, nullptr,
                       m_chunk_states, nullptr, d_y, d_k_mem, d_v_mem, d_q_mem, d_alpha, d_theta, nullptr,
                       d_m_initial, nullptr, seq_len, d, batch_size, chunk_size, false);
}
