// Backward of the exact Titans / Delta rule from checkpoints every C <= 64 tokens, in chunk-parallel matrix form on
// the fp32 matrix cores (v_mfma_f32_16x16x4_f32), head size 64.
//
// Semantics are those of core/kernels/titans_backward.cu:66-341 run segment by segment from the checkpoints of
// core/kernels/titans_forward.cu (the schedule of core/src/gpu_backward.rs:1770-1962) with error_clip and the
// M-norm projection off: every error is taken against the CURRENT memory, u_t = M_(t-1) k_t - v_t.
//
// The rule is linear in (M, S).  Inside a chunk that starts at the checkpoint (M0, S0), with the coefficients of
// the frozen-M0 form (mm_coef.h: a, beta, h, c, bb; W[t][j] = -theta_j c[t][j], wM = W[L-1], wS_j = -theta_j
// bb[j][L-1]) and am, bm = a, beta shifted by one token (am_0 = 1, bm_0 = 0), the errors of a chunk obey a unit
// lower triangular system
//   (I - Lam) U = R,   Lam[t][j] = W[t-1][j] (k_j . k_t)  (j < t),   R = am.(K M0^T) + bm.(K S0^T) - V
// and everything else is the frozen rule with its errors replaced by U plus the terms through T = (I - Lam)^-1:
//   dU = (W.P)^T dY + wM.(K dMo^T) + wS.(K dSo^T)     dR = T^T dU      (P = Q K^T; dMo, dSo: adjoints at chunk end)
//   dV = -dR     dQ = a.(dY M0) + beta.(dY S0) + (W.tril(dY U^T)) K
//   dK = (W.tril(dY U^T))^T Q + wM.(U dMo) + wS.(U dSo) + am.(dR M0) + bm.(dR S0) + (dG + dG^T) K,
//        dG[t][j] = W[t-1][j] strict_tril(dR U^T)[t][j]
//   adjoints at chunk start:  dM' = a_L dMo + (a.dY)^T Q + (am.dR)^T K,   dS' = beta_L dMo + h_L dSo + (beta.dY)^T Q + (bm.dR)^T K
// The last line is affine in (dMo, dSo) with matrices that depend on the chunk only, so the reverse scan over the
// chunks of a chain multiplies by four 64x64 matrices per step and the rest is chunk-parallel:
//   1. ex_local_kernel   per chunk: T (blocked inverse: 16x16 diagonal blocks by substitution, then
//                        (I + N)(I + N^2) D with N = D Lam_off, N^4 = 0), U, dU_loc = (W.P)^T dY, the four matrices
//                        Phi = (w.K)^T T (m.K) and the two additive terms of the scan
//   2. ex_scan_kernel    per (chain, 16-row block): the adjoints at every chunk boundary
//   3. ex_grads_kernel   per chunk: dQ, dK, dV, dtheta and the hand-off of the gate pass
//   4. cw_gates_sweep_kernel (chunkwise_gates.hip): dalpha, deta.  The inner products <M_s, J_t> it sweeps obey the
//      rule's own recurrence with J_t = dy_t q_t^T + dR_(t+1) k_(t+1)^T, i.e. per-token terms
//      xs[s][t] = -theta_s [ (dy_t.u_s)(q_t.k_s) + (dR_(t+1).u_s)(k_(t+1).k_s) ].
// The algebra is written out and checked against the reference's token loops in float64 in tests/np_rules.py
// (titans_exact_chunk_backward).
//
// Under a finite m_norm_max / error clip the pass also leaves the ChainTracks of chunkwise_chain.h behind (|u_t|^2 per
// token, sums of squares of the checkpoints); the caller tests on them whether a coupling could have fired.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "chunkwise_chain.h"
#include "chunkwise_grads.h"
#include "chunkwise_guard.h"
#include "exact_mm.h"
#include "mm_coef.h"
#include "mm_tiles.h"
#include "rule_common.h"
#include "runtime.h"

namespace nlh {
namespace {

using namespace mmt;

// Waves w and w + 4 share a SIMD.  Products with the lower triangular T (or its transpose) cost a 16-row block
// ib + 1 (or 4 - ib) quarter products, so the row blocks are dealt out as (0, 3) and (1, 2) per SIMD.
#define NLH_STRIP_ORIGIN_OF(w) \
    const int ib = w < 4 ? w >> 1 : 3 - ((w - 4) >> 1), m0 = 16 * ib, n0 = 32 * (w & 1), nh = w & 1; \
    (void)nh
#define NLH_STRIP_ORIGIN() \
    const int w = threadIdx.x >> 6; \
    NLH_STRIP_ORIGIN_OF(w)

// per chunk, for the scan: Phi_MM, Phi_SM, Phi_MS, Phi_SS (source state, destination state), C_M, C_S
constexpr size_t kExLocMats = 6;
constexpr size_t kDD = (size_t)HD * HD;

struct ChunkVecs { float wM[CW], wS[CW], am[CW], bm[CW]; };
__device__ __forceinline__ void chunk_vectors(ChunkVecs &cv, const Coef &cf, int L) {
    const int j = threadIdx.x;
    if (j < CW) {
        cv.wM[j] = -cf.th[j] * cf.cl[j];
        cv.wS[j] = -cf.th[j] * cf.bl[j];
        cv.am[j] = j == 0 ? 1.f : (j < L ? cf.a[j - 1] : 0.f);
        cv.bm[j] = (j == 0 || j >= L) ? 0.f : cf.beta[j - 1];
    }
}

// ── pass 1: chunk-local matrices ────────────────────────────────────────────
template <bool TRACK>
__global__ __launch_bounds__(kThr) void ex_local_kernel(
    const float *__restrict__ k, const float *__restrict__ v, const float *__restrict__ q, const float *__restrict__ d_y,
    const float *__restrict__ alpha, const float *__restrict__ theta, const float *__restrict__ eta,
    const float *__restrict__ m_ckpt, const float *__restrict__ s_ckpt, float *__restrict__ loc, float *__restrict__ locs,
    float *__restrict__ Tg, float *__restrict__ Ug, float *__restrict__ dUg, int s, int C, int nc, int nck, int has_s,
    int ntask, ChainTracks tr) {
    extern __shared__ float smem[];
    float *Ks = smem, *Vs = Ks + MAT, *Qs = Vs + MAT, *Ds = Qs + MAT, *Ms = Ds + MAT, *Ss = Ms + MAT, *Cc = Ss + MAT,
          *B8 = Cc + MAT, *B9 = B8 + MAT;
    __shared__ Coef cf;
    __shared__ ChunkVecs cv;
    // Persistent over a contiguous range of chunks.  A workgroup fills the compute unit's LDS, so nothing else would
    // hide its loads: the next chunk's tiles are requested at the start of this chunk's last phase (the longest one,
    // ten products back to back) and land in LDS at the top of the next round.
    Tile<float> tk, tv, tq, td, tm, ts;
    Gates gt;
    auto fetch_task = [&](int task, int tid) {
        const int chain = task / nc, ci = task % nc, t0 = ci * C, L = min(C, s - t0);
        const size_t tok = (size_t)chain * s + t0;
        gt = fetch_gates(alpha + tok, theta + tok, eta + tok, L, has_s != 0);
        fetch(tk, k + tok * HD, L, tid);
        fetch(tv, v + tok * HD, L, tid);
        fetch(tq, q + tok * HD, L, tid);
        fetch(td, d_y + tok * HD, L, tid);
        fetch(tm, m_ckpt + ((size_t)chain * nck + ci) * kDD, 64, tid);
        if (has_s) fetch(ts, s_ckpt + ((size_t)chain * nck + ci) * kDD, 64, tid);
    };
    const int per = (ntask + (int)gridDim.x - 1) / (int)gridDim.x, task_lo = blockIdx.x * per, task_hi = min(ntask, task_lo + per);
    if (task_lo < task_hi) fetch_task(task_lo, threadIdx.x);
    for (int itask = task_lo; itask < task_hi; itask++) {
    // thread and wave index through opaque copies, once per chunk (see mm_tiles.h)
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
    const int l = tid & 63;
    int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    asm volatile("" : "+s"(w));
    NLH_STRIP_ORIGIN_OF(w);
    auto MMA = [&](Strip &acc, auto fa, auto fb) { mma(acc, fa, fb, l); };
    auto MMAR = [&](Strip &acc, auto fa, auto fb, int p0, int p1) { mma_range(acc, fa, fb, p0, p1, l); };
    auto MMAT = [&](f32x4 &acc, auto fa, auto fb, int k0) { mma_tile16(acc, fa, fb, k0, l); };
    auto FORC = [&](Strip &acc, auto f) { for_c(acc, f, l); };
    const int chain = itask / nc, ci = itask % nc, t0 = ci * C, L = min(C, s - t0);
    const size_t task = (size_t)itask;
    (void)t0;
    {
        load_gates(cf, gt);
        coefficients(cf, gt, L, Cc, nullptr, nullptr);
        commit(Ks, tk, tid);
        commit(Vs, tv, tid);
        commit(Qs, tq, tid);
        commit(Ds, td, tid);
        commit(Ms, tm, tid);
        if (has_s) commit(Ss, ts, tid);
        if (TRACK) {
            float msq = wave_allreduce(tile_dot(tm, tm)), ssq = has_s ? wave_allreduce(tile_dot(ts, ts)) : 0.f;
            if (l == 0) *reinterpret_cast<float2 *>(tr.nrm + (task * 8 + w) * 2) = make_float2(msq, ssq);
        }
    }
    __syncthreads();
    chunk_vectors(cv, cf, L);
    if (threadIdx.x == 0) {
        float *sc = locs + task * 4;
        sc[0] = cf.a[L - 1]; sc[1] = cf.beta[L - 1]; sc[2] = cf.h[L - 1]; sc[3] = 0.f;
    }
    {
        Strip g = zero_strip(), km = zero_strip(), ks = zero_strip(), p = zero_strip();
        auto aK = [&](int m, int kk) { return Ks[(m0 + m) * LDM + kk]; };
        MMA(g, aK, [&](int kk, int n) { return Ks[(n0 + n) * LDM + kk]; });
        MMA(km, aK, [&](int kk, int n) { return Ms[(n0 + n) * LDM + kk]; });
        if (has_s) MMA(ks, aK, [&](int kk, int n) { return Ss[(n0 + n) * LDM + kk]; });
        MMA(p, [&](int m, int kk) { return Qs[(m0 + m) * LDM + kk]; }, [&](int kk, int n) { return Ks[(n0 + n) * LDM + kk]; });
        __syncthreads();   // the vectors are there
#pragma unroll
        for (int tl = 0; tl < 2; tl++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int row = m0 + row_of(i, l), col = n0 + 16 * tl + (l & 15);
                // R in place over V (own strip)
                float *d = Vs + row * LDM + col;
                *d = cv.am[row] * km.t[tl][i] + cv.bm[row] * ks.t[tl][i] - *d;
                const float nth = -cf.th[col];
                B8[row * LDM + col] = (col < row) ? nth * Cc[(row - 1) * LDM + col] * g.t[tl][i] : 0.f;   // Lam
                B9[row * LDM + col] = nth * Cc[row * LDM + col] * p.t[tl][i];                            // W.P
            }
    }
    __syncthreads();
    Strip dul = zero_strip();
    MMA(dul, [&](int m, int kk) { return B9[kk * LDM + m0 + m]; }, [&](int kk, int n) { return Ds[kk * LDM + n0 + n]; });
    if (w < 4 && l < 16) {
        // D_b = (I - Lam_bb)^-1 by substitution: lane c holds column c of block b = w
        const float *A = B8 + (16 * w) * LDM + 16 * w;
        float x[16];
#pragma unroll
        for (int r = 0; r < 16; r++) {
            float acc = r == l ? 1.f : 0.f;
#pragma unroll
            for (int j = 0; j < r; j++) acc = fmaf(A[r * LDM + j], x[j], acc);
            x[r] = acc;
        }
        float *Dd = Ms + (16 * w) * LDM + 16 * w + l;
#pragma unroll
        for (int r = 0; r < 16; r++) Dd[r * LDM] = x[r];
    }
    __syncthreads();
    {   // N = D Lam_off -> Ss; dU_loc -> B9 and out
#pragma unroll
        for (int tl = 0; tl < 2; tl++) {
            const int jb = 2 * (w & 1) + tl;
            f32x4 nacc = {0.f, 0.f, 0.f, 0.f};
            if (jb < ib)
                MMAT(nacc, [&](int m, int kk) { return Ms[(m0 + m) * LDM + kk]; },
                           [&](int kk, int n) { return B8[kk * LDM + 16 * jb + n]; }, 16 * ib);
#pragma unroll
            for (int i = 0; i < 4; i++) Ss[(m0 + row_of(i, l)) * LDM + 16 * jb + (l & 15)] = nacc[i];
        }
        float *go = dUg + task * kDD;
        FORC(dul, [&](int r, int c, float &x) {
            B9[(m0 + r) * LDM + n0 + c] = x;
            go[(m0 + r) * HD + n0 + c] = x;
        });
    }
    __syncthreads();
    auto aN = [&](int m, int kk) { return Ss[(m0 + m) * LDM + kk]; };
    // N is strictly block lower triangular (blocks of 16): its powers need only the block products that can be non-zero
#pragma unroll
    for (int tl = 0; tl < 2; tl++) {   // N^2 -> B8
        const int jb = 2 * (w & 1) + tl;
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        for (int kb = jb + 1; kb < ib; kb++)
            MMAT(acc, aN, [&](int kk, int n) { return Ss[kk * LDM + 16 * jb + n]; }, 16 * kb);
#pragma unroll
        for (int i = 0; i < 4; i++) B8[(m0 + row_of(i, l)) * LDM + 16 * jb + (l & 15)] = acc[i];
    }
    __syncthreads();
#pragma unroll
    for (int tl = 0; tl < 2; tl++) {   // X = (I + N)(I + N^2) = I + N + N^2 + N N^2 -> Cc
        const int jb = 2 * (w & 1) + tl;
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        for (int kb = jb + 2; kb < ib; kb++)
            MMAT(acc, aN, [&](int kk, int n) { return B8[kk * LDM + 16 * jb + n]; }, 16 * kb);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int row = m0 + row_of(i, l), col = 16 * jb + (l & 15);
            Cc[row * LDM + col] = acc[i] + Ss[row * LDM + col] + B8[row * LDM + col] + (row == col ? 1.f : 0.f);
        }
    }
    __syncthreads();
    {   // T = X D -> Ss and out
        float *go = Tg + task * kDD;
#pragma unroll
        for (int tl = 0; tl < 2; tl++) {
            const int jb = 2 * (w & 1) + tl;
            f32x4 t = {0.f, 0.f, 0.f, 0.f};
            MMAT(t, [&](int m, int kk) { return Cc[(m0 + m) * LDM + kk]; },
                       [&](int kk, int n) { return Ms[kk * LDM + 16 * jb + n]; }, 16 * jb);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int row = m0 + row_of(i, l), col = 16 * jb + (l & 15);
                Ss[row * LDM + col] = t[i];
                go[row * HD + col] = t[i];
            }
        }
    }
    __syncthreads();
    {   // U = T R -> out;  Z1 = T (am.K) -> B8,  Z2 = T (bm.K) -> Ms
        Strip u = zero_strip(), z1 = zero_strip(), z2 = zero_strip();
        auto aT = [&](int m, int kk) { return Ss[(m0 + m) * LDM + kk]; };
        // T is lower triangular: row block ib contracts over the first ib + 1 blocks of 16 (taken in pairs)
        const int pe = (ib >> 1) + 1;
        MMAR(u, aT, [&](int kk, int n) { return Vs[kk * LDM + n0 + n]; }, 0, pe);
        MMAR(z1, aT, [&](int kk, int n) { return cv.am[kk] * Ks[kk * LDM + n0 + n]; }, 0, pe);
        if (has_s) MMAR(z2, aT, [&](int kk, int n) { return cv.bm[kk] * Ks[kk * LDM + n0 + n]; }, 0, pe);
        float *go = Ug + task * kDD;
        FORC(u, [&](int r, int c, float &x) { go[(m0 + r) * HD + n0 + c] = x; });
        FORC(z1, [&](int r, int c, float &x) { B8[(m0 + r) * LDM + n0 + c] = x; });
        if (has_s) FORC(z2, [&](int r, int c, float &x) { Ms[(m0 + r) * LDM + n0 + c] = x; });
        if (TRACK) {   // squared error norm of the strip's 16 tokens over its 32 memory rows
            FORC(u, [&](int, int, float &x) { x *= x; });
            strip_row_sums(u);
            if (row_writer(l)) {
                float *eo = tr.e2 + (((size_t)chain * 2 + nh) * nc + ci) * CW + m0;
#pragma unroll
                for (int i = 0; i < 4; i++) eo[row_of(i, l)] = u.t[0][i];
            }
        }
    }
    __syncthreads();
    if (itask + 1 < task_hi) fetch_task(itask + 1, tid);
    float *out = loc + task * kExLocMats * kDD;
    auto store = [&](int which, Strip &x) {
        FORC(x, [&](int r, int c, float &y) { out[(size_t)which * kDD + (m0 + r) * HD + n0 + c] = y; });
    };
    // The four scan matrices leave in the order in which the scan's waves take them as the second operand of their
    // product: lane 16 (k / 16) + n % 16 of the wave for column half n / 32 takes, as its 16-byte piece j = (k % 16) / 2,
    // the elements (k, n), (k, n + 16), (k + 1, n), (k + 1, n + 16) with k even, n % 32 < 16.  Pieces are stored
    // [column half][j][lane], so a load instruction of the scan reads 1 KB of consecutive memory.  A lane of this strip
    // holds two pieces.
    auto store_operand = [&](int which, const Strip &x) {
        float *o = out + (size_t)which * kDD + (size_t)(((nh * 8 + 2 * (l >> 4)) * 64 + 16 * ib + (l & 15)) * 4);
        *reinterpret_cast<float4 *>(o) = make_float4(x.t[0][0], x.t[1][0], x.t[0][1], x.t[1][1]);
        *reinterpret_cast<float4 *>(o + 64 * 4) = make_float4(x.t[0][2], x.t[1][2], x.t[0][3], x.t[1][3]);
    };
    // one product at a time (no unrolling over the outputs): the next chunk's tiles are in registers during this phase
#pragma unroll 1
    for (int o = 0; o < (has_s ? 4 : 1); o++) {   // Phi_MM, Phi_SM, Phi_MS, Phi_SS = (w.K)^T Z
        const float *wv = (o & 1) ? cv.wS : cv.wM, *Z = (o & 2) ? Ms : B8;
        Strip x = zero_strip();
        MMA(x, [&](int m, int kk) { return wv[kk] * Ks[kk * LDM + m0 + m]; }, [&](int kk, int n) { return Z[kk * LDM + n0 + n]; });
        store_operand(o, x);
    }
#pragma unroll 1
    for (int o = 0; o < (has_s ? 2 : 1); o++) {   // C_M = (a.dY)^T Q + dU_loc^T Z1,  C_S = (beta.dY)^T Q + dU_loc^T Z2
        const float *vec = o ? cf.beta : cf.a, *Z = o ? Ms : B8;
        Strip x = zero_strip();
        MMA(x, [&](int m, int kk) { return vec[kk] * Ds[kk * LDM + m0 + m]; }, [&](int kk, int n) { return Qs[kk * LDM + n0 + n]; });
        MMA(x, [&](int m, int kk) { return B9[kk * LDM + m0 + m]; }, [&](int kk, int n) { return Z[kk * LDM + n0 + n]; });
        store(4 + o, x);
    }
    __syncthreads();   // LDS is rewritten by the next chunk
    }
}
constexpr size_t kExLocalLds = 9 * MAT * sizeof(float);

// ── pass 2: reverse scan over the chunks of a chain, one workgroup per 16-row block ──
//   X1' = a_L X1 + X1 Phi_MM + X2 Phi_SM + C_M,   X2' = beta_L X1 + h_L X2 + X1 Phi_MS + X2 Phi_SS + C_S
// ends [chain][nc + 1][64*64]: slot c = adjoint of the state at the start of chunk c (slot nc = 0, slot 0 = the
// gradient of the initial state, also written to first [chain][64*64]).
// Wave w: destination w / 4, source (w / 2) % 2, column half w % 2: one 16 x 64 x 32 product per step.  The two
// source waves of a destination strip then finish one 16 x 16 tile of it each (they swap the other tile through
// LDS), so every wave runs the same instructions: per step 12 loads, then 4 stores.  That matters: the memory
// counter of this hardware counts loads and stores together and in order, and the wait for the next step's operands
// at the top of a step can only leave this step's stores in flight if their number is the same on every path
// (with the stores under a branch the wait was for all of them: 4 of a step's 9 thousand cycles).
// Without momentum (the Delta rule) there is one state and one matrix: the two source waves split its contraction.
template <bool HAS_S>
__global__ __launch_bounds__(kThr) void ex_scan_kernel(const float *__restrict__ loc, const float *__restrict__ locs,
                                                       float *__restrict__ em, float *__restrict__ es_,
                                                       float *__restrict__ first_m, float *__restrict__ first_s, int nc) {
    __shared__ float X1[16 * LDM], X2[16 * LDM], part[8 * 256];
    // the four row blocks of a chain sit 8 workgroups apart: consecutive workgroups go to consecutive XCDs, so the
    // four share one XCD's L2 for the chunk matrices they all read
    const int chain0 = (blockIdx.x & 7) + 8 * (blockIdx.x >> 5), rb0 = (blockIdx.x >> 3) & 3;
    const bool whole = (int)(blockIdx.x | 31) < (int)gridDim.x;   // a full group of 32 workgroups
    const int chain = whole ? chain0 : blockIdx.x >> 2, r0 = 16 * (whole ? rb0 : blockIdx.x & 3);
    const int l = threadIdx.x & 63, w = threadIdx.x >> 6, dst = w >> 2, src = (w >> 1) & 1, half = w & 1;
    const int col = 32 * half + 16 * src + (l & 15), rw = 4 * (l >> 4);   // the tile this wave finishes: rows rw + i
    float *emp = em + (size_t)chain * (nc + 1) * kDD, *esp = HAS_S ? es_ + (size_t)chain * (nc + 1) * kDD : nullptr;
    for (int e = threadIdx.x; e < 16 * 64; e += kThr) {
        const int rr = e >> 6, cc = e & 63;
        X1[rr * LDM + cc] = 0.f;
        X2[rr * LDM + cc] = 0.f;
        emp[(size_t)nc * kDD + (r0 + rr) * HD + cc] = 0.f;
        if (HAS_S) esp[(size_t)nc * kDD + (r0 + rr) * HD + cc] = 0.f;
    }
    const bool active = HAS_S || dst == 0;   // wave-uniform; the idle waves of the Delta rule only keep the barriers
    constexpr int NB = HAS_S ? 8 : 4;   // 16-byte pieces of the operand per lane and step
    // The wave's second operand (a 64 x 32 piece of one chunk matrix) comes straight from memory in the lane order
    // of the product (ex_local_kernel writes it that way), requested a step ahead.
    float4 bn[NB], bc[NB];
    f32x4 cn = {0.f, 0.f, 0.f, 0.f}, out = {0.f, 0.f, 0.f, 0.f};
    float scn = 0.f;   // lanes 4 j + 0, 1, 2: a_L, beta_L, h_L of the next step
    auto prefetch = [&](int ci) {
        const float *lc = loc + ((size_t)chain * nc + ci) * kExLocMats * kDD;
        const float *sc = locs + ((size_t)chain * nc + ci) * 4;
        const float4 *bp = reinterpret_cast<const float4 *>(lc + (size_t)(HAS_S ? dst * 2 + src : 0) * kDD) +
                           (half * 8 + (HAS_S ? 0 : 4 * src)) * 64 + l;
#pragma unroll
        for (int j = 0; j < NB; j++) bn[j] = bp[j * 64];
        // a vector load (lane-dependent address) on purpose: a scalar load would join the LDS reads under one counter
        // that only knows "all done", and the first product of the step would wait for it to come back from memory
        scn = sc[l & 3];
        const float *Cm = lc + (4 + dst) * kDD + (r0 + rw) * HD + col;
#pragma unroll
        for (int i = 0; i < 4; i++) cn[i] = Cm[i * HD];
    };
    if (active) prefetch(nc - 1);
    __syncthreads();
    float *Xd = dst ? X2 : X1;
    float *gd = (dst ? esp : emp) + (size_t)(r0 + rw) * HD + col;
    const float *Xs = ((HAS_S && src) ? X2 : X1) + (l & 15) * LDM + 16 * (l >> 4) + (HAS_S ? 0 : 8 * src);
    for (int ci = nc - 1; ci >= 0; ci--) {
        if (active) {
#pragma unroll
            for (int j = 0; j < NB; j++) bc[j] = bn[j];
            const float aL = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, scn), 0)),
                        bL = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, scn), 1)),
                        hL = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, scn), 2));
            const f32x4 ca = cn;
            if (ci > 0) prefetch(ci - 1);
            f32x4 acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
#pragma unroll
            for (int j = 0; j < NB; j++) {   // contraction indices 16 (l / 16) + 2 j, + 1 (+ 8 for the second Delta wave)
                const float a0 = Xs[2 * j], a1 = Xs[2 * j + 1];
                acc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(a0, bc[j].x, acc[0], 0, 0, 0);
                acc[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a0, bc[j].y, acc[1], 0, 0, 0);
                acc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(a1, bc[j].z, acc[0], 0, 0, 0);
                acc[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a1, bc[j].w, acc[1], 0, 0, 0);
            }
            // the tile the partner wave (w ^ 2) finishes goes to LDS; this wave keeps tile `src`
            const f32x4 mine = src ? acc[1] : acc[0], theirs = src ? acc[0] : acc[1];
#pragma unroll
            for (int i = 0; i < 4; i++) part[w * 256 + i * 64 + l] = theirs[i];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float x1 = X1[(rw + i) * LDM + col];
                out[i] = mine[i] + ca[i] + (dst ? bL * x1 + hL * X2[(rw + i) * LDM + col] : aL * x1);
            }
        }
        __syncthreads();   // every read of the old X1 / X2 is done; the partners' tiles are in LDS
        if (active) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                out[i] += part[(w ^ 2) * 256 + i * 64 + l];
                Xd[(rw + i) * LDM + col] = out[i];
                gd[(size_t)ci * kDD + i * HD] = out[i];
            }
        }
        __syncthreads();   // the new X1 / X2 are complete
    }
    if (!active) return;
    float *gf = (dst ? first_s : first_m) + (size_t)chain * kDD + (size_t)(r0 + rw) * HD + col;
#pragma unroll
    for (int i = 0; i < 4; i++) gf[i * HD] = out[i];
}

// ── pass 3: gradients of one chunk ──────────────────────────────────────────
//   pvec [chain][token][4] = <M0, J_t>, <S0, J_t>, -theta_t u_t^T dMo k_t, -theta_t u_t^T dSo k_t
//   xs [chain][chunk][s][t] as above     scal [chunk][4] = <M0, dMo>, <S0, dMo>, <S0, dSo>
__global__ __launch_bounds__(kThr) void ex_grads_kernel(
    const float *__restrict__ k, const float *__restrict__ q, const float *__restrict__ d_y, const float *__restrict__ alpha,
    const float *__restrict__ theta, const float *__restrict__ eta, const float *__restrict__ m_ckpt,
    const float *__restrict__ s_ckpt, const float *__restrict__ Tg, const float *__restrict__ Ug,
    const float *__restrict__ dUg, const float *__restrict__ em, const float *__restrict__ es_, float *__restrict__ d_k,
    float *__restrict__ d_v, float *__restrict__ d_q, float *__restrict__ d_theta, float *__restrict__ pvec,
    float *__restrict__ xs, float *__restrict__ scal, int s, int C, int nc, int nck, int has_s, int ntask) {
    extern __shared__ float smem[];
    float *Ks = smem, *Qs = Ks + MAT, *Ds = Qs + MAT, *Ts = Ds + MAT, *Us = Ts + MAT, *A1 = Us + MAT, *A2 = A1 + MAT,
          *Cc = A2 + MAT, *B9 = Cc + MAT;
    __shared__ Coef cf;
    __shared__ ChunkVecs cv;
    __shared__ float part[6][2][CW];   // row sums per column half: p0, ps, g1, g2, dam, dbm
    __shared__ float part_th[4][CW];   // column sums of dW.c per 16-row block
    __shared__ float dots[3][8];
    // Persistent over a contiguous range of chunks, as ex_local_kernel: the next chunk's nine tiles are requested at the
    // start of this chunk's last phase.
    Tile<float> tk, tq, td, tt, tu, tdm, tds, tm, ts;
    Gates gt;
    // K, Q, dY of the next chunk are requested during this chunk's last phase (more does not fit next to its
    // accumulators); the other six tiles at the top of the chunk, behind two products that need K and Q only
    auto fetch_a = [&](int task, int tid) {
        const int chain = task / nc, ci = task % nc, t0 = ci * C, L = min(C, s - t0);
        const size_t tok = (size_t)chain * s + t0;
        gt = fetch_gates(alpha + tok, theta + tok, eta + tok, L, has_s != 0);
        fetch(tk, k + tok * HD, L, tid);
        fetch(tq, q + tok * HD, L, tid);
        fetch(td, d_y + tok * HD, L, tid);
    };
    auto fetch_b = [&](int task, int tid) {
        const int chain = task / nc, ci = task % nc;
        const size_t end = ((size_t)chain * (nc + 1) + ci + 1) * kDD;
        fetch(tt, Tg + (size_t)task * kDD, 64, tid);
        fetch(tu, Ug + (size_t)task * kDD, 64, tid);
        fetch(tdm, em + end, 64, tid);
        if (has_s) fetch(tds, es_ + end, 64, tid);
        fetch(tm, m_ckpt + ((size_t)chain * nck + ci) * kDD, 64, tid);
        if (has_s) fetch(ts, s_ckpt + ((size_t)chain * nck + ci) * kDD, 64, tid);
    };
    const int per = (ntask + (int)gridDim.x - 1) / (int)gridDim.x, task_lo = blockIdx.x * per, task_hi = min(ntask, task_lo + per);
    if (task_lo < task_hi) fetch_a(task_lo, threadIdx.x);
    for (int itask = task_lo; itask < task_hi; itask++) {
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
    const int l = tid & 63;
    int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    asm volatile("" : "+s"(w));
    NLH_STRIP_ORIGIN_OF(w);
    auto MMA = [&](Strip &acc, auto fa, auto fb) { mma(acc, fa, fb, l); };
    auto MMAR = [&](Strip &acc, auto fa, auto fb, int p0, int p1) { mma_range(acc, fa, fb, p0, p1, l); };
    auto FORC = [&](Strip &acc, auto f) { for_c(acc, f, l); };
    const int chain = itask / nc, ci = itask % nc, t0 = ci * C, L = min(C, s - t0);
    const size_t tok = (size_t)chain * s + t0, task = (size_t)itask;
    fetch_b(itask, tid);
    load_gates(cf, gt);
    coefficients(cf, gt, L, Cc, nullptr, nullptr);
    commit(Ks, tk, tid);
    commit(Qs, tq, tid);
    commit(Ds, td, tid);
    __syncthreads();
    chunk_vectors(cv, cf, L);
    auto aK = [&](int m, int kk) { return Ks[(m0 + m) * LDM + kk]; };
    Strip p = zero_strip(), g = zero_strip();   // Q K^T and K K^T while the other tiles are in flight
    MMA(p, [&](int m, int kk) { return Qs[(m0 + m) * LDM + kk]; }, [&](int kk, int n) { return Ks[(n0 + n) * LDM + kk]; });
    MMA(g, aK, [&](int kk, int n) { return Ks[(n0 + n) * LDM + kk]; });
    {
        commit(Ts, tt, tid);
        commit(Us, tu, tid);
        commit(A1, tdm, tid);
        if (has_s) commit(A2, tds, tid);
        const float x0 = wave_allreduce(tile_dot(tm, tdm));
        const float x1 = has_s ? wave_allreduce(tile_dot(ts, tdm)) : 0.f;
        const float x2 = has_s ? wave_allreduce(tile_dot(ts, tds)) : 0.f;
        if (l == 0) { dots[0][w] = x0; dots[1][w] = x1; dots[2][w] = x2; }
    }
    __syncthreads();
    if (tid < 3) {
        const float *pp = dots[tid];
        scal[task * 4 + tid] = ((pp[0] + pp[1]) + (pp[2] + pp[3])) + ((pp[4] + pp[5]) + (pp[6] + pp[7]));
    }
    auto publish = [&](int which, Strip &x) {   // row sums of x -> part[which][column half][row]
        strip_row_sums(x);
        if (row_writer(l)) {
#pragma unroll
            for (int i = 0; i < 4; i++) part[which][nh][m0 + row_of(i, l)] = x.t[0][i];
        }
    };
    auto aU = [&](int m, int kk) { return Us[(m0 + m) * LDM + kk]; };
    Strip udm = zero_strip(), uds = zero_strip();
    {
        Strip kdm = zero_strip(), kds = zero_strip();
        MMA(kdm, aK, [&](int kk, int n) { return A1[(n0 + n) * LDM + kk]; });
        MMA(udm, aU, [&](int kk, int n) { return A1[kk * LDM + n0 + n]; });
        if (has_s) {
            MMA(kds, aK, [&](int kk, int n) { return A2[(n0 + n) * LDM + kk]; });
            MMA(uds, aU, [&](int kk, int n) { return A2[kk * LDM + n0 + n]; });
        }
        const float *gi = dUg + task * kDD;
#pragma unroll
        for (int tl = 0; tl < 2; tl++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int row = m0 + row_of(i, l), col = n0 + 16 * tl + (l & 15);
                B9[row * LDM + col] = gi[row * HD + col] + cv.wM[row] * kdm.t[tl][i] + cv.wS[row] * kds.t[tl][i];   // dU
            }
    }
    __syncthreads();   // dU complete; dMo, dSo no longer needed
    {
        Strip dr = zero_strip();
        // T^T is upper triangular: row block ib contracts over the blocks ib .. 3 of 16 (taken in pairs)
        MMAR(dr, [&](int m, int kk) { return Ts[kk * LDM + m0 + m]; }, [&](int kk, int n) { return B9[kk * LDM + n0 + n]; },
             ib >> 1, 2);
        FORC(dr, [&](int r, int c, float &x) {
            if (m0 + r < L) d_v[(tok + m0 + r) * HD + n0 + c] = -x;
        });
        __syncthreads();   // T no longer needed
        FORC(dr, [&](int r, int c, float &x) { Ts[(m0 + r) * LDM + n0 + c] = x; });   // dR
    }
    __syncthreads();
    const float *dRs = Ts;
    Strip dwa;
    {
        Strip dlam = zero_strip(), dyu = zero_strip();
        auto bU = [&](int kk, int n) { return Us[(n0 + n) * LDM + kk]; };
        MMA(dlam, [&](int m, int kk) { return dRs[(m0 + m) * LDM + kk]; }, bU);
        MMA(dyu, [&](int m, int kk) { return Ds[(m0 + m) * LDM + kk]; }, bU);
#pragma unroll
        for (int tl = 0; tl < 2; tl++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int row = m0 + row_of(i, l), col = n0 + 16 * tl + (l & 15);
                const float nth = -cf.th[col];
                const float c0 = Cc[row * LDM + col], c1 = row > 0 ? Cc[(row - 1) * LDM + col] : 0.f;
                const float lam = (col < row && row < L) ? dlam.t[tl][i] : 0.f;
                const float yu = (col <= row && row < L) ? dyu.t[tl][i] : 0.f;
                B9[row * LDM + col] = nth * c0 * yu;            // dP = W . tril(dY U^T)
                A2[row * LDM + col] = lam * g.t[tl][i];         // dLam . G, read one row down below
                const float dg = nth * c1 * lam;                // dG, stored symmetrised
                if (col < row) { A1[row * LDM + col] = dg; A1[col * LDM + row] = dg; }
                if (col == row) A1[row * LDM + col] = 0.f;
                dwa.t[tl][i] = yu * p.t[tl][i];
            }
    }
    __syncthreads();
    {
        float *xo = xs + task * CW * CW;
        float cs[2] = {0.f, 0.f};
#pragma unroll
        for (int tl = 0; tl < 2; tl++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int row = m0 + row_of(i, l), col = n0 + 16 * tl + (l & 15);
                const float dw = dwa.t[tl][i] + (row + 1 < CW ? A2[(row + 1) * LDM + col] : 0.f);
                xo[col * CW + row] = -cf.th[col] * dw;          // [s][t]
                cs[tl] = fmaf(dw, Cc[row * LDM + col], cs[tl]);
            }
#pragma unroll
        for (int tl = 0; tl < 2; tl++) {
            float x = xor_add<16>(cs[tl]);
            x = xor_add<32>(x);
            if (l < 16) part_th[ib][n0 + 16 * tl + l] = x;
        }
    }
    __syncthreads();   // c and U no longer needed
    commit(Us, tm, tid);
    if (has_s) commit(Cc, ts, tid);
    __syncthreads();
    if (itask + 1 < task_hi) fetch_a(itask + 1, tid);
    const float *M0s = Us, *S0s = Cc, *dPs = B9, *dGs = A1;
    {
        Strip dym = zero_strip(), dys = zero_strip(), dq = zero_strip(), r0 = zero_strip(), r1 = zero_strip();
        auto aD = [&](int m, int kk) { return Ds[(m0 + m) * LDM + kk]; };
        MMA(dym, aD, [&](int kk, int n) { return M0s[kk * LDM + n0 + n]; });
        if (has_s) MMA(dys, aD, [&](int kk, int n) { return S0s[kk * LDM + n0 + n]; });
        MMA(dq, [&](int m, int kk) { return dPs[(m0 + m) * LDM + kk]; }, [&](int kk, int n) { return Ks[kk * LDM + n0 + n]; });
#pragma unroll
        for (int tl = 0; tl < 2; tl++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int row = m0 + row_of(i, l), col = n0 + 16 * tl + (l & 15);
                const float qv = Qs[row * LDM + col];
                r0.t[tl][i] = dym.t[tl][i] * qv;
                r1.t[tl][i] = dys.t[tl][i] * qv;
                if (row < L)
                    d_q[(tok + row) * HD + col] = cf.a[row] * dym.t[tl][i] + cf.beta[row] * dys.t[tl][i] + dq.t[tl][i];
            }
        publish(0, r0);
        publish(1, r1);
    }
    {   // d_k in two halves: fewer accumulators alive at once
        Strip dk = zero_strip();
        {
            Strip r2 = zero_strip(), r3 = zero_strip();
            MMA(dk, [&](int m, int kk) { return dPs[kk * LDM + m0 + m]; }, [&](int kk, int n) { return Qs[kk * LDM + n0 + n]; });
            MMA(dk, [&](int m, int kk) { return dGs[(m0 + m) * LDM + kk]; }, [&](int kk, int n) { return Ks[kk * LDM + n0 + n]; });
#pragma unroll
            for (int tl = 0; tl < 2; tl++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int row = m0 + row_of(i, l), col = n0 + 16 * tl + (l & 15);
                    const float kv = Ks[row * LDM + col];
                    r2.t[tl][i] = udm.t[tl][i] * kv;
                    r3.t[tl][i] = uds.t[tl][i] * kv;
                    dk.t[tl][i] += cv.wM[row] * udm.t[tl][i] + cv.wS[row] * uds.t[tl][i];
                }
            publish(2, r2);
            publish(3, r3);
        }
        {
            Strip drm = zero_strip(), drs = zero_strip(), r4 = zero_strip(), r5 = zero_strip();
            auto aR = [&](int m, int kk) { return dRs[(m0 + m) * LDM + kk]; };
            MMA(drm, aR, [&](int kk, int n) { return M0s[kk * LDM + n0 + n]; });
            if (has_s) MMA(drs, aR, [&](int kk, int n) { return S0s[kk * LDM + n0 + n]; });
#pragma unroll
            for (int tl = 0; tl < 2; tl++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int row = m0 + row_of(i, l), col = n0 + 16 * tl + (l & 15);
                    const float kv = Ks[row * LDM + col];
                    r4.t[tl][i] = drm.t[tl][i] * kv;
                    r5.t[tl][i] = drs.t[tl][i] * kv;
                    if (row < L)
                        d_k[(tok + row) * HD + col] = dk.t[tl][i] + cv.am[row] * drm.t[tl][i] + cv.bm[row] * drs.t[tl][i];
                }
            publish(4, r4);
            publish(5, r5);
        }
    }
    __syncthreads();
    if (tid < L) {
        const int t = tid;
        auto sum = [&](int which, int row) { return part[which][0][row] + part[which][1][row]; };
        const float g1 = sum(2, t), g2 = sum(3, t);
        const float dam = t + 1 < CW ? sum(4, t + 1) : 0.f, dbm = t + 1 < CW ? sum(5, t + 1) : 0.f;
        d_theta[tok + t] = -(((part_th[0][t] + part_th[1][t]) + (part_th[2][t] + part_th[3][t])) + cf.cl[t] * g1 + cf.bl[t] * g2);
        float *pv = pvec + (tok + t) * 4;
        pv[0] = sum(0, t) + dam;
        pv[1] = sum(1, t) + dbm;
        pv[2] = -cf.th[t] * g1;
        pv[3] = -cf.th[t] * g2;
    }
    __syncthreads();   // LDS is rewritten by the next chunk
    }
}
constexpr size_t kExGradsLds = 9 * MAT * sizeof(float);

template <class K>
void set_lds(K kernel, size_t bytes) {
    check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  (int)bytes), "dynamic LDS size");
}

}  // namespace

bool exact_backward_mm_applies(int d, int C) { return d == HD && C >= 1 && C <= CW; }

// Cost model from measurements on one MI355X: a chunk costs the two chunk-parallel kernels about 65 us of a compute
// unit whatever its length, a scan step 2.7 us; the fused sequential kernel walks a chain's tokens at 0.6 us each on a
// quarter of a compute unit's worth of workgroups (four per chain).
bool exact_backward_mm_pays(int seq_len, int batch, int C) {
    const int nc = ceil_div(seq_len, C), cus = compute_units();
    const double t_mm = (double)ceil_div(batch * nc, cus) * 65.0 + nc * 2.7;
    const double t_seq = (double)seq_len * 0.6 * ceil_div(batch * 4, cus);
    return t_mm < t_seq;
}

bool exact_backward_mm(const char *fn, bool has_s, const float *k, const float *v, const float *q, const float *alpha,
                       const float *theta, const float *eta, const float *m_ckpt, const float *s_ckpt, const float *d_y,
                       float *d_k, float *d_v, float *d_q, float *d_alpha, float *d_theta, float *d_eta, float *d_m_initial,
                       float *d_s_initial, int seq_len, int batch, int C, float error_clip, float m_norm_guard) {
    const ErrorScope es;
    if (seq_len <= 0 || batch <= 0 || !exact_backward_mm_applies(HD, C)) {
        fail("%s: the matrix form needs seq_len=%d and batch=%d positive and a checkpoint interval %d in [1, %d].", fn, seq_len, batch,
             C, CW);
        return true;
    }
    const int nc = ceil_div(seq_len, C), nck = n_ckpt_count(seq_len, C);
    const size_t nchunks = (size_t)batch * nc;
    const bool guard = error_clip > 0.f || m_norm_guard > 0.f;
    ChainTracks tracks{nullptr, nullptr};
    if (guard) tracks = chain_tracks(seq_len, batch, C);
    float *loc = scratch(32, nchunks * kExLocMats * kDD * sizeof(float));
    float *Tg = scratch(33, nchunks * kDD * sizeof(float));
    float *Ug = scratch(34, nchunks * kDD * sizeof(float));
    float *dUg = scratch(35, nchunks * kDD * sizeof(float));
    float *locs = scratch(4, nchunks * 4 * sizeof(float));
    float *em = scratch(5, (size_t)batch * (nc + 1) * kDD * sizeof(float));
    float *esn = has_s ? scratch(6, (size_t)batch * (nc + 1) * kDD * sizeof(float)) : nullptr;
    float *xs = scratch(7, nchunks * CW * CW * sizeof(float));
    float *pvec = scratch(8, (size_t)batch * seq_len * 4 * sizeof(float));
    float *scal = scratch(9, nchunks * 4 * sizeof(float));
    const int per = 8, rows = ceil_div(batch, per), nsum = has_s ? 2 : 1;
    float *tmp = scratch(10, (size_t)nsum * rows * kDD * sizeof(float));
    float *first = scratch(36, (size_t)2 * batch * kDD * sizeof(float));
    if (es.failed()) return true;
    float *first_m = first, *first_s = first + (size_t)batch * kDD;
    static bool attr_set = false;
    if (!attr_set) {
        set_lds(ex_local_kernel<false>, kExLocalLds);
        set_lds(ex_local_kernel<true>, kExLocalLds);
        set_lds(ex_grads_kernel, kExGradsLds);
        attr_set = true;
    }
    if (es.failed()) return true;
    const int cus = compute_units(), pgrid = nchunks < (size_t)cus ? (int)nchunks : cus;   // one workgroup per compute unit (LDS)
    {
        KernelTimer kt("ex_local_kernel");
        if (guard)
            hipLaunchKernelGGL(ex_local_kernel<true>, dim3((unsigned)pgrid), dim3(kThr), kExLocalLds, stream(), k, v, q, d_y,
                               alpha, theta, eta, m_ckpt, s_ckpt, loc, locs, Tg, Ug, dUg, seq_len, C, nc, nck, (int)has_s, (int)nchunks, tracks);
        else
            hipLaunchKernelGGL(ex_local_kernel<false>, dim3((unsigned)pgrid), dim3(kThr), kExLocalLds, stream(), k, v, q, d_y,
                               alpha, theta, eta, m_ckpt, s_ckpt, loc, locs, Tg, Ug, dUg, seq_len, C, nc, nck, (int)has_s, (int)nchunks, tracks);
        check_launch("ex_local_kernel");
    }
    {
        KernelTimer kt("ex_scan_kernel");
        if (has_s)
            hipLaunchKernelGGL(ex_scan_kernel<true>, dim3((unsigned)batch * 4), dim3(kThr), 0, stream(), loc, locs, em, esn,
                               first_m, first_s, nc);
        else
            hipLaunchKernelGGL(ex_scan_kernel<false>, dim3((unsigned)batch * 4), dim3(kThr), 0, stream(), loc, locs, em, esn,
                               first_m, first_s, nc);
        check_launch("ex_scan_kernel");
    }
    {
        KernelTimer kt("ex_grads_kernel");
        hipLaunchKernelGGL(ex_grads_kernel, dim3((unsigned)pgrid), dim3(kThr), kExGradsLds, stream(), k, q, d_y, alpha, theta,
                           eta, m_ckpt, s_ckpt, Tg, Ug, dUg, em, esn, d_k, d_v, d_q, d_theta, pvec, xs, scal, seq_len, C, nc, nck,
                           (int)has_s, (int)nchunks);
        check_launch("ex_grads_kernel");
    }
    chunkwise_gate_gradients(alpha, eta, pvec, xs, scal, d_alpha, d_eta, seq_len, batch, C, has_s, first_m, first_s, kDD, per,
                             nsum, tmp);
    if (es.failed()) return true;
    if (guard && couplings_may_fire_tracked(k, alpha, theta, eta, tracks, has_s, seq_len, batch, C, error_clip, m_norm_guard))
        return false;
    accumulate_over_batch2(tmp, d_m_initial, has_s ? tmp + (size_t)rows * kDD : nullptr, d_s_initial, rows, (int)kDD);
    return true;
}

}  // namespace nlh
