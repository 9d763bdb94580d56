// Backward of the frozen-M0 chunkwise Titans / Delta rule on bf16 tokens: the per-chunk
// gradients d_q, d_k, d_v, d_theta and what the gate pass needs, on the bf16 matrix cores.
//
// Same mathematics as cw_grads_bwd_kernel of chunkwise_mm.hip (which documents the
// formulas); inputs are the chunk-start states M0, S0 and the adjoints dMo, dSo of the
// chunk-end states from the adjoint scan.  With E = K M0^T - V, P = Q K^T, R = dY E^T,
// c = coefficient table, cl_j = c[L-1][j], bl_j = bb[j][L-1]:
//   X   = R.P                                   (to the gate pass)
//   dQ  = a.(dY M0) + beta.(dY S0) + (-theta_j c.R) K
//   Dk  = (c.P)^T dY + cl.(K dMo^T) + bl.(K dSo^T)        [token j][row i]
//   dE  = -theta_j Dk,  dV = -dE,  d_theta_j = -sum_i E Dk
//   DTe = (c.R)^T Q + cl.(E dMo) + bl.(E dSo)             [token j][column c]
//   dK  = -theta_j DTe + dE M0
// plus the row sums p0, ps, g1, g2 and the three state dots of the gate pass.
//
// Precision: k, v, q are exact in bf16.  E is formed against a hi + lo bf16 pair of M0
// (its two terms nearly cancel once the memory has learned); every other fp32 operand (dY,
// states, adjoints, E, c.P, c.R, dE) enters the matrix cores rounded to one bf16, products
// accumulate in fp32.  That is the bf16-input / fp32-accumulate contract: results agree with
// an fp32 evaluation of the same rule to a few 1e-3, inside the 2e-2 stated for this path.
//
// One workgroup per compute unit walks over chunks.  The inputs of the next chunk are requested right
// after this chunk's have been staged and stay in registers for the rest of the step (the staged copies
// need 11 LDS matrices and no transposed ones, which leaves the registers for that).  The pass moves
// 1.35 GB per launch at 128 chains x 4096 tokens (5 TB/s) and is bound by that traffic; the adjoint snapshots
// arrive as bf16, as the scan's own hi operand.  Every output tile is computed transposed
// (rows = feature, columns = token) so that a lane ends up with four consecutive features of
// one token: 16-byte stores.  Waves 0..3 (group A) hold P and produce X, c.P, c.R, Dk; waves
// 4..7 (group B) hold dQ and produce -theta c.R, dQ, DTe, dK.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "bf16_tiles.h"
#include "chunk_coef.h"
#include "chunkwise_chain.h"
#include "chunkwise_grads.h"
#include "runtime.h"

namespace nlh {
namespace {

// Per-chunk coefficients in HBM, written by cw_coef_bwd_kernel:
//   tab_b [chunk][block bi][rt][ct][lane l][r]: c[t][j] (zero outside j <= t < L) at
//         t = 32 (bi/2) + 16 rt + 4 (l/16) + r, j = 32 (bi%2) + 16 ct + l%16  (the order in which group A holds P, R)
//   vecs  [chunk][kVecB]: a_t, beta_t, cl_j, bl_j, theta_j, then four zeros and h_L
// Tiles entirely above the diagonal are neither written nor read.
constexpr int kTab = CW * CW;
constexpr int kVecB = 5 * CW + 16;
constexpr int kCtLd = CW + 4;   // row stride (floats) of the coefficient copy in LDS
constexpr int kCoefChunksPerWave = 4;
__device__ __forceinline__ bool live_b(int bi, int rt, int ct) { return 2 * (bi >> 1) + rt >= 2 * (bi & 1) + ct; }

// One wave per chunk, lane = token: the vectors from two scans of composed maps, the table from
// coef_table_columns, assembled in LDS as c[t][j] and gathered in the consumers' order on the way out, as
// 16-byte stores of consecutive lanes.
template <bool HAS_S>
__global__ __launch_bounds__(64) void cw_coef_bwd_kernel(const float *__restrict__ alpha,
                                                         const float *__restrict__ theta,
                                                         const float *__restrict__ eta,
                                                         float *__restrict__ tab_b, float *__restrict__ vecs,
                                                         int s, int C, int nc, int nchunks) {
    __shared__ __align__(16) float stage[(CW + 1) * kCtLd];
    __shared__ float gk[2 * CW], ge[2 * CW];
    const int j = threadIdx.x, first = blockIdx.x * kCoefChunksPerWave, last = min(nchunks, first + kCoefChunksPerWave);
    auto gates_of = [&](int chunk) {
        const int chain = chunk / nc, t0 = (chunk % nc) * C;
        return fetch_gates<HAS_S>(alpha, theta, eta, (size_t)chain * s + t0, min(C, s - t0));
    };
    // a wave walks over a few chunks with the next chunk's gates in flight (a wave per chunk would spend most of
    // its life waiting for its three loads, and LDS allows only eight waves per compute unit)
    Gates gn = gates_of(first);
    for (int chunk = first; chunk < last; chunk++) {
        const int L = min(C, s - (chunk % nc) * C);
        const Gates g = gn;
        gn = gates_of(min(chunk + 1, last - 1));
        const bool jv = j < L;
        const float keep = 1.f - g.al, et = g.et;   // 1, 0 beyond L
        const ChunkVectors cv = coef_vectors(keep, et, jv);
        float *vo = vecs + (size_t)chunk * kVecB;
        vo[j] = jv ? cv.a : 0.f;
        vo[CW + j] = jv ? cv.beta : 0.f;
        vo[2 * CW + j] = jv ? cv.cl : 0.f;
        vo[3 * CW + j] = jv ? cv.bl : 0.f;
        vo[4 * CW + j] = g.th;
        if (j < 4) vo[5 * CW + j] = 0.f;   // what tiles above the diagonal read
        if (j == 63) vo[5 * CW + 4] = cv.h;   // h at token L - 1
        coef_table_columns<kCtLd, false>(stage, gk, ge, keep, et, 1.f, L);
        float *ob = tab_b + (size_t)chunk * kTab;
        // the ten 16 x 16 tiles on or below the diagonal (token tile T >= column tile J), one 16-byte piece per lane each
#pragma unroll
        for (int T = 0; T < 4; T++)
#pragma unroll
            for (int J = 0; J <= T; J++) {
                const int tile = ((T >> 1) * 2 + (J >> 1)) * 4 + (T & 1) * 2 + (J & 1);   // (bi, rt, ct) of the layout above
                const float *p = stage + (16 * T + 4 * (j >> 4)) * kCtLd + 16 * J + (j & 15);
                *reinterpret_cast<f32x4 *>(ob + (tile * 64 + j) * 4) = f32x4{p[0], p[kCtLd], p[2 * kCtLd], p[3 * kCtLd]};
            }
    }
}

// Sum over the four 16-lane groups of a wave (lanes with equal l%16).
__device__ __forceinline__ float sum_groups(float x) {
    x += __shfl_xor(x, 16);
    x += __shfl_xor(x, 32);
    return x;
}
__device__ __forceinline__ float sum_wave(float x) {
#pragma unroll
    for (int m = 1; m < 64; m <<= 1) x += __shfl_xor(x, m);
    return x;
}
__device__ __forceinline__ f32x4 bf4_to_f32(const uint2 b) {
    return f32x4{__uint_as_float(b.x << 16), __uint_as_float(b.x & 0xffff0000u), __uint_as_float(b.y << 16),
                 __uint_as_float(b.y & 0xffff0000u)};
}
__device__ __forceinline__ f32x4 bf4_to_f32(const u16 *p) { return bf4_to_f32(*reinterpret_cast<const uint2 *>(p)); }

// TRACK: also leaves the ChainTracks of chunkwise_chain.h behind (what a test of the reference's couplings needs).
template <bool HAS_S, bool G16, bool TRACK>
__global__ __launch_bounds__(kTileThr) void cw_grads_bf16_kernel(
    const u16 *__restrict__ k, const u16 *__restrict__ v, const u16 *__restrict__ q, const float *__restrict__ d_y,
    const float *__restrict__ tab_b, const float *__restrict__ vecs,
    const float *__restrict__ m_states, const float *__restrict__ s_states, const u16 *__restrict__ dm_snap,
    const u16 *__restrict__ ds_snap, float *__restrict__ d_k, float *__restrict__ d_v, float *__restrict__ d_q,
    float *__restrict__ d_theta, float *__restrict__ pvec, float *__restrict__ xs, float *__restrict__ scal, int s,
    int C, int nc, int ntask, HeadRows dyr, GradOut16 go, ChainTracks tr) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    // Every input is staged once, in the order it arrives (rows = tokens or state rows); a product that contracts
    // over the row index reads its operand through ld_op_tr.
    u16 *Kr = reinterpret_cast<u16 *>(smem_raw), *Qr = Kr + BMAT;   // K [t][c], Q [t][c]
    u16 *Vr = Qr + BMAT, *dYr = Vr + BMAT;                           // V [t][i], dY [t][i]
    u16 *M0h = dYr + BMAT, *M0l = M0h + BMAT;                        // M0 [i][c] hi / lo
    u16 *S0r = M0l + BMAT;                                           // S0 [i][c]
    u16 *dMr = S0r + BMAT, *dSr = dMr + BMAT;                        // dMo [i][c], dSo [i][c]
    u16 *Er = dSr + BMAT, *CRt = Er + BMAT;                          // E [t][i]; (c.R)^T [j][t]
    u16 *CPt = Vr, *ThCR = M0l, *dEr = S0r;                          // reuse once their first tenants are dead
    float *cvec = reinterpret_cast<float *>(CRt + BMAT);             // a, beta, cl, bl, theta [64] each
    float *part = cvec + 5 * CW;                                     // [5][2][64]: p0, ps, rt, g1, g2 per half
    float *dots = part + 5 * 2 * CW;                                 // [3][8]
    float *Ctj = dots + 24;                                          // c [t][j], row stride kCtLd: group A -> group B

    const int tid = threadIdx.x, w = tid >> 6, l = tid & 63, g = l >> 4, r16 = l & 15;
    const bool grpA = w < 4;
    const int bi = w & 3, bm = 32 * (bi >> 1), bn = 32 * (bi & 1);
    // Staging maps.  A wave instruction reads whole or half 128-byte lines (the rate of line
    // requests, not bytes, bounds a compute unit).
    //   bf16 tile: row st_t, 8-element block st_cb (16 rows x 64 bytes per wave)
    //   fp32 tile: row ft, 4-element blocks fg0 and fg0 + 8 (8 rows x 128 bytes per wave and pass)
    const int st_t = 16 * (w & 3) + (l & 15), st_cb = 4 * (w >> 2) + (l >> 4);
    const int ft = 8 * w + (l >> 3), fg0 = l & 7;

    // inputs of the current task in registers (only while they are staged)
    uint4 nK, nQ, nV;
    f32x4 ndY[2], nM0[2], nS0[2], ntab[2][2];
    uint2 ndM[2], ndS[2];   // four bf16 each
    float nvec = 0.f;
    auto fetch = [&](int task) {
        const int chain = task / nc, ci = task % nc, t0 = ci * C, L = min(C, s - t0);
        const size_t tok = (size_t)chain * s + t0, row = tok + min(st_t, L - 1);
        nK = *reinterpret_cast<const uint4 *>(k + row * HD + st_cb * 8);
        nQ = *reinterpret_cast<const uint4 *>(q + row * HD + st_cb * 8);
        nV = *reinterpret_cast<const uint4 *>(v + row * HD + st_cb * 8);
        const size_t st0 = ((size_t)chain * (nc + 1) + ci) * HD * HD + ft * HD, st1 = st0 + HD * HD;
        const float *dy_row = d_y + dyr.offset(chain) + (size_t)(t0 + min(ft, L - 1)) * dyr.row_stride;
#pragma unroll
        for (int it = 0; it < 2; it++) {
            const int c4 = (fg0 + 8 * it) * 4;
            ndY[it] = *reinterpret_cast<const f32x4 *>(dy_row + c4);
            nM0[it] = *reinterpret_cast<const f32x4 *>(m_states + st0 + c4);
            ndM[it] = *reinterpret_cast<const uint2 *>(dm_snap + st1 + c4);
            if (HAS_S) {
                nS0[it] = *reinterpret_cast<const f32x4 *>(s_states + st0 + c4);
                ndS[it] = *reinterpret_cast<const uint2 *>(ds_snap + st1 + c4);
            }
        }
        nvec = vecs[(size_t)task * kVecB + min(tid, 5 * CW - 1)];
    };
    // The coefficient table of a task is requested separately, once the previous one has been used, by group A
    // only: group B wants the same numbers with the roles of t and j exchanged and takes them from the copy that
    // group A leaves in LDS.
    auto fetch_tab = [&](int task) {
        if (!grpA) return;
        const float *zero = vecs + (size_t)task * kVecB + 5 * CW;
        const float *tb = tab_b + (size_t)task * kTab;
#pragma unroll
        for (int rt = 0; rt < 2; rt++)
#pragma unroll
            for (int ct = 0; ct < 2; ct++)
                ntab[rt][ct] = *reinterpret_cast<const f32x4 *>(
                    live_b(bi, rt, ct) ? tb + (((bi * 2 + rt) * 2 + ct) * 64 + l) * 4 : zero);
    };

    // contiguous task range per workgroup: consecutive chunks of a chain share pages and cache lines
    const int per = (ntask + (int)gridDim.x - 1) / (int)gridDim.x, task_lo = blockIdx.x * per,
              task_hi = min(ntask, task_lo + per);
    if (task_lo >= task_hi) return;
    fetch_tab(task_lo);
    fetch(task_lo);

    for (int task = task_lo; task < task_hi; task++) {
        const int chain = task / nc, ci = task % nc, t0 = ci * C, L = min(C, s - t0);
        const size_t tok = (size_t)chain * s + t0;
        // where four consecutive columns `col` of token t0 + tl of a gradient go: the fp32 head-major tensor, or (G16) a
        // bf16 token-major slab in which chain = (level, batch element, head) addresses its own columns
        const size_t g_off = G16 ? go.rows.offset(chain) + (size_t)t0 * go.rows.row_stride : 0;
        auto put = [&](float *f32base, u16 *g16base, int tl, int col, f32x4 val) {
            if constexpr (G16) bf16_store(g16base + g_off + (size_t)tl * go.rows.row_stride + col, 0, val);
            else *reinterpret_cast<f32x4 *>(f32base + (tok + tl) * HD + col) = val;
        };
        // ── load and stage everything ──
        {
            if (st_t >= L) { nK = make_uint4(0, 0, 0, 0); nQ = nK; nV = nK; }
            if (ft >= L) { ndY[0] = zero4(); ndY[1] = zero4(); }
            *reinterpret_cast<uint4 *>(Kr + st_t * LDB + st_cb * 8) = nK;
            *reinterpret_cast<uint4 *>(Qr + st_t * LDB + st_cb * 8) = nQ;
            *reinterpret_cast<uint4 *>(Vr + st_t * LDB + st_cb * 8) = nV;
            float d0 = 0.f, d1 = 0.f, d2 = 0.f, msq = 0.f, ssq = 0.f;
#pragma unroll
            for (int it = 0; it < 2; it++) {
                const int c4 = (fg0 + 8 * it) * 4, off = ft * LDB + c4;
                bf16_store(dYr, off, ndY[it]);
                split_store(M0h, M0l, off, nM0[it]);
                *reinterpret_cast<uint2 *>(dMr + off) = ndM[it];
                const f32x4 fdM = bf4_to_f32(ndM[it]);
                f32x4 fdS = zero4();
                if (HAS_S) {
                    *reinterpret_cast<uint2 *>(dSr + off) = ndS[it];
                    bf16_store(S0r, off, nS0[it]);
                    fdS = bf4_to_f32(ndS[it]);
                }
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    d0 = fmaf(nM0[it][i], fdM[i], d0);
                    if (HAS_S) { d1 = fmaf(nS0[it][i], fdM[i], d1); d2 = fmaf(nS0[it][i], fdS[i], d2); }
                    if (TRACK) {
                        msq = fmaf(nM0[it][i], nM0[it][i], msq);
                        if (HAS_S) ssq = fmaf(nS0[it][i], nS0[it][i], ssq);
                    }
                }
            }
            d0 = sum_wave(d0); d1 = sum_wave(d1); d2 = sum_wave(d2);
            if (l == 0) { dots[w] = d0; dots[8 + w] = d1; dots[16 + w] = d2; }
            if (TRACK) {
                msq = sum_wave(msq);
                ssq = sum_wave(ssq);
                if (l == 0) *reinterpret_cast<float2 *>(tr.nrm + (((size_t)chain * nc + ci) * 8 + w) * 2) = make_float2(msq, ssq);
            }
            if (tid < 5 * CW) cvec[tid] = nvec;
            if (grpA) {   // c[t .. t+3][j] of this wave's block
#pragma unroll
                for (int rt = 0; rt < 2; rt++)
#pragma unroll
                    for (int ct = 0; ct < 2; ct++)
#pragma unroll
                        for (int r = 0; r < 4; r++)
                            Ctj[(bm + 16 * rt + 4 * g + r) * kCtLd + bn + 16 * ct + r16] = ntab[rt][ct][r];
            }
        }
        __syncthreads();
        fetch(min(task + 1, task_hi - 1));

        // ── P, E^T (group A); dQ^T = a.(M0^T dY^T) + beta.(S0^T dY^T), p0, ps (group B) ──
        f32x4 keep[2][2] = {{zero4(), zero4()}, {zero4(), zero4()}};   // group A: P [t][j]; group B: dQ^T [c][t]
        if (grpA) {
            f32x4 e[2][2] = {{zero4(), zero4()}, {zero4(), zero4()}};
#pragma unroll
            for (int ks = 0; ks < 2; ks++) {
                bf16x8 bK[2];
#pragma unroll
                for (int ct = 0; ct < 2; ct++) bK[ct] = ld_op(Kr, bn + 16 * ct, ks);
#pragma unroll
                for (int rt = 0; rt < 2; rt++) {
                    const bf16x8 aq = ld_op(Qr, bm + 16 * rt, ks);
                    const bf16x8 mh = ld_op(M0h, bm + 16 * rt, ks), ml = ld_op(M0l, bm + 16 * rt, ks);
#pragma unroll
                    for (int ct = 0; ct < 2; ct++) {
                        keep[rt][ct] = mfma32(aq, bK[ct], keep[rt][ct]);   // P[t][j]
                        e[rt][ct] = mfma32(mh, bK[ct], e[rt][ct]);         // E^T[i][t]
                        e[rt][ct] = mfma32(ml, bK[ct], e[rt][ct]);
                    }
                }
            }
            // -identity operand of E^T = M0 K^T - V^T: rows i = bm + 16 rt + l%16 meet contraction
            // indices 32 (bm/32) + 8 (l/16) + e
            bf16x8 negI[2];
#pragma unroll
            for (int rt = 0; rt < 2; rt++) {
                const int hit = 16 * rt + r16 - 8 * g;
                uint4 bits;
                bits.x = (hit == 0 ? 0xBF80u : 0u) | (hit == 1 ? 0xBF800000u : 0u);
                bits.y = (hit == 2 ? 0xBF80u : 0u) | (hit == 3 ? 0xBF800000u : 0u);
                bits.z = (hit == 4 ? 0xBF80u : 0u) | (hit == 5 ? 0xBF800000u : 0u);
                bits.w = (hit == 6 ? 0xBF80u : 0u) | (hit == 7 ? 0xBF800000u : 0u);
                negI[rt] = __builtin_bit_cast(bf16x8, bits);
            }
#pragma unroll
            for (int ct = 0; ct < 2; ct++) {
                const bf16x8 bv = ld_op(Vr, bn + 16 * ct, bm >> 5);
                float esq = 0.f;
#pragma unroll
                for (int rt = 0; rt < 2; rt++) {
                    e[rt][ct] = mfma32(negI[rt], bv, e[rt][ct]);
                    bf16_store(Er, (bn + 16 * ct + r16) * LDB + bm + 16 * rt + 4 * g, e[rt][ct]);   // E[t][i .. i+3]
                    if (TRACK) {
#pragma unroll
                        for (int r = 0; r < 4; r++) esq = fmaf(e[rt][ct][r], e[rt][ct][r], esq);
                    }
                }
                if (TRACK) {   // token bn + 16 ct + l % 16, this wave's 32 memory rows (half bm / 32)
                    esq = sum_groups(esq);
                    if (g == 0) tr.e2[(((size_t)chain * 2 + (bm >> 5)) * nc + ci) * CW + bn + 16 * ct + r16] = esq;
                }
            }
        } else {
            // one product at a time: its row sums and its share of dQ^T, then the accumulators are free
            auto half = [&](const u16 *Sr, int which, int voff) {   // Sr [i][c]: read as S^T
                f32x4 ym[2][2] = {{zero4(), zero4()}, {zero4(), zero4()}};
#pragma unroll
                for (int ks = 0; ks < 2; ks++) {
                    bf16x8 bD[2];
#pragma unroll
                    for (int ct = 0; ct < 2; ct++) bD[ct] = ld_op(dYr, bn + 16 * ct, ks);
#pragma unroll
                    for (int rt = 0; rt < 2; rt++) {
                        const bf16x8 am = ld_op_tr<LDB>(Sr, bm + 16 * rt, ks);
#pragma unroll
                        for (int ct = 0; ct < 2; ct++) ym[rt][ct] = mfma32(am, bD[ct], ym[rt][ct]);   // [c][t]
                    }
                }
#pragma unroll
                for (int ct = 0; ct < 2; ct++) {
                    const int t = bn + 16 * ct + r16;
                    const float at = cvec[voff + t];
                    float p0 = 0.f;
#pragma unroll
                    for (int rt = 0; rt < 2; rt++) {
                        const f32x4 qv = bf4_to_f32(Qr + t * LDB + bm + 16 * rt + 4 * g);
#pragma unroll
                        for (int r = 0; r < 4; r++) p0 = fmaf(ym[rt][ct][r], qv[r], p0);
                        keep[rt][ct] += at * ym[rt][ct];
                    }
                    p0 = sum_groups(p0);
                    if (g == 0) part[(which * 2 + (bi >> 1)) * CW + t] = p0;
                }
            };
            half(M0h, 0, 0);
            if (HAS_S) {
                half(S0r, 1, CW);
            } else {
#pragma unroll
                for (int ct = 0; ct < 2; ct++)
                    if (g == 0) part[(1 * 2 + (bi >> 1)) * CW + bn + 16 * ct + r16] = 0.f;
            }
        }
        __syncthreads();

        // ── R = dY E^T: X, (c.P)^T, (c.R)^T (group A); R^T: -theta c.R (group B) ──
        {
            f32x4 rr[2][2] = {{zero4(), zero4()}, {zero4(), zero4()}};
            const u16 *Am = grpA ? dYr : Er, *Bm = grpA ? Er : dYr;
#pragma unroll
            for (int ks = 0; ks < 2; ks++) {
                bf16x8 bb[2];
#pragma unroll
                for (int ct = 0; ct < 2; ct++) bb[ct] = ld_op(Bm, bn + 16 * ct, ks);
#pragma unroll
                for (int rt = 0; rt < 2; rt++) {
                    const bf16x8 aa = ld_op(Am, bm + 16 * rt, ks);
#pragma unroll
                    for (int ct = 0; ct < 2; ct++) rr[rt][ct] = mfma32(aa, bb[ct], rr[rt][ct]);
                }
            }
            if (grpA) {   // rr = R[t][j] at the positions of P
                float *xo = xs + (size_t)task * kTab;
#pragma unroll
                for (int rt = 0; rt < 2; rt++)
#pragma unroll
                    for (int ct = 0; ct < 2; ct++) {
                        const int off = (bn + 16 * ct + r16) * LDB + bm + 16 * rt + 4 * g;   // [j][t .. t+3]
                        if (live_b(bi, rt, ct))   // tiles with every t < j are never read
                            *reinterpret_cast<f32x4 *>(xo + (bn + 16 * ct + r16) * CW + bm + 16 * rt + 4 * g) =
                                -cvec[4 * CW + bn + 16 * ct + r16] * (rr[rt][ct] * keep[rt][ct]);
                        bf16_store(CPt, off, ntab[rt][ct] * keep[rt][ct]);
                        bf16_store(CRt, off, ntab[rt][ct] * rr[rt][ct]);
                    }
            } else {      // rr = R^T[j][t]
#pragma unroll
                for (int rt = 0; rt < 2; rt++) {
                    const f32x4 th = *reinterpret_cast<const f32x4 *>(cvec + 4 * CW + bm + 16 * rt + 4 * g);
#pragma unroll
                    for (int ct = 0; ct < 2; ct++) {   // [t][j .. j+3]
                        const f32x4 c4 = *reinterpret_cast<const f32x4 *>(Ctj + (bn + 16 * ct + r16) * kCtLd + bm +
                                                                          16 * rt + 4 * g);
                        bf16_store(ThCR, (bn + 16 * ct + r16) * LDB + bm + 16 * rt + 4 * g, -(th * c4 * rr[rt][ct]));
                    }
                }
            }
        }
        __syncthreads();

        f32x4 dte[2][2] = {{zero4(), zero4()}, {zero4(), zero4()}};   // group B: DTe^T [c][j] (theta applied later)
        if (grpA) {
            // ── Dk^T [i][j] = dY^T (c.P) + cl.(dMo K^T) + bl.(dSo K^T); dE, dV, d_theta ──
            f32x4 dk[2][2] = {{zero4(), zero4()}, {zero4(), zero4()}};
            auto state_term = [&](const u16 *Ar, int voff) {   // dk += cvec[voff + j] . (Ar K^T)
                f32x4 t1[2][2] = {{zero4(), zero4()}, {zero4(), zero4()}};
#pragma unroll
                for (int ks = 0; ks < 2; ks++) {
                    bf16x8 bK[2];
#pragma unroll
                    for (int ct = 0; ct < 2; ct++) bK[ct] = ld_op(Kr, bn + 16 * ct, ks);
#pragma unroll
                    for (int rt = 0; rt < 2; rt++) {
                        const bf16x8 am = ld_op(Ar, bm + 16 * rt, ks);
#pragma unroll
                        for (int ct = 0; ct < 2; ct++) t1[rt][ct] = mfma32(am, bK[ct], t1[rt][ct]);
                    }
                }
#pragma unroll
                for (int ct = 0; ct < 2; ct++) {
                    const float cj = cvec[voff + bn + 16 * ct + r16];
#pragma unroll
                    for (int rt = 0; rt < 2; rt++) dk[rt][ct] += cj * t1[rt][ct];
                }
            };
            state_term(dMr, 2 * CW);
            if (HAS_S) state_term(dSr, 3 * CW);
#pragma unroll
            for (int ks = 0; ks < 2; ks++) {
                bf16x8 bP[2];
#pragma unroll
                for (int ct = 0; ct < 2; ct++) bP[ct] = ld_op(CPt, bn + 16 * ct, ks);
#pragma unroll
                for (int rt = 0; rt < 2; rt++) {
                    const bf16x8 ay = ld_op_tr<LDB>(dYr, bm + 16 * rt, ks);   // dY^T
#pragma unroll
                    for (int ct = 0; ct < 2; ct++) dk[rt][ct] = mfma32(ay, bP[ct], dk[rt][ct]);
                }
            }
#pragma unroll
            for (int ct = 0; ct < 2; ct++) {
                const int j = bn + 16 * ct + r16;
                const float thj = cvec[4 * CW + j];
                float rs = 0.f;
#pragma unroll
                for (int rt = 0; rt < 2; rt++) {
                    const f32x4 x = dk[rt][ct];                                              // Dk[j][i .. i+3]
                    const f32x4 ev = bf4_to_f32(Er + j * LDB + bm + 16 * rt + 4 * g);
#pragma unroll
                    for (int r = 0; r < 4; r++) rs = fmaf(ev[r], x[r], rs);
                    dk[rt][ct] = thj * x;                                                    // dV = theta_j Dk = -dE
                }
                rs = sum_groups(rs);
                if (g == 0) part[(2 * 2 + (bi >> 1)) * CW + j] = rs;
            }
            // S0 was last read two barriers ago: dE may take its place now
#pragma unroll
            for (int ct = 0; ct < 2; ct++) {
                const int j = bn + 16 * ct + r16;
#pragma unroll
                for (int rt = 0; rt < 2; rt++) {
                    bf16_store(dEr, j * LDB + bm + 16 * rt + 4 * g, -dk[rt][ct]);
                    if (j < L) put(d_v, go.gv, j, bm + 16 * rt + 4 * g, dk[rt][ct]);
                }
            }
        } else {
            // ── dQ^T += K^T (-theta c.R)^T; DTe^T [c][j] = Q^T (c.R) + cl.(dMo^T E^T) + bl.(dSo^T E^T); g1, g2 ──
#pragma unroll
            for (int ks = 0; ks < 2; ks++) {
                bf16x8 bT[2];
#pragma unroll
                for (int ct = 0; ct < 2; ct++) bT[ct] = ld_op(ThCR, bn + 16 * ct, ks);
#pragma unroll
                for (int rt = 0; rt < 2; rt++) {
                    const bf16x8 ak = ld_op_tr<LDB>(Kr, bm + 16 * rt, ks);   // K^T
#pragma unroll
                    for (int ct = 0; ct < 2; ct++) keep[rt][ct] = mfma32(ak, bT[ct], keep[rt][ct]);
                }
            }
#pragma unroll
            for (int ct = 0; ct < 2; ct++) {
                const int t = bn + 16 * ct + r16;
                if (t < L) {
#pragma unroll
                    for (int rt = 0; rt < 2; rt++)
                        put(d_q, go.gq, t, bm + 16 * rt + 4 * g, keep[rt][ct]);
                }
            }
            auto state_term = [&](const u16 *Ar, int which, int voff) {   // dte += cvec[voff + j] . (Ar^T E^T); g sums
                f32x4 t3[2][2] = {{zero4(), zero4()}, {zero4(), zero4()}};
#pragma unroll
                for (int ks = 0; ks < 2; ks++) {
                    bf16x8 bE[2];
#pragma unroll
                    for (int ct = 0; ct < 2; ct++) bE[ct] = ld_op(Er, bn + 16 * ct, ks);
#pragma unroll
                    for (int rt = 0; rt < 2; rt++) {
                        const bf16x8 am = ld_op_tr<LDB>(Ar, bm + 16 * rt, ks);
#pragma unroll
                        for (int ct = 0; ct < 2; ct++) t3[rt][ct] = mfma32(am, bE[ct], t3[rt][ct]);
                    }
                }
#pragma unroll
                for (int ct = 0; ct < 2; ct++) {
                    const int j = bn + 16 * ct + r16;
                    const float cj = cvec[voff + j];
                    float g1 = 0.f;
#pragma unroll
                    for (int rt = 0; rt < 2; rt++) {
                        const f32x4 kv = bf4_to_f32(Kr + j * LDB + bm + 16 * rt + 4 * g);
#pragma unroll
                        for (int r = 0; r < 4; r++) g1 = fmaf(t3[rt][ct][r], kv[r], g1);
                        dte[rt][ct] += cj * t3[rt][ct];
                    }
                    g1 = sum_groups(g1);
                    if (g == 0) part[(which * 2 + (bi >> 1)) * CW + j] = g1;
                }
            };
            state_term(dMr, 3, 2 * CW);
            if (HAS_S) {
                state_term(dSr, 4, 3 * CW);
            } else {
#pragma unroll
                for (int ct = 0; ct < 2; ct++)
                    if (g == 0) part[(4 * 2 + (bi >> 1)) * CW + bn + 16 * ct + r16] = 0.f;
            }
#pragma unroll
            for (int ks = 0; ks < 2; ks++) {
                bf16x8 bC[2];
#pragma unroll
                for (int ct = 0; ct < 2; ct++) bC[ct] = ld_op(CRt, bn + 16 * ct, ks);
#pragma unroll
                for (int rt = 0; rt < 2; rt++) {
                    const bf16x8 aq = ld_op_tr<LDB>(Qr, bm + 16 * rt, ks);   // Q^T
#pragma unroll
                    for (int ct = 0; ct < 2; ct++) dte[rt][ct] = mfma32(aq, bC[ct], dte[rt][ct]);
                }
            }
        }
        fetch_tab(min(task + 1, task_hi - 1));   // the table registers are free since the second phase
        __syncthreads();       // dE complete

        if (!grpA) {
            // ── dK^T [c][j] = -theta_j DTe^T + M0^T dE^T ──
            f32x4 em[2][2] = {{zero4(), zero4()}, {zero4(), zero4()}};
#pragma unroll
            for (int ks = 0; ks < 2; ks++) {
                bf16x8 bE[2];
#pragma unroll
                for (int ct = 0; ct < 2; ct++) bE[ct] = ld_op(dEr, bn + 16 * ct, ks);
#pragma unroll
                for (int rt = 0; rt < 2; rt++) {
                    const bf16x8 am = ld_op_tr<LDB>(M0h, bm + 16 * rt, ks);   // M0^T
#pragma unroll
                    for (int ct = 0; ct < 2; ct++) em[rt][ct] = mfma32(am, bE[ct], em[rt][ct]);
                }
            }
#pragma unroll
            for (int ct = 0; ct < 2; ct++) {
                const int j = bn + 16 * ct + r16;
                const float thj = cvec[4 * CW + j];
                if (j < L) {
#pragma unroll
                    for (int rt = 0; rt < 2; rt++)
                        put(d_k, go.gk, j, bm + 16 * rt + 4 * g, em[rt][ct] - thj * dte[rt][ct]);
                }
            }
        } else if (tid < L) {
            const int t = tid;
            d_theta[tok + t] = -(part[(2 * 2) * CW + t] + part[(2 * 2 + 1) * CW + t]);
            const float nth = -cvec[4 * CW + t];
            *reinterpret_cast<f32x4 *>(pvec + (tok + t) * 4) =
                f32x4{part[t] + part[CW + t], part[2 * CW + t] + part[3 * CW + t],
                      nth * (part[6 * CW + t] + part[7 * CW + t]), nth * (part[8 * CW + t] + part[9 * CW + t])};
        } else if (tid >= 64 && tid < 67) {
            const float *p = dots + 8 * (tid - 64);
            scal[(size_t)task * 4 + (tid - 64)] = p[0] + p[1] + p[2] + p[3] + p[4] + p[5] + p[6] + p[7];
        }
        __syncthreads();   // LDS is rewritten by the next task
    }
}

constexpr size_t kGradsLds = 11 * BMAT * sizeof(u16) + (5 * CW + 10 * CW + 24 + CW * kCtLd) * sizeof(float);

}  // namespace

size_t chunkwise_grads_table_floats() { return kTab; }
size_t chunkwise_grads_vec_floats() { return kVecB; }

void chunkwise_backward_coefficients(const float *alpha, const float *theta, const float *eta,
                                     float *tab_b, float *vecs, int seq_len, int batch, int chunk_size, bool has_s) {
    const int nc = ceil_div(seq_len, chunk_size), ntask = batch * nc;
    KernelTimer kt("cw_coef_bwd_kernel");
    if (has_s)
        hipLaunchKernelGGL(cw_coef_bwd_kernel<true>, dim3(ceil_div(ntask, kCoefChunksPerWave)), dim3(64), 0, stream(), alpha, theta,
                           eta, tab_b, vecs, seq_len, chunk_size, nc, ntask);
    else
        hipLaunchKernelGGL(cw_coef_bwd_kernel<false>, dim3(ceil_div(ntask, kCoefChunksPerWave)), dim3(64), 0, stream(), alpha, theta,
                           nullptr, tab_b, vecs, seq_len, chunk_size, nc, ntask);
    check_launch("cw_coef_bwd_kernel");
}

bool chunkwise_grads_bf16(const uint16_t *k, const uint16_t *v, const uint16_t *q, const float *d_y,
                          const float *m_states, const float *s_states, const uint16_t *dm_snap,
                          const uint16_t *ds_snap, float *d_k, float *d_v, float *d_q, float *d_theta, float *pvec,
                          float *xs, float *scal, const float *tab_b, const float *vecs,
                          int seq_len, int batch, int chunk_size, bool has_s, int grid, const HeadRows *dy_rows,
                          const GradOut16 *out16, const ChainTracks *tracks) {
    const ErrorScope es;
    if (tracks && out16) { fail("chunkwise_grads_bf16: the in-pass test is not served together with bf16 gradient slabs."); return true; }
    const int nc = ceil_div(seq_len, chunk_size), ntask = batch * nc;
    const HeadRows dyr = dy_rows ? *dy_rows : head_major_rows(seq_len, HD);
    static bool attr_set = false;
    if (!attr_set) {
        const void *fns[6] = {reinterpret_cast<const void *>(cw_grads_bf16_kernel<true, false, false>),
                              reinterpret_cast<const void *>(cw_grads_bf16_kernel<false, false, false>),
                              reinterpret_cast<const void *>(cw_grads_bf16_kernel<true, true, false>),
                              reinterpret_cast<const void *>(cw_grads_bf16_kernel<false, true, false>),
                              reinterpret_cast<const void *>(cw_grads_bf16_kernel<true, false, true>),
                              reinterpret_cast<const void *>(cw_grads_bf16_kernel<false, false, true>)};
        for (const void *f : fns) check_hip(hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kGradsLds), "dynamic LDS size");
        attr_set = true;
    }
    if (es.failed()) return true;
    const GradOut16 go = out16 ? *out16 : GradOut16{};
    KernelTimer kt("cw_grads_bf16_kernel");
    const ChainTracks tr = tracks ? *tracks : ChainTracks{nullptr, nullptr};
#define NLH_CWG(HS, G, T) \
    hipLaunchKernelGGL((cw_grads_bf16_kernel<HS, G, T>), dim3(grid), dim3(kTileThr), kGradsLds, stream(), k, v, q, d_y, tab_b, vecs, \
                       m_states, HS ? s_states : nullptr, dm_snap, HS ? ds_snap : nullptr, d_k, d_v, d_q, d_theta, pvec, xs, scal, \
                       seq_len, chunk_size, nc, ntask, dyr, go, tr)
    if (tracks) { if (has_s) NLH_CWG(true, false, true); else NLH_CWG(false, false, true); }
    else if (has_s) { if (out16) NLH_CWG(true, true, false); else NLH_CWG(true, false, false); }
    else { if (out16) NLH_CWG(false, true, false); else NLH_CWG(false, false, false); }
#undef NLH_CWG
    check_launch("cw_grads_bf16_kernel");
    return true;
}

}  // namespace nlh
