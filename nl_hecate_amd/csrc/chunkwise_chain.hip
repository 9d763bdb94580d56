// Frozen-M0 chunkwise Titans / Delta rule on bf16 tokens with the memory resident on chip.
//
// Semantics are those of core/kernels/titans_chunkwise_forward.cu / _backward.cu with
// error_clip and the M-norm projection off (see chunkwise_mm.hip for the matrix form:
// coefficients r, bb, c, a, beta, h and W[t][j] = -theta_j c[t][j]).
//
// One workgroup owns one chain (batch element x head) and walks its chunks in order.  The
// fp32 master copy of M and S lives in registers (accumulator layout of the matrix cores),
// a bf16 hi/lo split of it in LDS as the operand of the products of the next chunk, so a
// state never travels through HBM between chunks; HBM sees each token once (k, v, q in,
// y out) plus one state snapshot per chunk for the backward.  Per chunk, with
// E = K M0^T - V,  P = Q K^T:
//   Y  = a.(Q M0^T) + beta.(Q S0^T) + (W.P) E
//   M' = a_L M0 + beta_L S0 + (E.wM)^T K        S' = h_L S0 + (E.wS)^T K
// All products run on v_mfma_f32_16x16x32_bf16.  k, v, q are exact in bf16; every fp32
// operand (states, E, W.P) enters as a hi + lo pair of bf16 (16 mantissa bits), the
// accumulation is fp32.
//
// Eight waves compute, one 16x32 output strip each per product.  The coefficients depend on
// the gates only: a chunk-parallel kernel runs their 64-step scalar recurrences up front and
// leaves W in the accumulator order of the chain kernel, which prefetches one chunk ahead.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "bf16_tiles.h"
#include "chunkwise_chain.h"
#include "runtime.h"

namespace nlh {
namespace {

constexpr int kChainThr = 512;     // 8 waves

// Work split of the eight waves: a 64x64 product is four 32x32 blocks (2x2 tiles of 16x16; an
// A or B operand read from LDS then serves two tiles).  Wave w works on block bi = w%4 with
// origin (32 (bi/2), 32 (bi%2)); waves 0..3 (group X) compute E and then Y, waves 4..7
// (group Y) compute W.P and then the state update, and hold the fp32 master state.
//
// Per-chunk coefficients in HBM, written by cw_coef_kernel:
//   table [chunk][block bi][rt][ct][lane l][r]: W[t][j] = -theta_j c[t][j] (zero outside j <= t < L)
//         at j = 32 (bi/2) + 16 rt + 4 (l/16) + r, t = 32 (bi%2) + 16 ct + l%16: the order in which
//         lane l of a group-Y wave holds P^T; tiles entirely above the diagonal are neither
//         written nor read
//   vecs  [chunk][kVecFloats]: a_t, beta_t, wM_j = -theta_j c[L-1][j], wS_j = -theta_j bb[j][L-1],
//         then a_L, beta_L, h_L, one unused float and four zeros
constexpr int kTableFloats = CW * CW;
constexpr int kVecFloats = 4 * CW + 16;
__device__ __forceinline__ bool tile_live(int bi, int rt, int ct) { return 2 * (bi & 1) + ct >= 2 * (bi >> 1) + rt; }

// Coefficients of one chunk from its gates: two waves per chunk.  Wave role 0 (lane j): the
// column recurrences c[t][j], bb[j][t] over t.  Role 1 (lane t): a_t, beta_t, h_t.
template <bool HAS_S>
__global__ __launch_bounds__(256) void cw_coef_kernel(const float *__restrict__ alpha,
                                                      const float *__restrict__ theta,
                                                      const float *__restrict__ eta, float *__restrict__ table,
                                                      float *__restrict__ vecs, int s, int C, int nc, int nchunks) {
    const int chunk = blockIdx.x * 2 + (threadIdx.x >> 7), role = (threadIdx.x >> 6) & 1, j = threadIdx.x & 63;
    if (chunk >= nchunks) return;
    const int chain = chunk / nc, ci = chunk % nc, t0 = ci * C, L = min(C, s - t0);
    const Gates g = fetch_gates<HAS_S>(alpha, theta, eta, (size_t)chain * s + t0, L);
    const float keep_j = 1.f - g.al;   // 1 beyond L
    const float eta_j = g.et;          // 0 beyond L
    float *vo = vecs + (size_t)chunk * kVecFloats;
    if (role == 0) {
        float *to = table + (size_t)chunk * kTableFloats;
        float b = 1.f, cc = 1.f, blv = 0.f;
        const bool jv = j < L;
        const float nth = -g.th;
        // destination of W[t][j]: block 2 (j/32) + t/32, rt = (j/16)%2, ct = (t/16)%2,
        // lane 16 ((j%16)/4) + t%16, element j%4
        const int jbase = (j >> 5) * 2048 + ((j >> 4) & 1) * 512 + ((j & 15) >> 2) * 64 + (j & 3);
#pragma unroll
        for (int t = 0; t < CW; t++) {
            const float keep = lane_bcast(keep_j, t), et = lane_bcast(eta_j, t);
            const bool after = t > j;
            b *= after ? et : 1.f;
            cc = after ? fmaf(keep, cc, b) : cc;
            blv = (t == L - 1) ? b : blv;
            if ((t >> 4) >= (j >> 4))
                to[jbase + (t >> 5) * 1024 + ((t >> 4) & 1) * 256 + (t & 15) * 4] =
                    (jv && t >= j && t < L) ? nth * cc : 0.f;
        }
        vo[2 * CW + j] = jv ? nth * cc : 0.f;
        vo[3 * CW + j] = jv ? nth * blv : 0.f;
    } else {
        float a = 1.f, h = 1.f, beta = 0.f, ka = 0.f, kb = 0.f, kh = 0.f;
#pragma unroll
        for (int t = 0; t < CW; t++) {
            const float keep = lane_bcast(keep_j, t), et = lane_bcast(eta_j, t);
            a *= keep;
            h *= et;
            beta = fmaf(keep, beta, h);
            if (t == j) { ka = a; kb = beta; kh = h; }
        }
        vo[j] = j < L ? ka : 0.f;
        vo[CW + j] = j < L ? kb : 0.f;
        if (j == L - 1) { vo[4 * CW] = ka; vo[4 * CW + 1] = kb; vo[4 * CW + 2] = kh; }
        if (j < 4) vo[4 * CW + 4 + j] = 0.f;   // zero pad: what tiles of W above the diagonal read
    }
}

// Pipeline of one chunk step.  Every global load of chunk c+1 (tokens, W, coefficient vectors)
// is issued at the top of step c and first touched at the bottom of step c, after the matrix
// work and before the stores of step c, so no wait inside a step ever meets a load in flight
// or a store just issued.
template <bool HAS_S>
__global__ __launch_bounds__(kChainThr) void cw_chain_fwd_kernel(
    const u16 *__restrict__ k, const u16 *__restrict__ v, const u16 *__restrict__ q,
    const float *__restrict__ table, const float *__restrict__ vecs, const float *__restrict__ m_initial,
    const float *__restrict__ s_initial, float *__restrict__ m_states, float *__restrict__ s_states,
    float *__restrict__ y, int s, int C, int nc) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    u16 *Kr = reinterpret_cast<u16 *>(smem_raw);   // K [t][c]
    u16 *Kt0 = Kr + BMAT, *Kt1 = Kt0 + BMAT;       // K^T [c][t] of this chunk / V [t][i] until K^T of the next lands
    u16 *Qr0 = Kt1 + BMAT, *Qr1 = Qr0 + BMAT;      // Q [t][c], alternating between chunks
    u16 *Mh = Qr1 + BMAT, *Ml = Mh + BMAT;         // chunk-start M [i][c], hi / lo
    u16 *Sh = Ml + BMAT, *Sl = Sh + BMAT;          // chunk-start S
    u16 *Eh = Sl + BMAT, *El = Eh + BMAT;          // E^T [i][t]
    u16 *EMh = El + BMAT, *EMl = EMh + BMAT;       // (E.wM)^T
    u16 *ESh = EMl + BMAT, *ESl = ESh + BMAT;      // (E.wS)^T
    u16 *WPh = ESl + BMAT, *WPl = WPh + BMAT;      // W.P [t][j]
    float *cvec = reinterpret_cast<float *>(WPl + BMAT);   // a, beta, wM, wS [64] each, then a_L, beta_L, h_L

    const int chain = blockIdx.x, tid = threadIdx.x, w = tid >> 6, l = tid & 63, g = l >> 4, r16 = l & 15;
    const bool grpX = w < 4;
    const int bi = w & 3, bm = 32 * (bi >> 1), bn = 32 * (bi & 1);   // origin of this wave's 32x32 block
    const size_t chain_tok = (size_t)chain * s;
    const size_t state0 = (size_t)chain * (nc + 1) * HD * HD;

    // -V enters E = K M0^T - V as one more step of the product: A = V (rows t), B = -identity.
    // Output columns bn + 16 ct + l%16 meet contraction indices 32 (bn/32) + 8 (l/16) + e.
    bf16x8 negI[2];
#pragma unroll
    for (int ct = 0; ct < 2; ct++) {
        const int hit = 16 * ct + r16 - 8 * g;   // element of this lane's eight that is -1 (bf16 0xBF80), if in 0..7
        uint4 bits;
        bits.x = (hit == 0 ? 0xBF80u : 0u) | (hit == 1 ? 0xBF800000u : 0u);
        bits.y = (hit == 2 ? 0xBF80u : 0u) | (hit == 3 ? 0xBF800000u : 0u);
        bits.z = (hit == 4 ? 0xBF80u : 0u) | (hit == 5 ? 0xBF800000u : 0u);
        bits.w = (hit == 6 ? 0xBF80u : 0u) | (hit == 7 ? 0xBF800000u : 0u);
        negI[ct] = __builtin_bit_cast(bf16x8, bits);
    }

    // Registers of the next chunk.  Every wave: 8 consecutive bf16 of one row of K, Q, V
    // (lane -> row st_t, 8-column block st_cb) and W at the accumulator positions of its P^T
    // block (used by group Y).  Threads 0..271: one float of the coefficient vectors.
    const int st_t = 32 * (w & 1) + (l & 31), st_cb = 2 * (w >> 1) + (l >> 5);
    uint4 sk, sq, sv;
    f32x4 wn[2][2], wc[2][2];
    float vn = 0.f;
    // All loads are unconditional (rows beyond a short last chunk re-read its last row and are
    // zeroed when committed; tiles of W above the diagonal read the zero pad of vecs).
    auto fetch = [&](int c) {
        const int L = min(C, s - c * C);
        const size_t o = (chain_tok + (size_t)c * C + min(st_t, L - 1)) * HD + st_cb * 8;
        sk = *reinterpret_cast<const uint4 *>(k + o);
        sq = *reinterpret_cast<const uint4 *>(q + o);
        sv = *reinterpret_cast<const uint4 *>(v + o);
        const size_t chunk = (size_t)chain * nc + c;
        const float *tb = table + chunk * kTableFloats, *vo = vecs + chunk * kVecFloats;
#pragma unroll
        for (int rt = 0; rt < 2; rt++)
#pragma unroll
            for (int ct = 0; ct < 2; ct++)
                wn[rt][ct] = *reinterpret_cast<const f32x4 *>(
                    tile_live(bi, rt, ct) ? tb + (((bi * 2 + rt) * 2 + ct) * 64 + l) * 4 : vo + 4 * CW + 4);
        vn = vo[min(tid, 4 * CW + 3)];
    };
    auto land = [&](int c) {   // wait for the loads here; zero the rows beyond a short chunk
        if (st_t >= min(C, s - c * C)) { sk = make_uint4(0, 0, 0, 0); sq = sk; sv = sk; }
#pragma unroll
        for (int rt = 0; rt < 2; rt++)
#pragma unroll
            for (int ct = 0; ct < 2; ct++) wc[rt][ct] = wn[rt][ct];
        // V and the vectors are written to LDS later, behind the stores of this step: pin their
        // arrival to this point
        asm volatile("" : "+v"(sv.x), "+v"(sv.y), "+v"(sv.z), "+v"(sv.w), "+v"(vn));
    };
    auto commit_rows = [&](u16 *dst, const uint4 &x) { *reinterpret_cast<uint4 *>(dst + st_t * LDB + st_cb * 8) = x; };
    auto commit_kt = [&](u16 *Kt) {
        const unsigned kw[4] = {sk.x, sk.y, sk.z, sk.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            Kt[(st_cb * 8 + 2 * i) * LDB + st_t] = (u16)(kw[i] & 0xffffu);
            Kt[(st_cb * 8 + 2 * i + 1) * LDB + st_t] = (u16)(kw[i] >> 16);
        }
    };
    auto commit_vecs = [&]() {
        if (tid < 4 * CW + 4) cvec[tid] = vn;
    };

    // fp32 master state (group Y), transposed block:
    //   Mm[rt][ct][r] = M[i = bn + 16 ct + l%16][c = bm + 16 rt + 4 (l/16) + r]
    // Group X has no state; it borrows the same registers as accumulators of Q M0^T and Q S0^T.
    f32x4 Mm[2][2], Sm[2][2];
    auto state_off = [&](int rt, int ct) { return (bn + 16 * ct + r16) * HD + bm + 16 * rt + 4 * g; };
    auto publish_state = [&](int slot) {   // -> HBM snapshot
#pragma unroll
        for (int rt = 0; rt < 2; rt++)
#pragma unroll
            for (int ct = 0; ct < 2; ct++) {
                const size_t o = state0 + (size_t)slot * HD * HD + state_off(rt, ct);
                *reinterpret_cast<f32x4 *>(m_states + o) = Mm[rt][ct];
                if (HAS_S) *reinterpret_cast<f32x4 *>(s_states + o) = Sm[rt][ct];
            }
    };
    auto stage_state = [&]() {             // -> LDS operands of the next chunk
#pragma unroll
        for (int rt = 0; rt < 2; rt++)
#pragma unroll
            for (int ct = 0; ct < 2; ct++) {
                const int off = (bn + 16 * ct + r16) * LDB + bm + 16 * rt + 4 * g;
                split_store(Mh, Ml, off, Mm[rt][ct]);
                if (HAS_S) split_store(Sh, Sl, off, Sm[rt][ct]);
            }
    };

    fetch(0);
    if (!grpX) {
#pragma unroll
        for (int rt = 0; rt < 2; rt++)
#pragma unroll
            for (int ct = 0; ct < 2; ct++) {
                const size_t o = (size_t)chain * HD * HD + state_off(rt, ct);
                Mm[rt][ct] = *reinterpret_cast<const f32x4 *>(m_initial + o);
                Sm[rt][ct] = HAS_S ? *reinterpret_cast<const f32x4 *>(s_initial + o) : zero4();
            }
        publish_state(0);
        stage_state();
    }
    land(0);
    commit_rows(Kr, sk);
    commit_rows(Qr0, sq);
    commit_kt(Kt0);
    commit_rows(Kt1, sv);
    commit_vecs();
    __syncthreads();

    for (int c = 0; c < nc; c++) {
        const int t0 = c * C, L = min(C, s - t0);
        const size_t tok = chain_tok + t0;
        const bool more = c + 1 < nc;
        // this chunk: Q in Qc, K^T in Kc, V in Kn (until K^T of the next chunk replaces it)
        u16 *Qc = (c & 1) ? Qr1 : Qr0, *Kc = (c & 1) ? Kt1 : Kt0;
        u16 *Qn = (c & 1) ? Qr0 : Qr1, *Kn = (c & 1) ? Kt0 : Kt1;
        if (more) fetch(c + 1);
        // ── first half: E^T, (E.wM)^T, (E.wS)^T (group X) and W.P (group Y) ──
        {
            bf16x8 aK[2][2];
#pragma unroll
            for (int rt = 0; rt < 2; rt++)
#pragma unroll
                for (int ks = 0; ks < 2; ks++) aK[rt][ks] = ld_op(Kr, bm + 16 * rt, ks);
            f32x4 acc[2][2] = {{zero4(), zero4()}, {zero4(), zero4()}};
            if (grpX) {
                const bf16x8 aV[2] = {ld_op(Kn, bm, bn >> 5), ld_op(Kn, bm + 16, bn >> 5)};
#pragma unroll
                for (int ks = 0; ks < 2; ks++)
#pragma unroll
                    for (int ct = 0; ct < 2; ct++) {
                        const bf16x8 bh = ld_op(Mh, bn + 16 * ct, ks), bl = ld_op(Ml, bn + 16 * ct, ks);
#pragma unroll
                        for (int rt = 0; rt < 2; rt++) {   // E[t][i]: rows t, columns i
                            acc[rt][ct] = mfma32(aK[rt][ks], bh, acc[rt][ct]);
                            acc[rt][ct] = mfma32(aK[rt][ks], bl, acc[rt][ct]);
                        }
                    }
#pragma unroll
                for (int rt = 0; rt < 2; rt++) {
                    const f32x4 wm = *reinterpret_cast<const f32x4 *>(cvec + 2 * CW + bm + 16 * rt + 4 * g);
                    const f32x4 wsv = *reinterpret_cast<const f32x4 *>(cvec + 3 * CW + bm + 16 * rt + 4 * g);
#pragma unroll
                    for (int ct = 0; ct < 2; ct++) {
                        const f32x4 ev = mfma32(aV[rt], negI[ct], acc[rt][ct]);
                        const int off = (bn + 16 * ct + r16) * LDB + bm + 16 * rt + 4 * g;   // [i][t .. t+3]
                        split_store(Eh, El, off, ev);
                        split_store(EMh, EMl, off, ev * wm);
                        if (HAS_S) split_store(ESh, ESl, off, ev * wsv);
                    }
                }
            } else {
#pragma unroll
                for (int ks = 0; ks < 2; ks++)
#pragma unroll
                    for (int ct = 0; ct < 2; ct++) {
                        const bf16x8 bq = ld_op(Qc, bn + 16 * ct, ks);
#pragma unroll
                        for (int rt = 0; rt < 2; rt++)     // P^T[j][t]: rows j, columns t
                            acc[rt][ct] = mfma32(aK[rt][ks], bq, acc[rt][ct]);
                    }
#pragma unroll
                for (int rt = 0; rt < 2; rt++)
#pragma unroll
                    for (int ct = 0; ct < 2; ct++)         // [t][j .. j+3]
                        split_store(WPh, WPl, (bn + 16 * ct + r16) * LDB + bm + 16 * rt + 4 * g,
                                    wc[rt][ct] * acc[rt][ct]);
            }
        }
        __syncthreads();
        // ── second half: Y (group X) and the state update (group Y) ──
        f32x4 y2[2][2] = {{zero4(), zero4()}, {zero4(), zero4()}};   // group X: (W.P) E; group Y: unused
        if (grpX) {
            // rows t in [bm, bm+32), columns i in [bn, bn+32)
            f32x4(&y0)[2][2] = Mm, (&y1)[2][2] = Sm;
#pragma unroll
            for (int rt = 0; rt < 2; rt++)
#pragma unroll
                for (int ct = 0; ct < 2; ct++) { y0[rt][ct] = zero4(); y1[rt][ct] = zero4(); }
#pragma unroll
            for (int ks = 0; ks < 2; ks++) {
                bf16x8 aQ[2], aWh[2], aWl[2];
#pragma unroll
                for (int rt = 0; rt < 2; rt++) {
                    aQ[rt] = ld_op(Qc, bm + 16 * rt, ks);
                    aWh[rt] = ld_op(WPh, bm + 16 * rt, ks);
                    aWl[rt] = ld_op(WPl, bm + 16 * rt, ks);
                }
#pragma unroll
                for (int ct = 0; ct < 2; ct++) {
                    const int i0 = bn + 16 * ct;
                    const bf16x8 mh = ld_op(Mh, i0, ks), ml = ld_op(Ml, i0, ks);
                    const bf16x8 eh = ld_op(Eh, i0, ks), el = ld_op(El, i0, ks);
#pragma unroll
                    for (int rt = 0; rt < 2; rt++) {
                        y0[rt][ct] = mfma32(aQ[rt], mh, y0[rt][ct]);
                        y0[rt][ct] = mfma32(aQ[rt], ml, y0[rt][ct]);
                        y2[rt][ct] = mfma32(aWh[rt], eh, y2[rt][ct]);
                        y2[rt][ct] = mfma32(aWl[rt], eh, y2[rt][ct]);
                        y2[rt][ct] = mfma32(aWh[rt], el, y2[rt][ct]);
                    }
                    if (HAS_S) {
                        const bf16x8 sh = ld_op(Sh, i0, ks), sl = ld_op(Sl, i0, ks);
#pragma unroll
                        for (int rt = 0; rt < 2; rt++) {
                            y1[rt][ct] = mfma32(aQ[rt], sh, y1[rt][ct]);
                            y1[rt][ct] = mfma32(aQ[rt], sl, y1[rt][ct]);
                        }
                    }
                }
            }
#pragma unroll
            for (int rt = 0; rt < 2; rt++) {
                const f32x4 at = *reinterpret_cast<const f32x4 *>(cvec + bm + 16 * rt + 4 * g);
                const f32x4 bt = *reinterpret_cast<const f32x4 *>(cvec + CW + bm + 16 * rt + 4 * g);
#pragma unroll
                for (int ct = 0; ct < 2; ct++) y2[rt][ct] += at * y0[rt][ct] + bt * y1[rt][ct];
            }
        } else {
            // transposed state block: rows c in [bm, bm+32), columns i in [bn, bn+32)
            f32x4 am[2][2] = {{zero4(), zero4()}, {zero4(), zero4()}}, as[2][2] = {{zero4(), zero4()}, {zero4(), zero4()}};
#pragma unroll
            for (int ks = 0; ks < 2; ks++) {
                bf16x8 aKt[2];
#pragma unroll
                for (int rt = 0; rt < 2; rt++) aKt[rt] = ld_op(Kc, bm + 16 * rt, ks);
#pragma unroll
                for (int ct = 0; ct < 2; ct++) {
                    const int i0 = bn + 16 * ct;
                    const bf16x8 mh = ld_op(EMh, i0, ks), ml = ld_op(EMl, i0, ks);
#pragma unroll
                    for (int rt = 0; rt < 2; rt++) {
                        am[rt][ct] = mfma32(aKt[rt], mh, am[rt][ct]);
                        am[rt][ct] = mfma32(aKt[rt], ml, am[rt][ct]);
                    }
                    if (HAS_S) {
                        const bf16x8 sh = ld_op(ESh, i0, ks), sl = ld_op(ESl, i0, ks);
#pragma unroll
                        for (int rt = 0; rt < 2; rt++) {
                            as[rt][ct] = mfma32(aKt[rt], sh, as[rt][ct]);
                            as[rt][ct] = mfma32(aKt[rt], sl, as[rt][ct]);
                        }
                    }
                }
            }
            const float aL = cvec[4 * CW], betaL = cvec[4 * CW + 1], hL = cvec[4 * CW + 2];
#pragma unroll
            for (int rt = 0; rt < 2; rt++)
#pragma unroll
                for (int ct = 0; ct < 2; ct++) {
                    Mm[rt][ct] = aL * Mm[rt][ct] + betaL * Sm[rt][ct] + am[rt][ct];
                    if (HAS_S) Sm[rt][ct] = hL * Sm[rt][ct] + as[rt][ct];
                }
        }
        // tokens of the next chunk land: K and V of this one are no longer read
        if (more) {
            land(c + 1);
            commit_rows(Kr, sk);
            commit_rows(Qn, sq);
            commit_kt(Kn);
        }
        // results of this chunk leave
        if (grpX) {
#pragma unroll
            for (int rt = 0; rt < 2; rt++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int t = bm + 16 * rt + 4 * g + r;
                    if (t < L) {
#pragma unroll
                        for (int ct = 0; ct < 2; ct++) y[(tok + t) * HD + bn + 16 * ct + r16] = y2[rt][ct][r];
                    }
                }
        } else {
            publish_state(c + 1);
        }
        __syncthreads();
        if (more) {
            if (!grpX) stage_state();
            commit_rows(Kc, sv);   // K^T of this chunk is no longer read
            commit_vecs();
        }
        __syncthreads();
    }
}

constexpr size_t kChainFwdLds = 17 * BMAT * sizeof(u16) + (4 * CW + 4) * sizeof(float);

template <bool HAS_S>
void launch_forward(const char *fn, const u16 *k, const u16 *v, const u16 *q, const float *alpha, const float *theta,
                    const float *eta, const float *m_initial, const float *s_initial, float *m_states,
                    float *s_states, float *y, int seq_len, int batch, int chunk_size) {
    const int nc = ceil_div(seq_len, chunk_size), nchunks = batch * nc;
    float *table = scratch(3, (size_t)nchunks * kTableFloats * sizeof(float));
    float *vecs = scratch(4, (size_t)nchunks * kVecFloats * sizeof(float));
    static bool attr_set = false;
    if (!attr_set) {
        check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(cw_chain_fwd_kernel<HAS_S>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)kChainFwdLds),
                  "dynamic LDS size");
        attr_set = true;
    }
    if (failed()) return;
    hipLaunchKernelGGL(cw_coef_kernel<HAS_S>, dim3(ceil_div(nchunks, 2)), dim3(256), 0, stream(), alpha, theta, eta,
                       table, vecs, seq_len, chunk_size, nc, nchunks);
    check_launch("cw_coef_kernel");
    hipLaunchKernelGGL(cw_chain_fwd_kernel<HAS_S>, dim3(batch), dim3(kChainThr), kChainFwdLds, stream(), k, v, q,
                       table, vecs, m_initial, s_initial, m_states, s_states, y, seq_len, chunk_size, nc);
    check_launch(fn);
}

}  // namespace

bool chunkwise_chain_forward_bf16(const char *fn, const uint16_t *k, const uint16_t *v, const uint16_t *q,
                                  const float *alpha, const float *theta, const float *eta, const float *m_initial,
                                  const float *s_initial, float *m_states, float *s_states, float *y, int seq_len,
                                  int d, int batch, int chunk_size, bool has_s) {
    if (d != HD || chunk_size < 1 || chunk_size > CW || seq_len <= 0 || batch <= 0) return false;
    if (has_s)
        launch_forward<true>(fn, k, v, q, alpha, theta, eta, m_initial, s_initial, m_states, s_states, y, seq_len,
                             batch, chunk_size);
    else
        launch_forward<false>(fn, k, v, q, alpha, theta, nullptr, m_initial, nullptr, m_states, nullptr, y, seq_len,
                              batch, chunk_size);
    return true;
}

}  // namespace nlh
