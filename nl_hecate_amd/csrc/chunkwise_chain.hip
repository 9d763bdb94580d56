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
#include "chunk_coef.h"
#include "chunkwise_chain.h"
#include "lane_ops.h"
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
constexpr int kStageLd = CW + 4;   // row stride (floats) of the table while it is assembled in LDS
constexpr int kCoefChunksPerWave = 4;
__device__ __forceinline__ bool tile_live(int bi, int rt, int ct) { return 2 * (bi & 1) + ct >= 2 * (bi >> 1) + rt; }

// Coefficients of one chunk from its gates: one wave per chunk, lane = token.  The vectors come from two scans
// of composed maps, the table from coef_table_columns; it is assembled in LDS as W[t][j] and leaves in the
// consumers' order as 16-byte stores of consecutive lanes.
template <bool HAS_S>
__global__ __launch_bounds__(64) void cw_coef_kernel(const float *__restrict__ alpha,
                                                     const float *__restrict__ theta,
                                                     const float *__restrict__ eta, float *__restrict__ table,
                                                     float *__restrict__ vecs, int s, int C, int nc, int nchunks) {
    __shared__ __align__(16) float stage[(CW + 1) * kStageLd];
    __shared__ float gk[2 * CW], ge[2 * CW];
    const int j = threadIdx.x, first = blockIdx.x * kCoefChunksPerWave, last = min(nchunks, first + kCoefChunksPerWave);
    auto gates_of = [&](int chunk) {
        const int chain = chunk / nc, t0 = (chunk % nc) * C;
        return fetch_gates<HAS_S>(alpha, theta, eta, (size_t)chain * s + t0, min(C, s - t0));
    };
    // a wave walks over a few chunks with the next chunk's gates in flight: a wave per chunk would spend most of
    // its life waiting for its three loads, and LDS allows only eight waves per compute unit
    Gates gn = gates_of(first);
    for (int chunk = first; chunk < last; chunk++) {
        const int L = min(C, s - (chunk % nc) * C);
        const Gates g = gn;
        gn = gates_of(min(chunk + 1, last - 1));
        const bool jv = j < L;
        const float keep = 1.f - g.al, et = g.et, nth = -g.th;   // 1, 0, 0 beyond L
        const ChunkVectors cv = coef_vectors(keep, et, jv);
        float *vo = vecs + (size_t)chunk * kVecFloats;
        vo[j] = jv ? cv.a : 0.f;
        vo[CW + j] = jv ? cv.beta : 0.f;
        vo[2 * CW + j] = nth * cv.cl;
        vo[3 * CW + j] = nth * cv.bl;
        if (j == 63) { vo[4 * CW] = cv.a; vo[4 * CW + 1] = cv.beta; vo[4 * CW + 2] = cv.h; }   // the values at token L - 1
        if (j < 4) vo[4 * CW + 4 + j] = 0.f;   // zero pad: what tiles of W above the diagonal read
        coef_table_columns<kStageLd, true>(stage, gk, ge, keep, et, nth, L);
        float *out = table + (size_t)chunk * kTableFloats;
        // the ten 16 x 16 tiles on or below the diagonal (token tile T >= column tile J), one 16-byte piece per lane each
#pragma unroll
        for (int T = 0; T < 4; T++)
#pragma unroll
            for (int J = 0; J <= T; J++) {
                const int tile = ((J >> 1) * 2 + (T >> 1)) * 4 + (J & 1) * 2 + (T & 1);   // (bi, rt, ct) of the layout above
                *reinterpret_cast<f32x4 *>(out + (tile * 64 + j) * 4) =
                    *reinterpret_cast<const f32x4 *>(stage + (16 * T + (j & 15)) * kStageLd + 16 * J + 4 * (j >> 4));
            }
    }
}

// Pipeline of one chunk step.  Every global load of chunk c+1 (tokens, W, coefficient vectors)
// is issued at the top of step c and first touched at the bottom of step c, after the matrix
// work and before the stores of step c, so no wait inside a step ever meets a load in flight
// or a store just issued.  The requests and their landing are unconditional (past the end they
// repeat the last chunk): memory waits are placed per program point, not per path.
//
// The rows of M and S never mix, so a chain is split over two workgroups of 32 rows each
// (chain_half_of_block: both halves of a chain share an XCD's L2 and are dispatched together
// for K, Q and W).  Waves 0..3 (group X): E, then Y^T, one 16-token strip each.  Waves 4..7
// (group Y): one 32x32 block of W.P each, then one 16-column strip of the transposed state
// update; they hold the fp32 master state.
// TRACK: also leaves the per-token error norms and the chunk-start state norms of ChainTracks behind.
template <bool HAS_S, bool TRACK>
__global__ __launch_bounds__(kChainThr) void cw_chain_fwd_kernel(
    const u16 *__restrict__ k, const u16 *__restrict__ v, const u16 *__restrict__ q,
    const float *__restrict__ table, const float *__restrict__ vecs, const float *__restrict__ m_initial,
    const float *__restrict__ s_initial, float *__restrict__ m_states, float *__restrict__ s_states,
    float *__restrict__ y, int s, int C, int nc, int batch, HeadRows yr, ChainTracks tr) {
    constexpr int HMAT = 32 * LDB;   // a 32-row matrix
    extern __shared__ __align__(16) unsigned char smem_raw[];
    u16 *Kr = reinterpret_cast<u16 *>(smem_raw);   // K [t][c]
    u16 *Kt0 = Kr + BMAT, *Kt1 = Kt0 + BMAT;       // K^T [c][t] of this chunk / V [t][i] until K^T of the next lands
    u16 *Qr0 = Kt1 + BMAT, *Qr1 = Qr0 + BMAT;      // Q [t][c], alternating between chunks
    u16 *WPh = Qr1 + BMAT, *WPl = WPh + BMAT;      // W.P [t][j]
    u16 *Mh = WPl + BMAT, *Ml = Mh + HMAT;         // chunk-start M [i][c], this workgroup's 32 rows, hi / lo
    u16 *Sh = Ml + HMAT, *Sl = Sh + HMAT;          // chunk-start S
    u16 *Eh = Sl + HMAT, *El = Eh + HMAT;          // E^T [i][t]
    u16 *EMh = El + HMAT, *EMl = EMh + HMAT;       // (E.wM)^T
    u16 *ESh = EMl + HMAT, *ESl = ESh + HMAT;      // (E.wS)^T
    float *cvec = reinterpret_cast<float *>(ESl + HMAT);   // a, beta, wM, wS [64] each, then a_L, beta_L, h_L

    const int tid = threadIdx.x, w = tid >> 6, l = tid & 63, g = l >> 4, r16 = l & 15;
    int chain, half;
    chain_half_of_block(batch, chain, half);
    const int i0 = 32 * half;
    const bool grpX = w < 4;
    const int bi = w & 3, bm = 32 * (bi >> 1), bn = 32 * (bi & 1);   // group Y: 32x32 block of P^T; group X: strip bi
    const size_t chain_tok = (size_t)chain * s;
    const size_t state0 = (size_t)chain * (nc + 1) * HD * HD;
    const size_t y_off = yr.offset(chain);

    // -V enters E = K M0^T - V as one more step of the product: A = V (rows t, this half's 32
    // columns as contraction), B = -identity: column 16 ct + l%16 meets contraction index 8 (l/16) + e.
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

    // Registers of the next chunk.  K, Q: row st_t, 8-element block st_cb (16 rows x 64 bytes per
    // wave instruction).  V (threads 0..255): row vt, block vcb of this half's 32 columns.  Group Y:
    // W at the accumulator positions of its P^T block.  Threads 0..259: one float of the vectors.
    const int st_t = 16 * (w & 3) + (l & 15), st_cb = 4 * (w >> 2) + (l >> 4);
    const int vt = (tid >> 2) & 63, vcb = tid & 3;
    uint4 sk, sq, sv;
    f32x4 wn[2][2], wc[2][2];
    float vn = 0.f;
    auto fetch = [&](int c) {
        const int L = min(C, s - c * C);
        const size_t tok = chain_tok + (size_t)c * C;
        const size_t o = (tok + min(st_t, L - 1)) * HD + st_cb * 8;
        sk = *reinterpret_cast<const uint4 *>(k + o);
        sq = *reinterpret_cast<const uint4 *>(q + o);
        sv = *reinterpret_cast<const uint4 *>(v + (tok + min(vt, L - 1)) * HD + i0 + vcb * 8);
        const size_t chunk = (size_t)chain * nc + c;
        const float *tb = table + chunk * kTableFloats, *vo = vecs + chunk * kVecFloats;
#pragma unroll
        for (int rt = 0; rt < 2; rt++)
#pragma unroll
            for (int ct = 0; ct < 2; ct++)
                wn[rt][ct] = *reinterpret_cast<const f32x4 *>(
                    (!grpX && tile_live(bi, rt, ct)) ? tb + (((bi * 2 + rt) * 2 + ct) * 64 + l) * 4 : vo + 4 * CW + 4);
        vn = vo[min(tid, 4 * CW + 3)];
    };
    auto land = [&](int c) {   // wait for the loads here; zero the rows beyond a short chunk
        const int L = min(C, s - c * C);
        if (st_t >= L) { sk = make_uint4(0, 0, 0, 0); sq = sk; }
        if (vt >= L) sv = make_uint4(0, 0, 0, 0);
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
    auto commit_v = [&](u16 *dst) {
        if (tid < 256) *reinterpret_cast<uint4 *>(dst + vt * LDB + vcb * 8) = sv;
    };
    auto commit_vecs = [&]() {
        if (tid < 4 * CW + 4) cvec[tid] = vn;
    };

    // fp32 master state (group Y), transposed strip:
    //   Mm[ct][r] = M[i = i0 + 16 ct + l%16][c = 16 bi + 4 (l/16) + r]
    // Group X has no state; it borrows the same registers as accumulators of M0 Q^T and S0 Q^T.
    f32x4 Mm[2], Sm[2];
    auto publish_state = [&](int slot) {   // -> HBM snapshot
#pragma unroll
        for (int ct = 0; ct < 2; ct++) {
            const size_t o = state0 + (size_t)slot * HD * HD + (i0 + 16 * ct + r16) * HD + 16 * bi + 4 * g;
            *reinterpret_cast<f32x4 *>(m_states + o) = Mm[ct];
            if (HAS_S) *reinterpret_cast<f32x4 *>(s_states + o) = Sm[ct];
        }
    };
    auto stage_state = [&]() {             // -> LDS operands of the next chunk
#pragma unroll
        for (int ct = 0; ct < 2; ct++) {
            const int off = (16 * ct + r16) * LDB + 16 * bi + 4 * g;
            split_store(Mh, Ml, off, Mm[ct]);
            if (HAS_S) split_store(Sh, Sl, off, Sm[ct]);
        }
    };

    fetch(0);
    if (!grpX) {
#pragma unroll
        for (int ct = 0; ct < 2; ct++) {
            const size_t o = (size_t)chain * HD * HD + (i0 + 16 * ct + r16) * HD + 16 * bi + 4 * g;
            Mm[ct] = *reinterpret_cast<const f32x4 *>(m_initial + o);
            Sm[ct] = HAS_S ? *reinterpret_cast<const f32x4 *>(s_initial + o) : zero4();
        }
        publish_state(0);
        stage_state();
    }
    land(0);
    commit_rows(Kr, sk);
    commit_rows(Qr0, sq);
    commit_kt(Kt0);
    commit_v(Kt1);
    commit_vecs();
    __syncthreads();

    for (int c = 0; c < nc; c++) {
        const int t0 = c * C, L = min(C, s - t0);
        const size_t tok = chain_tok + t0;
        // this chunk: Q in Qc, K^T in Kc, V in Kn (until K^T of the next chunk replaces it)
        u16 *Qc = (c & 1) ? Qr1 : Qr0, *Kc = (c & 1) ? Kt1 : Kt0;
        u16 *Qn = (c & 1) ? Qr0 : Qr1, *Kn = (c & 1) ? Kt0 : Kt1;
        fetch(min(c + 1, nc - 1));
        if (TRACK && !grpX) {   // sums of squares of this wave's part of the chunk-start states
            float msq = 0.f, ssq = 0.f;
#pragma unroll
            for (int ct = 0; ct < 2; ct++)
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    msq = fmaf(Mm[ct][e], Mm[ct][e], msq);
                    if (HAS_S) ssq = fmaf(Sm[ct][e], Sm[ct][e], ssq);
                }
            msq = wave_allreduce(msq);
            ssq = wave_allreduce(ssq);
            if (l == 0)
                *reinterpret_cast<float2 *>(tr.nrm + ((((size_t)chain * nc + c) * 2 + half) * 4 + bi) * 2) = make_float2(msq, ssq);
        }
        // ── first half: E^T, (E.wM)^T, (E.wS)^T (group X) and W.P (group Y) ──
        if (grpX) {
            // E[t][i]: rows t = 16 bi .., columns i = 16 ct ..
            const bf16x8 aK[2] = {ld_op(Kr, 16 * bi, 0), ld_op(Kr, 16 * bi, 1)};
            const bf16x8 aV = ld_op(Kn, 16 * bi, 0);
            const f32x4 wm = *reinterpret_cast<const f32x4 *>(cvec + 2 * CW + 16 * bi + 4 * g);
            const f32x4 wsv = *reinterpret_cast<const f32x4 *>(cvec + 3 * CW + 16 * bi + 4 * g);
            f32x4 esq = zero4();
#pragma unroll
            for (int ct = 0; ct < 2; ct++) {
                f32x4 e = zero4();
#pragma unroll
                for (int ks = 0; ks < 2; ks++) {
                    e = mfma32(aK[ks], ld_op(Mh, 16 * ct, ks), e);
                    e = mfma32(aK[ks], ld_op(Ml, 16 * ct, ks), e);
                }
                e = mfma32(aV, negI[ct], e);
                if (TRACK) esq += e * e;
                const int off = (16 * ct + r16) * LDB + 16 * bi + 4 * g;   // [i][t .. t+3]
                split_store(Eh, El, off, e);
                split_store(EMh, EMl, off, e * wm);
                if (HAS_S) split_store(ESh, ESl, off, e * wsv);
            }
            if (TRACK) {   // a lane holds tokens 16 bi + 4 g .. + 3 of rows 16 ct + l % 16: sum over the 16 lanes of the group
#pragma unroll
                for (int e = 0; e < 4; e++) esq[e] = group_allreduce<16>(esq[e]);
                if (r16 == 0)
                    *reinterpret_cast<f32x4 *>(tr.e2 + (((size_t)chain * 2 + half) * nc + c) * CW + 16 * bi + 4 * g) = esq;
            }
        } else {
            bf16x8 aK[2][2];
#pragma unroll
            for (int rt = 0; rt < 2; rt++)
#pragma unroll
                for (int ks = 0; ks < 2; ks++) aK[rt][ks] = ld_op(Kr, bm + 16 * rt, ks);
            f32x4 acc[2][2] = {{zero4(), zero4()}, {zero4(), zero4()}};
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
        __syncthreads();
        // ── second half: Y^T (group X) and the state update (group Y) ──
        f32x4 y2[2] = {zero4(), zero4()};   // group X: E^T (W.P)^T, then the finished Y^T; group Y: unused
        if (grpX) {
            // Y^T[i][t]: rows i = 16 rt .., columns t = 16 bi ..: a lane ends up with four consecutive
            // i of one token
            f32x4(&y0)[2] = Mm, (&y1)[2] = Sm;
            y0[0] = y0[1] = y1[0] = y1[1] = zero4();
#pragma unroll
            for (int ks = 0; ks < 2; ks++) {
                const bf16x8 bQ = ld_op(Qc, 16 * bi, ks), bWh = ld_op(WPh, 16 * bi, ks), bWl = ld_op(WPl, 16 * bi, ks);
#pragma unroll
                for (int rt = 0; rt < 2; rt++) {
                    const bf16x8 eh = ld_op(Eh, 16 * rt, ks);
                    y0[rt] = mfma32(ld_op(Mh, 16 * rt, ks), bQ, y0[rt]);
                    y0[rt] = mfma32(ld_op(Ml, 16 * rt, ks), bQ, y0[rt]);
                    y2[rt] = mfma32(eh, bWh, y2[rt]);
                    y2[rt] = mfma32(eh, bWl, y2[rt]);
                    y2[rt] = mfma32(ld_op(El, 16 * rt, ks), bWh, y2[rt]);
                    if (HAS_S) {
                        y1[rt] = mfma32(ld_op(Sh, 16 * rt, ks), bQ, y1[rt]);
                        y1[rt] = mfma32(ld_op(Sl, 16 * rt, ks), bQ, y1[rt]);
                    }
                }
            }
            const float at = cvec[16 * bi + r16], bt = cvec[CW + 16 * bi + r16];
#pragma unroll
            for (int rt = 0; rt < 2; rt++) y2[rt] += at * y0[rt] + bt * y1[rt];
        } else {
            // transposed state strip: rows c = 16 bi .., columns i = 16 ct ..
            f32x4 am[2] = {zero4(), zero4()}, as[2] = {zero4(), zero4()};
#pragma unroll
            for (int ks = 0; ks < 2; ks++) {
                const bf16x8 aKt = ld_op(Kc, 16 * bi, ks);
#pragma unroll
                for (int ct = 0; ct < 2; ct++) {
                    am[ct] = mfma32(aKt, ld_op(EMh, 16 * ct, ks), am[ct]);
                    am[ct] = mfma32(aKt, ld_op(EMl, 16 * ct, ks), am[ct]);
                    if (HAS_S) {
                        as[ct] = mfma32(aKt, ld_op(ESh, 16 * ct, ks), as[ct]);
                        as[ct] = mfma32(aKt, ld_op(ESl, 16 * ct, ks), as[ct]);
                    }
                }
            }
            const float aL = cvec[4 * CW], betaL = cvec[4 * CW + 1], hL = cvec[4 * CW + 2];
#pragma unroll
            for (int ct = 0; ct < 2; ct++) {
                Mm[ct] = aL * Mm[ct] + betaL * Sm[ct] + am[ct];
                if (HAS_S) Sm[ct] = hL * Sm[ct] + as[ct];
            }
        }
        // tokens of the next chunk land: K and V of this one are no longer read
        land(min(c + 1, nc - 1));
        commit_rows(Kr, sk);
        commit_rows(Qn, sq);
        commit_kt(Kn);
        // results of this chunk leave
        if (grpX) {
            const int t = 16 * bi + r16;
            if (t < L) {
#pragma unroll
                for (int rt = 0; rt < 2; rt++)
                    *reinterpret_cast<f32x4 *>(y + y_off + (size_t)(t0 + t) * yr.row_stride + i0 + 16 * rt + 4 * g) = y2[rt];
            }
        } else {
            publish_state(c + 1);
        }
        __syncthreads();
        if (!grpX) stage_state();
        commit_v(Kc);   // K^T of this chunk is no longer read
        commit_vecs();
        __syncthreads();
    }
}

constexpr size_t kChainFwdLds = (7 * BMAT + 10 * 32 * LDB) * sizeof(u16) + (4 * CW + 4) * sizeof(float);

template <bool HAS_S>
void launch_forward(const char *fn, const u16 *k, const u16 *v, const u16 *q, const float *alpha, const float *theta,
                    const float *eta, const float *m_initial, const float *s_initial, float *m_states,
                    float *s_states, float *y, int seq_len, int batch, int chunk_size, const HeadRows &yr,
                    const ChainTracks *tracks) {
    const ErrorScope es;
    const int nc = ceil_div(seq_len, chunk_size), nchunks = batch * nc;
    float *table = scratch(3, (size_t)nchunks * kTableFloats * sizeof(float));
    float *vecs = scratch(4, (size_t)nchunks * kVecFloats * sizeof(float));
    static bool attr_set = false;
    if (!attr_set) {
        check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(cw_chain_fwd_kernel<HAS_S, false>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)kChainFwdLds),
                  "dynamic LDS size");
        check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(cw_chain_fwd_kernel<HAS_S, true>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)kChainFwdLds),
                  "dynamic LDS size");
        attr_set = true;
    }
    if (es.failed()) return;
    {
        KernelTimer kt("cw_coef_kernel");
        hipLaunchKernelGGL(cw_coef_kernel<HAS_S>, dim3(ceil_div(nchunks, kCoefChunksPerWave)), dim3(64), 0, stream(), alpha, theta, eta,
                           table, vecs, seq_len, chunk_size, nc, nchunks);
    }
    check_launch("cw_coef_kernel");
    {
        KernelTimer kt("cw_chain_fwd_kernel");
        if (tracks)
            hipLaunchKernelGGL((cw_chain_fwd_kernel<HAS_S, true>), dim3(2 * batch), dim3(kChainThr), kChainFwdLds, stream(), k,
                               v, q, table, vecs, m_initial, s_initial, m_states, s_states, y, seq_len, chunk_size, nc, batch,
                               yr, *tracks);
        else
            hipLaunchKernelGGL((cw_chain_fwd_kernel<HAS_S, false>), dim3(2 * batch), dim3(kChainThr), kChainFwdLds, stream(), k,
                               v, q, table, vecs, m_initial, s_initial, m_states, s_states, y, seq_len, chunk_size, nc, batch,
                               yr, ChainTracks{nullptr, nullptr});
    }
    check_launch(fn);
}

}  // namespace

bool chunkwise_chain_forward_bf16(const char *fn, const uint16_t *k, const uint16_t *v, const uint16_t *q,
                                  const float *alpha, const float *theta, const float *eta, const float *m_initial,
                                  const float *s_initial, float *m_states, float *s_states, float *y, int seq_len,
                                  int d, int batch, int chunk_size, bool has_s, const HeadRows *y_rows,
                                  const ChainTracks *tracks) {
    if (d != HD || chunk_size < 1 || chunk_size > CW || seq_len <= 0 || batch <= 0) return false;
    const HeadRows yr = y_rows ? *y_rows : head_major_rows(seq_len, HD);
    if (has_s)
        launch_forward<true>(fn, k, v, q, alpha, theta, eta, m_initial, s_initial, m_states, s_states, y, seq_len,
                             batch, chunk_size, yr, tracks);
    else
        launch_forward<false>(fn, k, v, q, alpha, theta, nullptr, m_initial, nullptr, m_states, nullptr, y, seq_len,
                              batch, chunk_size, yr, tracks);
    return true;
}

}  // namespace nlh
