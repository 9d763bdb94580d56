// Backward of the frozen-M0 chunkwise Titans / Delta rule on bf16 tokens: the adjoint scan.
//
// dMo, dSo are the adjoints of a chunk's end state; walking the chunks of a chain backwards,
//   dE  = (W.P)^T dY + wM.(K dMo^T) + wS.(K dSo^T)          [token j][row i]
//   dM0 = a_L dMo + (a.dY)^T Q + dE^T K
//   dS0 = beta_L dMo + h_L dSo + (beta.dY)^T Q
// with P = Q K^T, W[t][j] = -theta_j c[t][j], wM_j = -theta_j c[L-1][j], wS_j = -theta_j bb[j][L-1]
// (the adjoint of the chunk map of chunkwise_mm.hip, written without its 64x64 transfer
// matrices).  The rows of dM, dS never mix, so a chain is split over two workgroups of 32 rows
// each; each walks all chunks with its rows of dM and dS in registers (fp32) and, as bf16
// hi + lo pairs, in LDS as operands of the next step.  HBM sees k, q, dY and the coefficient
// table once per step and receives one adjoint snapshot per chunk, in bf16: dm_snap[chain][c] is the
// adjoint of the state at the start of chunk c (slot num_chunks = 0), rounded as the gradient pass
// would round it; slot 0, the gradient of the initial state, leaves in fp32 (dm_first).
//
// Every fp32 operand enters the bf16 matrix cores as a hi + lo pair: this path is recurrent.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "bf16_tiles.h"
#include "chunkwise_grads.h"
#include "runtime.h"

namespace nlh {
namespace {

constexpr int HMAT = 32 * LDB;   // elements of a 32-row bf16 matrix
constexpr int DYS = 48;          // row stride of a [token][32 rows] bf16 matrix (read through ld_op_tr)
constexpr int DYM = 64 * DYS;
constexpr int kLate = 2 * BMAT + 6 * DYM;   // elements of one copy of a chunk's staged inputs
constexpr int kCvec = 5 * CW + 8;

template <bool HAS_S>
__global__ __launch_bounds__(kTileThr) void cw_adjoint_chain_kernel(
    const u16 *__restrict__ k, const u16 *__restrict__ q, const float *__restrict__ d_y,
    const float *__restrict__ tab_b, const float *__restrict__ vecs, u16 *__restrict__ dm_snap,
    u16 *__restrict__ ds_snap, float *__restrict__ dm_first, float *__restrict__ ds_first, int s, int C, int nc, int batch, int tab_floats, int vec_floats, HeadRows dyr) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    u16 *WPh = reinterpret_cast<u16 *>(smem_raw), *WPl = WPh + BMAT;   // (W.P)^T [j][t]
    u16 *dMh = WPl + BMAT, *dMl = dMh + HMAT;                          // dMo [i][c]
    u16 *dSh = dMl + HMAT, *dSl = dSh + HMAT;                          // dSo [i][c]
    u16 *dEh = dSl + HMAT, *dEl = dEh + HMAT;                          // dE^T [i][j]
    // The staged inputs of a chunk exist twice, so that the next step's copy is written while this step's is
    // still in use: K [j][c], Q [t][c], dY, a.dY, beta.dY hi / lo [t][i] (this workgroup's 32 rows i), and the
    // vectors a, beta, cl, bl, theta [64] each, .., h_L
    u16 *late = dEl + HMAT;
    float *cvecs = reinterpret_cast<float *>(late + 2 * kLate);
    const int tid = threadIdx.x, w = tid >> 6, l = tid & 63, g = l >> 4, r16 = l & 15;
    int chain, half;
    chain_half_of_block(batch, chain, half);
    const int i0 = 32 * half;
    const size_t chain_tok = (size_t)chain * s, state0 = (size_t)chain * (nc + 1) * HD * HD;
    const size_t dy_off = dyr.offset(chain);
    const int st_t = 16 * (w & 3) + (l & 15), st_cb = 4 * (w >> 2) + (l >> 4);   // bf16 tile: row, 8-element block
    const int yt = tid >> 3, yg = tid & 7;                                        // dY tile: row t, 4-element block

    // zero what is never written again: tiles of (W.P)^T above the diagonal
    for (int e = tid; e < BMAT / 2; e += kTileThr) {
        reinterpret_cast<unsigned *>(WPh)[e] = 0u;
        reinterpret_cast<unsigned *>(WPl)[e] = 0u;
    }

    // registers of the next step (chunk c - 1)
    uint4 nK, nQ;
    f32x4 ndY;
    float na = 0.f, nb = 0.f, nvec = 0.f;
    const int tt = w >> 1, jt0 = 2 * (w & 1);   // phase A: P tiles (tt, jt0) and (tt, jt0 + 1)
    auto fetch = [&](int c) {
        const int L = min(C, s - c * C);
        const size_t tok = chain_tok + (size_t)c * C;
        const size_t row = tok + min(st_t, L - 1);
        nK = *reinterpret_cast<const uint4 *>(k + row * HD + st_cb * 8);
        nQ = *reinterpret_cast<const uint4 *>(q + row * HD + st_cb * 8);
        ndY = *reinterpret_cast<const f32x4 *>(d_y + dy_off + (size_t)(c * C + min(yt, L - 1)) * dyr.row_stride + i0 +
                                               yg * 4);
        const size_t chunk = (size_t)chain * nc + c;
        const float *vo = vecs + chunk * vec_floats;
        na = vo[yt];
        nb = vo[CW + yt];
        nvec = vo[min(tid, 5 * CW + 7)];
    };
    // The coefficient tiles are used by the first phase of a step only; the next step's are requested right
    // after that use, into the same registers (a value that had to outlive the next request would be copied at
    // the bottom of the loop, behind a wait for that request).
    f32x4 ctab[2];
    auto fetch_tab = [&](int c) {
        const size_t chunk = (size_t)chain * nc + c;
        const float *vo = vecs + chunk * vec_floats, *tb = tab_b + chunk * tab_floats;
#pragma unroll
        for (int x = 0; x < 2; x++) {
            const int jt = jt0 + x, bi = 2 * (tt >> 1) + (jt >> 1);
            ctab[x] = *reinterpret_cast<const f32x4 *>(
                jt <= tt ? tb + (((bi * 2 + (tt & 1)) * 2 + (jt & 1)) * 64 + l) * 4 : vo + 5 * CW);
        }
    };
    // Registers -> LDS, everything in the order it arrives (rows = tokens): the products that contract over
    // tokens read their operands through ld_op_tr.  Called during the step before, into the copy that step
    // does not use.
    auto commit = [&](int c, int par) {
        const int L = min(C, s - c * C);
        u16 *Kr = late + par * kLate, *Qr = Kr + BMAT;
        u16 *dYh = Qr + BMAT, *dYl = dYh + DYM, *dYah = dYl + DYM, *dYal = dYah + DYM, *dYbh = dYal + DYM, *dYbl = dYbh + DYM;
        if (st_t >= L) { nK = make_uint4(0, 0, 0, 0); nQ = nK; }
        if (yt >= L) ndY = zero4();
        *reinterpret_cast<uint4 *>(Kr + st_t * LDB + st_cb * 8) = nK;
        *reinterpret_cast<uint4 *>(Qr + st_t * LDB + st_cb * 8) = nQ;
        const int off = yt * DYS + yg * 4;
        split_store(dYh, dYl, off, ndY);
        split_store(dYah, dYal, off, na * ndY);
        if (HAS_S) split_store(dYbh, dYbl, off, nb * ndY);
        if (tid < kCvec) cvecs[par * kCvec + tid] = nvec;
    };

    // fp32 master: transposed tile rows c = 16 (w/2) + 4 (l/16) + r, column i = 16 (w%2) + l%16
    const int rt = w >> 1, ct = w & 1;
    f32x4 dM = zero4(), dS = zero4();
    // The snapshot a later pass reads is the bf16 value that this scan itself uses as the hi operand: it leaves
    // from the LDS copy at the top of the next step, as whole 128-byte rows (from the accumulator layout a wave
    // would store 32-byte pieces of 16 different lines).  The gradient of the initial state (slot 0) leaves in fp32.
    auto publish = [&](int slot) {
        const int e = (i0 + 16 * ct + r16) * HD + 16 * rt + 4 * g, off = (16 * ct + r16) * LDB + 16 * rt + 4 * g;
        split_store(dMh, dMl, off, dM);
        if (HAS_S) split_store(dSh, dSl, off, dS);
        if (slot == 0) {
            *reinterpret_cast<f32x4 *>(dm_first + (size_t)chain * HD * HD + e) = dM;
            if (HAS_S) *reinterpret_cast<f32x4 *>(ds_first + (size_t)chain * HD * HD + e) = dS;
        }
    };
    auto store_snapshot = [&](int slot) {   // threads 0..255: a row piece of dMo, 256..511: of dSo
        const int which = tid >> 8, row = (tid & 255) >> 3, c8 = (tid & 7) * 8;
        if (which && !HAS_S) return;
        const uint4 x = *reinterpret_cast<const uint4 *>((which ? dSh : dMh) + row * LDB + c8);
        *reinterpret_cast<uint4 *>((which ? ds_snap : dm_snap) + state0 + (size_t)slot * HD * HD + (i0 + row) * HD + c8) = x;
    };

    // (W.P)^T of chunk c from its staged K, Q (copy par): this wave's two tiles of P[t][j].  It does not depend
    // on the scan, so it is computed a step ahead, in the shadow of the step's last phase.
    auto weights = [&](int par) {
        const float *cvec = cvecs + par * kCvec;
        const u16 *Kr = late + par * kLate, *Qr = Kr + BMAT;
        const bf16x8 aq[2] = {ld_op(Qr, 16 * tt, 0), ld_op(Qr, 16 * tt, 1)};
#pragma unroll
        for (int x = 0; x < 2; x++) {
            const int jt = jt0 + x;
            if (jt <= tt) {
                f32x4 p = zero4();
#pragma unroll
                for (int ks = 0; ks < 2; ks++) p = mfma32(aq[ks], ld_op(Kr, 16 * jt, ks), p);
                const float nth = -cvec[4 * CW + 16 * jt + r16];
                split_store(WPh, WPl, (16 * jt + r16) * LDB + 16 * tt + 4 * g, nth * ctab[x] * p);   // [j][t .. t+3]
            }
        }
    };

    // Two barriers per step.  First phase: the next chunk's inputs go to LDS (requested a step earlier), the ones
    // after that are requested, dE.  Second phase: dM0, dS0, the next chunk's (W.P)^T, the new state to LDS.
    fetch(nc - 1);
    fetch_tab(nc - 1);
    publish(nc);
    commit(nc - 1, (nc - 1) & 1);
    fetch(max(nc - 2, 0));
    __syncthreads();
    weights((nc - 1) & 1);
    fetch_tab(max(nc - 2, 0));
    __syncthreads();
    for (int c = nc - 1; c >= 0; c--) {
        const int L = min(C, s - c * C), par = c & 1;
        const float *cvec = cvecs + par * kCvec;
        const u16 *Kr = late + par * kLate, *Qr = Kr + BMAT;
        const u16 *dYh = Qr + BMAT, *dYl = dYh + DYM, *dYah = dYl + DYM, *dYal = dYah + DYM, *dYbh = dYal + DYM, *dYbl = dYbh + DYM;
        store_snapshot(c + 1);
        commit(max(c - 1, 0), par ^ 1);
        fetch(max(c - 2, 0));
        // ── dE[j][i]: tile rows j = 16 rt.., columns i = 16 ct.. ──
        {
            f32x4 e1 = zero4(), e2 = zero4(), e3 = zero4();
#pragma unroll
            for (int ks = 0; ks < 2; ks++) {
                const bf16x8 wh = ld_op(WPh, 16 * rt, ks), wl = ld_op(WPl, 16 * rt, ks), ak = ld_op(Kr, 16 * rt, ks);
                const bf16x8 yh = ld_op_tr<DYS>(dYh, 16 * ct, ks), yl = ld_op_tr<DYS>(dYl, 16 * ct, ks);
                e1 = mfma32(wh, yh, e1);
                e1 = mfma32(wl, yh, e1);
                e1 = mfma32(wh, yl, e1);
                e2 = mfma32(ak, ld_op(dMh, 16 * ct, ks), e2);
                e2 = mfma32(ak, ld_op(dMl, 16 * ct, ks), e2);
                if (HAS_S) {
                    e3 = mfma32(ak, ld_op(dSh, 16 * ct, ks), e3);
                    e3 = mfma32(ak, ld_op(dSl, 16 * ct, ks), e3);
                }
            }
            const int j4 = 16 * rt + 4 * g;
            const f32x4 th = *reinterpret_cast<const f32x4 *>(cvec + 4 * CW + j4);
            const f32x4 cl = *reinterpret_cast<const f32x4 *>(cvec + 2 * CW + j4);
            const f32x4 bl = *reinterpret_cast<const f32x4 *>(cvec + 3 * CW + j4);
            split_store(dEh, dEl, (16 * ct + r16) * LDB + j4, e1 - th * (cl * e2 + bl * e3));   // [i][j .. j+3]
        }
        __syncthreads();
        // ── dM0^T, dS0^T: tile rows c = 16 rt.., columns i = 16 ct.. ──
        {
            f32x4 am = zero4(), as = zero4();
#pragma unroll
            for (int ks = 0; ks < 2; ks++) {
                const bf16x8 aq = ld_op_tr<LDB>(Qr, 16 * rt, ks), ak = ld_op_tr<LDB>(Kr, 16 * rt, ks);   // Q^T, K^T
                am = mfma32(aq, ld_op_tr<DYS>(dYah, 16 * ct, ks), am);
                am = mfma32(aq, ld_op_tr<DYS>(dYal, 16 * ct, ks), am);
                am = mfma32(ak, ld_op(dEh, 16 * ct, ks), am);
                am = mfma32(ak, ld_op(dEl, 16 * ct, ks), am);
                if (HAS_S) {
                    as = mfma32(aq, ld_op_tr<DYS>(dYbh, 16 * ct, ks), as);
                    as = mfma32(aq, ld_op_tr<DYS>(dYbl, 16 * ct, ks), as);
                }
            }
            const float aL = cvec[L - 1], betaL = cvec[CW + L - 1], hL = cvec[5 * CW + 4];
            const f32x4 dMn = aL * dM + am;
            if (HAS_S) dS = betaL * dM + hL * dS + as;
            dM = dMn;
        }
        publish(c);
        // (W.P)^T of the next step's chunk (staged during this step's first phase), then the tiles after it
        weights(par ^ 1);
        fetch_tab(max(c - 2, 0));
        __syncthreads();
    }
}

constexpr size_t kAdjointLds = (2 * BMAT + 6 * HMAT + 2 * kLate) * sizeof(u16) + 2 * kCvec * sizeof(float);

}  // namespace

bool chunkwise_adjoint_bf16(const uint16_t *k, const uint16_t *q, const float *d_y, const float *tab_b,
                            const float *vecs, uint16_t *dm_snap, uint16_t *ds_snap, float *dm_first,
                            float *ds_first, int seq_len, int batch, int chunk_size, bool has_s,
                            const HeadRows *dy_rows) {
    const ErrorScope es;
    const int nc = ceil_div(seq_len, chunk_size);
    const HeadRows dyr = dy_rows ? *dy_rows : head_major_rows(seq_len, HD);
    static bool attr_set = false;
    if (!attr_set) {
        check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(cw_adjoint_chain_kernel<true>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)kAdjointLds), "dynamic LDS size");
        check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(cw_adjoint_chain_kernel<false>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)kAdjointLds), "dynamic LDS size");
        attr_set = true;
    }
    if (es.failed()) return true;
    const int tabf = (int)chunkwise_grads_table_floats(), vecf = (int)chunkwise_grads_vec_floats();
    KernelTimer kt("cw_adjoint_chain_kernel");
    if (has_s)
        hipLaunchKernelGGL(cw_adjoint_chain_kernel<true>, dim3(2 * batch), dim3(kTileThr), kAdjointLds, stream(), k, q,
                           d_y, tab_b, vecs, dm_snap, ds_snap, dm_first, ds_first, seq_len, chunk_size, nc, batch, tabf,
                           vecf, dyr);
    else
        hipLaunchKernelGGL(cw_adjoint_chain_kernel<false>, dim3(2 * batch), dim3(kTileThr), kAdjointLds, stream(), k, q,
                           d_y, tab_b, vecs, dm_snap, nullptr, dm_first, nullptr, seq_len, chunk_size, nc, batch, tabf,
                           vecf, dyr);
    check_launch("cw_adjoint_chain_kernel");
    return true;
}

}  // namespace nlh
