// Fused checkpointed backward of the exact memory rules (Titans LMM / Delta).
//
// One launch walks all C-token segments of every chain in reverse.  The state
// trajectory a reverse sweep needs is never written to device memory:
//
//   level 1  from the segment's checkpoint, replay the forward once; park the
//            state every SUB tokens in LDS ("sub-checkpoints") and every
//            token's error e_t = M_t k_t - v_t (one float per row) in LDS.
//   level 2  for each SUB-token block, last to first: reload its sub-checkpoint,
//            replay SUB tokens keeping all SUB+1 states in registers, then run
//            the reverse recurrence over those registers.
//
// With C = 64 and SUB = 8 a workgroup holds 8 sub-checkpoints (64 KB of LDS) and
// 9 states in VGPRs; the forward is recomputed twice, which is cheaper than
// 32 KB of state traffic per token per chain.
//
// Work split is the row split of the other memory-rule kernels with one row per
// lane (a 16-row slab of a 64x64 chain per workgroup): rows are independent
// recurrences, d_M/d_S stay in registers across segments, and only the column
// sums d_q/d_k and the gate gradients are combined across waves (LDS) and
// across the workgroups of a chain (partial buffers + finalize kernel).
//
// Error clipping and M-norm projection couple the rows; those cases take the
// replay-through-memory schedule instead.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "../../include/nl_hecate_ffi.h"
#include "chunkwise_guard.h"
#include "rule_common.h"

namespace nlh {

constexpr int SUB = 8;        // tokens per register-resident block
constexpr int NSUB_MAX = 8;   // sub-checkpoints held in LDS
constexpr int C_MAX = SUB * NSUB_MAX;

struct FusedArgs {
    const float *k, *v, *q, *alpha, *theta, *eta, *m_ckpt, *s_ckpt, *d_y;
    float *d_k, *d_v, *d_q, *d_alpha, *d_theta, *d_eta;
    float *ws_dq, *ws_dk, *ws_gate;   // partial sums when parts > 1
    float *d_m_out, *d_s_out;         // [B, dd]
    int seq_len, C, n_ckpt, parts, batch;
    float *msq_part;   // may be null: [batch * parts] upper bounds of max_t sum(M_t^2) over the replayed states (FwdArgs)
};

// FROZEN: frozen-M0 chunkwise rule, segment = chunk
// (core/kernels/titans_chunkwise_backward.cu:118-358).
// TRACK: keep the bound of max_t |M_t|_F^2 over the replayed states (FusedArgs::msq_part)
template <int D, bool HAS_S, bool FROZEN, bool TRACK>
__global__ __launch_bounds__(kThreads) void rule_bwd_fused_kernel(FusedArgs a) {
    constexpr int LPR = D / 4;
    constexpr int RG = 64 / LPR;
    constexpr int ROWS_WG = kWaves * RG;
    constexpr int DD = D * D;
    constexpr bool ALL_VALID = (D % ROWS_WG) == 0;  // every lane owns a real row

    __shared__ __align__(16) float4 subck[NSUB_MAX][HAS_S ? 2 : 1][kThreads];
    __shared__ float ebuf[C_MAX * ROWS_WG];
    __shared__ __align__(16) float tA[2][SUB * D];   // k
    __shared__ __align__(16) float tB[2][SUB * D];   // v (level 1) or q (level 2)
    __shared__ __align__(16) float tC[2][SUB * D];   // dY (level 2)
    __shared__ float tg[2][3 * SUB];
    __shared__ __align__(16) float sdq[2][SUB * kWaves * D];
    __shared__ __align__(16) float sdk[2][SUB * kWaves * D];
    __shared__ float sdv[2][SUB * ROWS_WG];
    constexpr int NG = HAS_S ? 3 : 2;  // gate gradients per token: alpha, theta(, eta)
    __shared__ float sgate[2][kWaves * NG * SUB];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int cb = lane % LPR, g = lane / LPR;
    const int g16 = lane >> 4;  // DPP row of the lane
    int chain, part;
    map_block(a.parts, chain, part);
    const int row_local = wave * RG + g;
    const int row = part * ROWS_WG + row_local;
    const bool valid = ALL_VALID || row < D;
    const int rr = valid ? row : 0;
    const size_t roff = (size_t)rr * D + cb * 4;
    const int seq_len = a.seq_len, C = a.C;

    const size_t tok = (size_t)chain * seq_len;
    const float *kb = a.k + tok * D, *vb = a.v + tok * D, *qb = a.q + tok * D;
    const float *dyb = a.d_y + tok * D;
    const float *ab = a.alpha + tok, *thb = a.theta + tok;
    const float *eb = HAS_S ? a.eta + tok : nullptr;
    const float *mck = a.m_ckpt + (size_t)chain * a.n_ckpt * DD;
    const float *sck = HAS_S ? a.s_ckpt + (size_t)chain * a.n_ckpt * DD : nullptr;

    float4 dM = f4_zero(), dS = f4_zero();
    float4 M = f4_zero(), S = f4_zero();
    float4 M0f = f4_zero(), dM0 = f4_zero();  // FROZEN: chunk-start M and its gradient
    float nmax = 0.f;

    // ── work items: (segment, phase, block) in processing order ──
    const int nseg = (seq_len + C - 1) / C;
    auto seg_t0 = [&](int sg) { return sg * C; };
    auto seg_t1 = [&](int sg) { return min(sg * C + C, seq_len); };
    auto seg_nsub = [&](int sg) { return (seg_t1(sg) - seg_t0(sg) + SUB - 1) / SUB; };

    TileRegs<D, SUB> rA, rB, rC;
    GateRegs<SUB> rG;
    auto load_item = [&](int sg, int phase, int j) {
        const int t0 = seg_t0(sg) + j * SUB, lo = seg_t0(sg), hi = seg_t1(sg);
        rA.load(kb, t0, lo, hi, tid);
        if (phase == 0) {
            rB.load(vb, t0, lo, hi, tid);
        } else {
            rB.load(qb, t0, lo, hi, tid);
            rC.load(dyb, t0, lo, hi, tid);
        }
        rG.load(ab, thb, eb, t0, lo, hi, tid);
    };

    // Pending output flush: the block of tokens [ft0, ft1) sits in out buffer fob.
    int ft0 = 0, ft1 = 0, fob = 0;
    auto flush = [&]() {
        if (ft1 <= ft0) return;
        const size_t pbase = ((size_t)part * a.batch + chain) * seq_len;
        for (int idx = tid; idx < SUB * D; idx += kThreads) {
            int tt = idx / D, col = idx % D, t = ft0 + tt;
            if (t >= ft1) continue;
            float sq_ = 0.f, sk_ = 0.f;
#pragma unroll
            for (int w = 0; w < kWaves; w++) {
                sq_ += sdq[fob][(tt * kWaves + w) * D + col];
                sk_ += sdk[fob][(tt * kWaves + w) * D + col];
            }
            if (a.parts == 1) {
                a.d_q[(tok + t) * D + col] = sq_;
                a.d_k[(tok + t) * D + col] = sk_;
            } else {
                a.ws_dq[(pbase + t) * D + col] = sq_;
                a.ws_dk[(pbase + t) * D + col] = sk_;
            }
        }
        for (int idx = tid; idx < SUB * ROWS_WG; idx += kThreads) {
            int tt = idx / ROWS_WG, r = idx % ROWS_WG, t = ft0 + tt;
            int orow = part * ROWS_WG + r;
            if (t < ft1 && orow < D) a.d_v[(tok + t) * D + orow] = sdv[fob][idx];
        }
        if (tid < SUB && ft0 + tid < ft1) {
            float ga = 0.f, ge = 0.f, gt = 0.f;
#pragma unroll
            for (int w = 0; w < kWaves; w++) {
                ga += sgate[fob][w * (NG * SUB) + tid * NG + 0];
                gt += sgate[fob][w * (NG * SUB) + tid * NG + 1];
                if (HAS_S) ge += sgate[fob][w * (NG * SUB) + tid * NG + 2];
            }
            const int t = ft0 + tid;
            if (a.parts == 1) {
                a.d_alpha[tok + t] = -ga;
                if (HAS_S) a.d_eta[tok + t] = ge;
                a.d_theta[tok + t] = -gt;
            } else {
                float *wg = a.ws_gate + (pbase + t) * 4;
                wg[0] = -ga; wg[1] = ge; wg[2] = -gt;
            }
        }
        ft1 = ft0;  // done
    };

    int sg = nseg - 1, phase = 0, j = 0;
    bool have = nseg > 0;
    if (have) load_item(sg, phase, j);
    int it = 0, ob = 0;
    while (have) {
        const int buf = it & 1;
        rA.store_lds(tA[buf], tid);
        rB.store_lds(tB[buf], tid);
        if (phase == 1) rC.store_lds(tC[buf], tid);
        rG.store_lds(tg[buf], tid);
        __syncthreads();
        flush();
        // next item
        int nsg = sg, nphase = phase, nj = j;
        bool nhave = true;
        if (phase == 0) {
            if (j + 1 < seg_nsub(sg)) nj = j + 1;
            else { nphase = 1; nj = seg_nsub(sg) - 1; }
        } else {
            if (j > 0) nj = j - 1;
            else if (sg > 0) { nsg = sg - 1; nphase = 0; nj = 0; }
            else nhave = false;
        }
        if (nhave) load_item(nsg, nphase, nj);

        const int t0s = seg_t0(sg), t1 = seg_t1(sg);
        const int tb0 = t0s + j * SUB;
        // FULL blocks (all SUB tokens inside the segment) run as straight-line
        // code: no per-token branch, so LDS reads and the independent parts of
        // neighbouring tokens overlap the dependent chain.
        auto level1 = [&](auto full_c) {
            constexpr bool FULL = decltype(full_c)::value;
#pragma unroll
            for (int i = 0; i < SUB; i++) {
                const int t = tb0 + i;
                if (!FULL && t >= t1) break;
                const float4 kk = *reinterpret_cast<const float4 *>(&tA[buf][i * D + cb * 4]);
                const float vv = tB[buf][i * D + rr];
                const float al = tg[buf][i], th = tg[buf][SUB + i], et = tg[buf][2 * SUB + i];
                float p = group_allreduce<LPR>(dot4(FROZEN ? M0f : M, kk));
                float e = valid ? p - vv : 0.f;
                ebuf[(t - t0s) * ROWS_WG + row_local] = e;  // same value from all lanes of the row
                const float te = th * e;
                if (HAS_S) {
                    S = f4_axpby(et, S, -te, kk);
                    M = f4_axpby(1.f - al, M, 1.f, S);
                } else {
                    M = f4_axpby(1.f - al, M, -te, kk);
                }
                if (TRACK) nmax = fmaxf(nmax, dot4(M, M));
            }
        };
        auto level2 = [&](auto full_c) {
            constexpr bool FULL = decltype(full_c)::value;
            float4 Mtr[SUB + 1], Str[SUB];
            float ev[SUB];
            float gsum[NG * SUB];  // per-lane gate-gradient partials, [token][component]
#pragma unroll
            for (int i = 0; i < NG * SUB; i++) gsum[i] = 0.f;
#pragma unroll
            for (int i = 0; i < SUB; i++) {
                const int t = tb0 + i;
                Mtr[i] = M;
                Str[i] = S;
                ev[i] = 0.f;
                if (FULL || t < t1) {
                    const float4 kk = *reinterpret_cast<const float4 *>(&tA[buf][i * D + cb * 4]);
                    const float al = tg[buf][i], th = tg[buf][SUB + i], et = tg[buf][2 * SUB + i];
                    const float e = ebuf[(t - t0s) * ROWS_WG + row_local];
                    ev[i] = e;
                    const float te = th * e;
                    if (HAS_S) {
                        S = f4_axpby(et, S, -te, kk);
                        M = f4_axpby(1.f - al, M, 1.f, S);
                    } else {
                        M = f4_axpby(1.f - al, M, -te, kk);
                    }
                }
            }
            Mtr[SUB] = M;
#pragma unroll
            for (int i = SUB - 1; i >= 0; i--) {
                const int t = tb0 + i;
                if (FULL || t < t1) {
                    const float4 kk = *reinterpret_cast<const float4 *>(&tA[buf][i * D + cb * 4]);
                    const float4 qq = *reinterpret_cast<const float4 *>(&tB[buf][i * D + cb * 4]);
                    const float dy = valid ? tC[buf][i * D + rr] : 0.f;
                    const float al = tg[buf][i], th = tg[buf][SUB + i], et = tg[buf][2 * SUB + i];
                    const float4 Mt = Mtr[i], Mn = Mtr[i + 1];
                    const float e = ev[i];
                    f4_fma(dM, dy, qq);
                    float4 cq = f4_scale(dy, Mn);
                    if (HAS_S) f4_add(dS, dM);
                    float4 &G = HAS_S ? dS : dM;
                    float pa = dot4(Mt, dM);
                    float pe = HAS_S ? dot4(Str[i], dS) : 0.f;
                    const float gk = group_allreduce<LPR>(dot4(G, kk));
                    const float derr = -th * gk;
                    float pt = (cb == 0) ? e * gk : 0.f;
                    sdv[ob][i * ROWS_WG + row_local] = -derr;  // same value from all lanes of the row
                    float4 ck = f4_scale(-th * e, G);
                    f4_fma(ck, derr, FROZEN ? M0f : Mt);
                    if (HAS_S) dS = f4_scale(et, dS);
                    if (FROZEN) {
                        dM = f4_scale(1.f - al, dM);
                        f4_fma(dM0, derr, kk);
                    } else {
                        dM = f4_axpby(1.f - al, dM, derr, kk);
                    }
                    // column sums over the row groups of the wave
                    if constexpr (D == 64) {
                        // reduce-scatter: lane (g, cb) ends with column 4*cb + g
                        float fq, fk;
                        colreduce4x2(cq, ck, fq, fk);
                        sdq[ob][(i * kWaves + wave) * D + cb * 4 + g] = fq;
                        sdk[ob][(i * kWaves + wave) * D + cb * 4 + g] = fk;
                    } else {
                        cq.x = stride_allreduce<LPR>(cq.x); cq.y = stride_allreduce<LPR>(cq.y);
                        cq.z = stride_allreduce<LPR>(cq.z); cq.w = stride_allreduce<LPR>(cq.w);
                        ck.x = stride_allreduce<LPR>(ck.x); ck.y = stride_allreduce<LPR>(ck.y);
                        ck.z = stride_allreduce<LPR>(ck.z); ck.w = stride_allreduce<LPR>(ck.w);
                        if (g == 0) {
                            *reinterpret_cast<float4 *>(&sdq[ob][(i * kWaves + wave) * D + cb * 4]) = cq;
                            *reinterpret_cast<float4 *>(&sdk[ob][(i * kWaves + wave) * D + cb * 4]) = ck;
                        }
                    }
                    gsum[i * NG + 0] = pa;
                    gsum[i * NG + 1] = pt;
                    if (HAS_S) gsum[i * NG + 2] = pe;
                }
            }
            // one batched wave reduction for the block's gate gradients
            float gtot[NG * SUB / 4];
            wave_reduce_scatter<NG * SUB>(gsum, gtot);
#pragma unroll
            for (int n = 0; n < NG * SUB / 4; n++)  // same value from the 16 lanes of a DPP row
                sgate[ob][wave * (NG * SUB) + 4 * n + 2 * (g16 & 1) + (g16 >> 1)] = gtot[n];
        };
        const bool full = tb0 + SUB <= t1;
        if (phase == 0) {
            // ── level 1: forward replay, park sub-checkpoint and errors ──
            if (j == 0) {
                M = S = f4_zero();
                if (valid) {
                    M = *reinterpret_cast<const float4 *>(mck + (size_t)sg * DD + roff);
                    if (HAS_S) S = *reinterpret_cast<const float4 *>(sck + (size_t)sg * DD + roff);
                }
                if (FROZEN) M0f = M;
            }
            subck[j][0][tid] = M;
            if (HAS_S) subck[j][HAS_S ? 1 : 0][tid] = S;
            if (full) level1(std::true_type{});
            else level1(std::false_type{});
        } else {
            // ── level 2: replay the block into registers, then reverse it ──
            M = subck[j][0][tid];
            if (HAS_S) S = subck[j][HAS_S ? 1 : 0][tid];
            if (full) level2(std::true_type{});
            else level2(std::false_type{});
            if (FROZEN && j == 0) {  // chunk start: the error path joins d_M
                f4_add(dM, dM0);
                dM0 = f4_zero();
            }
            ft0 = tb0;
            ft1 = min(tb0 + SUB, t1);
            fob = ob;
            ob ^= 1;
        }
        sg = nsg; phase = nphase; j = nj; have = nhave;
        it++;
    }
    __syncthreads();
    flush();
    if (valid) {
        *reinterpret_cast<float4 *>(a.d_m_out + (size_t)chain * DD + roff) = dM;
        if (HAS_S) *reinterpret_cast<float4 *>(a.d_s_out + (size_t)chain * DD + roff) = dS;
    }
    if (TRACK) {
        __syncthreads();   // the flush above was the last reader of the staging buffers
        const float tot = block_allreduce(nmax, tg[0], tid);
        if (tid == 0) a.msq_part[chain * a.parts + part] = tot;
    }
}

template <int D, bool HAS_S, bool FROZEN>
static void launch_fused_d(const FusedArgs &a) {
    KernelTimer kt("rule_bwd_fused_kernel");
    if (a.msq_part)
        hipLaunchKernelGGL((rule_bwd_fused_kernel<D, HAS_S, FROZEN, true>), dim3(a.batch * a.parts), dim3(kThreads), 0, stream(), a);
    else
        hipLaunchKernelGGL((rule_bwd_fused_kernel<D, HAS_S, FROZEN, false>), dim3(a.batch * a.parts), dim3(kThreads), 0, stream(), a);
    check_launch("rule_bwd_fused_kernel");
}

template <bool HAS_S, bool FROZEN>
static bool backward_ckpt_fused_t(const float *k, const float *v, const float *q,
                                  const float *alpha, const float *theta, const float *eta,
                                  const float *m_ckpt, const float *s_ckpt, const float *d_y,
                                  float *d_k, float *d_v, float *d_q,
                                  float *d_alpha, float *d_theta, float *d_eta,
                                  float *d_m_initial, float *d_s_initial,
                                  int seq_len, int d, int batch, int C, float m_norm_guard) {
    const ErrorScope es;
    if (C > C_MAX) return false;
    if (d != 8 && d != 16 && d != 32 && d != 64 && d != 128) return false;
    const size_t dd = (size_t)d * d;
    const int rows_wg = kWaves * (64 / (d / 4));
    FusedArgs a{k, v, q, alpha, theta, eta, m_ckpt, s_ckpt, d_y, d_k, d_v, d_q, d_alpha, d_theta, d_eta,
                nullptr, nullptr, nullptr, nullptr, nullptr,
                seq_len, C, n_ckpt_count(seq_len, C), ceil_div(d, rows_wg), batch, nullptr};
    if (m_norm_guard > 0.f) a.msq_part = scratch(23, (size_t)batch * a.parts * sizeof(float));
    a.d_m_out = scratch(0, (size_t)batch * dd * sizeof(float));
    if (HAS_S) a.d_s_out = scratch(1, (size_t)batch * dd * sizeof(float));
    if (a.parts > 1) {
        size_t n = (size_t)a.parts * batch * seq_len;
        a.ws_dq = scratch(2, n * d * sizeof(float));
        a.ws_dk = scratch(3, n * d * sizeof(float));
        a.ws_gate = scratch(4, n * 4 * sizeof(float));
    }
    if (es.failed()) return true;
    switch (d) {
        case 8: launch_fused_d<8, HAS_S, FROZEN>(a); break;
        case 16: launch_fused_d<16, HAS_S, FROZEN>(a); break;
        case 32: launch_fused_d<32, HAS_S, FROZEN>(a); break;
        case 64: launch_fused_d<64, HAS_S, FROZEN>(a); break;
        case 128: launch_fused_d<128, HAS_S, FROZEN>(a); break;
    }
    if (a.parts > 1)
        finalize_parts(a.ws_dq, a.ws_dk, a.ws_gate, d_q, d_k, d_alpha, d_theta,
                       HAS_S ? d_eta : nullptr, a.parts, batch, seq_len, d, 0, seq_len);
    if (es.failed()) return true;
    if (a.msq_part && norm_bound_exceeded(a.msq_part, batch, a.parts, m_norm_guard)) return false;
    accumulate_over_batch2(a.d_m_out, d_m_initial, HAS_S ? a.d_s_out : nullptr, d_s_initial, batch, (int)dd);
    return true;
}

bool backward_ckpt_fused(bool has_s, bool frozen, const float *k, const float *v, const float *q,
                         const float *alpha, const float *theta, const float *eta,
                         const float *m_ckpt, const float *s_ckpt, const float *d_y,
                         float *d_k, float *d_v, float *d_q,
                         float *d_alpha, float *d_theta, float *d_eta,
                         float *d_m_initial, float *d_s_initial,
                         int seq_len, int d, int batch, int C, float m_norm_guard) {
#define NLH_FUSED(HS, FZ)                                                                        \
    return backward_ckpt_fused_t<HS, FZ>(k, v, q, alpha, theta, eta, m_ckpt, s_ckpt, d_y, d_k,  \
                                         d_v, d_q, d_alpha, d_theta, d_eta, d_m_initial,        \
                                         d_s_initial, seq_len, d, batch, C, m_norm_guard)
    if (has_s) { if (frozen) NLH_FUSED(true, true); else NLH_FUSED(true, false); }
    if (frozen) NLH_FUSED(false, true);
    NLH_FUSED(false, false);
#undef NLH_FUSED
}

}  // namespace nlh
