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
// dF.  Chunks of up to 64 tokens use the explicit (low-rank) form of G_t, H_t:
// a chunk-parallel kernel prepares every product that does not depend on the
// sweep, the sweep kernel keeps only the per-token recurrence, and a second
// chunk-parallel kernel turns dg, dh into d_x.  Longer chunks replay G_t, H_t
// into a per-chunk trajectory in scratch memory.
#include <hip/hip_runtime.h>
#include <math.h>

#include "../../include/nl_hecate_ffi.h"
#include "lane_ops.h"
#include "quad_rows.h"
#include "runtime.h"
#include "selfref_generic.h"

namespace nlh {
namespace {

constexpr int kTB = 16;  // tokens staged in LDS at a time
using f32x4 = float __attribute__((ext_vector_type(4)));

// core/src/tensor.rs:202-207, 221-227.  The gates sit on the per-token critical path of the forward,
// so exp, log and the reciprocal are the hardware approximations (v_exp_f32, v_log_f32, v_rcp_f32: about
// one ulp each, three orders of magnitude inside the parity bar) instead of the library routines.
__device__ __forceinline__ float sr_sigmoid(float x) {
    if (x >= 15.f) return 1.f;
    if (x <= -15.f) return 0.f;
    return __builtin_amdgcn_rcpf(1.f + __expf(-x));
}
__device__ __forceinline__ float sr_softplus(float x) {
    if (x >= 15.f) return x;
    if (x <= -15.f) return 0.f;
    return __logf(1.f + __expf(x));
}

// ── forward ────────────────────────────────────────────────────────────────
// core/src/chunkwise_self_ref.rs:95-218.  mems [B,6,D*D] is updated in place;
// frozen [B,nc,6,D*D] receives the chunk-start snapshots; the per-token caches
// are what the backward consumes.
//
// Inside a chunk the six memories are M_c,t = F_c G_t + H_t (F_c the chunk-start
// snapshot, G and H as in the header), so a token costs two products with G
// (g = G x, p = G q), six with the frozen F_c (k, v, q, the two gates = F_c g,
// y = F_mem p) and one rank-1 update of G (and H) instead of eleven products
// and six updates with the M_c themselves; M_c = F_c G_L + H_L is formed once
// per chunk on the fp32 matrix cores.  Two LDS exchanges per token: (g_t, p_{t-1})
// and (k_t, v_t, q_t, gate sums); y is written one token late.
template <int D, bool SG>
__global__ __launch_bounds__(4 * D) void selfref_fwd_kernel(
    float *__restrict__ mems, const float *__restrict__ emb, float *__restrict__ y,
    float *__restrict__ k_cache, float *__restrict__ v_cache, float *__restrict__ q_cache,
    float *__restrict__ alpha_cache, float *__restrict__ theta_cache,
    float *__restrict__ amean_cache, float *__restrict__ emean_cache, float *__restrict__ frozen,
    int s, int C, int nc) {
    constexpr int CP = D / 4, NT = 4 * D, NW = (NT + 63) / 64, DD = D * D, LD = D + 4, JT = D / 16;
    __shared__ __align__(16) float xt[2][kTB][D];
    __shared__ __align__(16) float vec[5][D];   // g, p | k, v, q in row order
    __shared__ __align__(16) float gpart[4];      // per-wave sums of H x
    __shared__ __align__(16) float csum[2][NW][D];  // per-wave column sums of F_eta, F_alpha
    __shared__ __align__(16) float Gs[D * LD];  // G_L, then H-free staging of the chunk-end products
    __shared__ __align__(16) float Fs[D * LD];  // a wave touches its own 16 rows only

    const int tid = threadIdx.x, r = tid >> 2, cq = tid & 3, wave = tid >> 6, lane = tid & 63;
    const int c0 = cq * CP, ml = lane & 15, kg = lane >> 4, wr = 16 * wave;
    const size_t b = blockIdx.x;
    float *mb = mems + b * 6 * DD + r * D + c0;
    const float *xb = emb + b * (size_t)s * D;
    float *fb = frozen + b * (size_t)nc * 6 * DD + r * D + c0;

    float F[6][CP], G[CP], H[CP];
#pragma unroll
    for (int c = 0; c < 6; c++) lds_read<CP>(F[c], mb + c * DD);
#pragma unroll
    for (int i = 0; i < CP; i++) { G[i] = (c0 + i == r) ? 1.f : 0.f; H[i] = 0.f; }

    // F_c <- F_c G + H for the six memories; ends with every wave's F in registers.
    auto fold = [&]() {
        __syncthreads();
        vec_store<CP>(Gs + r * LD + c0, G);
        __syncthreads();
#pragma unroll
        for (int c = 0; c < 6; c++) {
            vec_store<CP>(Fs + r * LD + c0, F[c]);
            f32x4 acc[JT];
#pragma unroll
            for (int jt = 0; jt < JT; jt++) acc[jt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int k0 = 0; k0 < D; k0 += 4) {
                const float a = Fs[(wr + ml) * LD + k0 + kg];
#pragma unroll
                for (int jt = 0; jt < JT; jt++)
                    acc[jt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, Gs[(k0 + kg) * LD + 16 * jt + ml], acc[jt], 0, 0, 0);
            }
#pragma unroll
            for (int jt = 0; jt < JT; jt++) {
#pragma unroll
                for (int v = 0; v < 4; v++) Fs[(wr + 4 * kg + v) * LD + 16 * jt + ml] = acc[jt][v];
            }
            lds_read<CP>(F[c], Fs + r * LD + c0);
#pragma unroll
            for (int i = 0; i < CP; i++) F[c][i] += H[i];
        }
    };

    // The gates are means over the rows of F_eta g + H x and F_alpha g + H x: the frozen parts are
    // dots of g with the column means of F_eta, F_alpha, refreshed with each snapshot.
    float cse[CP], csa[CP];
    auto column_means = [&]() {
        float eo[CP / 4], ao[CP / 4];
        rows_reduce_scatter<CP>(F[3], eo);
        rows_reduce_scatter<CP>(F[4], ao);
        const int rho = lane >> 4, zoff = c0 + (CP / 2) * (rho >> 1) + (CP / 4) * (rho & 1);
        __syncthreads();
        if (((lane & 15) >> 2) == 0) {
#pragma unroll
            for (int i = 0; i < CP / 4; i++) { csum[0][wave][zoff + i] = eo[i]; csum[1][wave][zoff + i] = ao[i]; }
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < CP; i++) cse[i] = csa[i] = 0.f;
#pragma unroll
        for (int w = 0; w < NW; w++) {
            float te[CP], ta[CP];
            lds_read<CP>(te, &csum[0][w][c0]);
            lds_read<CP>(ta, &csum[1][w][c0]);
#pragma unroll
            for (int i = 0; i < CP; i++) { cse[i] += te[i]; csa[i] += ta[i]; }
        }
#pragma unroll
        for (int i = 0; i < CP; i++) { cse[i] *= 1.f / D; csa[i] *= 1.f / D; }
    };

    // x tiles: one float4 per thread per tile of kTB tokens
    const int xtt = tid / (D / 4), xj = (tid % (D / 4)) * 4;
    auto load_x = [&](int tile) -> float4 {
        const int t = tile * kTB + xtt;
        return t < s ? *reinterpret_cast<const float4 *>(xb + (size_t)t * D + xj) : make_float4(0, 0, 0, 0);
    };
    const int ntiles = (s + kTB - 1) / kTB;
    *reinterpret_cast<float4 *>(&xt[0][xtt][xj]) = load_x(0);
    __syncthreads();

    bool have_p = false;
    float p_r = 0.f, hq_r = 0.f;
    int chunk_t = 0, ci = 0;  // first token and index of the next chunk
    // y_{t-1} = F_mem p_{t-1} + H_{t-1} q_{t-1} from the column form of p
    auto emit_y = [&](int t_prev, bool valid) {
        float pc[CP];
        lds_read<CP>(pc, &vec[1][c0]);
        const float y_r = quad_allreduce(dotn<CP>(F[5], pc)) + hq_r;
        if (valid && cq == 3) y[(b * s + t_prev) * D + r] = y_r;
    };

    for (int tile = 0; tile < ntiles; tile++) {
        const int xb_cur = tile & 1;
        float4 xnext = make_float4(0, 0, 0, 0);
        if (tile + 1 < ntiles) xnext = load_x(tile + 1);
        const int nt = min(kTB, s - tile * kTB);
        for (int tt = 0; tt < nt; tt++) {
            const int t = tile * kTB + tt;
            if (t == chunk_t) {
                if (t > 0) {
                    if (cq == 1) vec[1][r] = p_r;
                    lds_barrier();
                    emit_y(t - 1, true);
                    have_p = false;
                    fold();
#pragma unroll
                    for (int i = 0; i < CP; i++) { G[i] = (c0 + i == r) ? 1.f : 0.f; H[i] = 0.f; }
                }
#pragma unroll
                for (int c = 0; c < 6; c++) vec_store<CP>(fb + ((size_t)ci * 6 + c) * DD, F[c]);
                column_means();
                ci++;
                chunk_t += C;
            }
            float xc[CP];
            lds_read<CP>(xc, &xt[xb_cur][tt][c0]);
            const float g_r = quad_allreduce(dotn<CP>(G, xc));
            const float hx_r = SG ? 0.f : quad_allreduce(dotn<CP>(H, xc));
            if (!SG) {  // sum of H x over the rows, for both gate means
                const float hs = rows_allreduce(hx_r);
                if (lane == 0) gpart[wave] = hs;
            }
            if (cq == 0) vec[0][r] = g_r;
            if (cq == 1) vec[1][r] = p_r;
            lds_barrier();
            emit_y(t - 1, have_p);  // no branch around it: its product overlaps the five below
            float gc[CP];
            lds_read<CP>(gc, &vec[0][c0]);
            float pr[3];
#pragma unroll
            for (int c = 0; c < 3; c++) pr[c] = quad_allreduce(dotn<CP>(F[c], gc)) + hx_r;
            const float k_r = pr[0], v_r = pr[1], q_r = pr[2];
            float em = quad_allreduce(dotn<CP>(cse, gc)), am = quad_allreduce(dotn<CP>(csa, gc));
            if (!SG) {
                float hm = 0.f;
#pragma unroll
                for (int w = 0; w < NW; w++) hm += gpart[w];
                em = fmaf(hm, 1.f / D, em); am = fmaf(hm, 1.f / D, am);
            }
            const float alpha = sr_sigmoid(am), theta = sr_softplus(em);
            if (tid == 0) {
                alpha_cache[b * s + t] = alpha; theta_cache[b * s + t] = theta;
                amean_cache[b * s + t] = am; emean_cache[b * s + t] = em;
            }
            if (cq < 3) {
                const float val = cq == 0 ? k_r : cq == 1 ? v_r : q_r;
                vec[2 + cq][r] = val;
                float *dst = cq == 0 ? k_cache : cq == 1 ? v_cache : q_cache;
                dst[(b * s + t) * D + r] = val;
            }
            lds_barrier();
            float kc[CP], qc[CP];
            lds_read<CP>(kc, &vec[2][c0]);
            lds_read<CP>(qc, &vec[4][c0]);
            // the read uses the memory before this token's update (:138)
            p_r = quad_allreduce(dotn<CP>(G, qc));
            hq_r = SG ? 0.f : quad_allreduce(dotn<CP>(H, qc));
            have_p = true;
            const float keep = 1.f - alpha;
            // self-generated target F_c v: the error is F_c (k - v)  (:155-166, :200)
            const float su = theta * (SG ? k_r - v_r : k_r), sv = theta * v_r;
#pragma unroll
            for (int i = 0; i < CP; i++) {
                G[i] = fmaf(-su, kc[i], keep * G[i]);
                if (!SG) H[i] = fmaf(sv, kc[i], keep * H[i]);
            }
        }
        if (tile + 1 < ntiles) {
            *reinterpret_cast<float4 *>(&xt[xb_cur ^ 1][xtt][xj]) = xnext;
            lds_barrier();
        }
    }
    if (cq == 1) vec[1][r] = p_r;
    lds_barrier();
    emit_y(s - 1, true);
    fold();
#pragma unroll
    for (int c = 0; c < 6; c++) vec_store<CP>(mb + c * DD, F[c]);
}

// ── backward ───────────────────────────────────────────────────────────────
// Staged tile arrays, [kTB][D] floats each.
enum { A_K = 0, A_V, A_Q, A_X, A_DY, A_G, A_P, A_DQ, A_DP, A_DG, A_DH, A_HX, A_HQ, A_COUNT };

// Chunks of up to kLrC tokens use the explicit form of the shared factors,
//     G_t = A_t I - sum_{s<t} c_ts u_s k_s^T,   H_t = sum_{s<t} c_ts v_s k_s^T,
//     A_t = prod_{r<t} (1-a_r),   c_ts = th_s prod_{s<r<t} (1-a_r),
// so that no G_t, H_t is ever written to memory: products G_t^T y, H_t^T y of a
// tile of tokens become two small LDS-resident matrix products, and the inner
// product <G_t, dG_{t+1}> + <H_t, dH_{t+1}> the alpha gradient needs follows
// from a scalar recurrence (see the reverse sweep).
constexpr int kLrC = 64;

// out_t = [A_t a1_t] + sum_{s<t} c_ts R_s ([l2_s . a2_t] - [l1_s . a1_t]) for the tokens of one tile, written
// to dst[tt * dst_stride + j]; t = li0 + tt is the token's index in its chunk, the a1 terms exist with
// HAS1, the a2 term with HAS2.  With L1 = u, R = k this is G_t^T a1 (plus H_t^T a2 for L2 = v); with
// L1 = k, R = u it is G_t a1; with L2 = k, R = v it is H_t a2.  Two products on the fp32 matrix cores:
// S = a2 L2^T - a1 L1^T (tokens x earlier tokens; wave w takes the earlier tokens 16 w ..), masked and
// scaled by c into Wt, then Wt R (wave w takes columns 16 w ..).  Tile rows have stride TL, the chunk
// arrays KL, Wt kWL (all = 4 mod 64, so the operand reads of a wave fall on 64 banks).  Rows of the
// chunk arrays behind the chunk's last token are read (times zero) and must be finite.  Called by
// every thread of the workgroup; one barrier inside, the caller synchronises before Wt, the tile or
// dst (when it is in LDS) are touched again.
constexpr int kWL = kLrC + 4;

template <int D, bool HAS1, bool HAS2>
__device__ __forceinline__ void lowrank_tile(const float *a1, const float *L1, const float *a2, const float *L2,
                                             const float *R, int li0, int nt, const float *CT, const float *cA,
                                             float *Wt, float *dst, size_t dst_stride, int tid) {
    constexpr int TL = D + 4, KL = D + 4, NW = D / 16;
    const int lane = tid & 63, wave = tid >> 6, ml = lane & 15, kg = lane >> 4;
    const int nprev = li0 + nt - 1;  // earlier tokens any token of the tile sees
    for (int st = wave; st < kLrC / 16; st += NW) {
        f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
        if (16 * st < nprev) {
#pragma unroll
            for (int k0 = 0; k0 < D; k0 += 4) {
                if (HAS1)
                    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(-a1[ml * TL + k0 + kg],
                                                               L1[(16 * st + ml) * KL + k0 + kg], acc, 0, 0, 0);
                if (HAS2)
                    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a2[ml * TL + k0 + kg],
                                                               L2[(16 * st + ml) * KL + k0 + kg], acc, 0, 0, 0);
            }
        }
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const int tt = 4 * kg + v, li = li0 + tt, s1 = 16 * st + ml;
            Wt[tt * kWL + s1] = (tt < nt && s1 < li) ? CT[li * kLrC + s1] * acc[v] : 0.f;
        }
    }
    __syncthreads();
    f32x4 o = f32x4{0.f, 0.f, 0.f, 0.f};
    // all of Wt's columns: those behind the tile's last token are zero, and a fixed trip count lets the
    // operand reads of the whole product be issued ahead of the first matrix instruction
#pragma unroll
    for (int k0 = 0; k0 < kLrC; k0 += 4)
        o = __builtin_amdgcn_mfma_f32_16x16x4f32(Wt[ml * kWL + k0 + kg], R[(k0 + kg) * KL + 16 * wave + ml], o, 0, 0, 0);
#pragma unroll
    for (int v = 0; v < 4; v++) {
        const int tt = 4 * kg + v, j = 16 * wave + ml;
        if (tt < nt) dst[(size_t)tt * dst_stride + j] = HAS1 ? fmaf(cA[li0 + tt], a1[tt * TL + j], o[v]) : o[v];
    }
}

// LDS of the chunk-parallel kernels: the chunk's keys KC and u = k - v (or v) XC, rows of stride D + 4;
// the table c_ts; one tile of products Wt; gates and the vectors c_L, A (kLrC + 1 entries).
template <int D>
struct ChunkLds {
    static constexpr int KL = D + 4;
    float *KC, *XC, *CT, *Wt, *cal, *cth, *cL, *cA, *tiles;
    __device__ explicit ChunkLds(float *base) {
        KC = base; XC = KC + kLrC * KL; CT = XC + kLrC * KL; Wt = CT + kLrC * kLrC;
        cal = Wt + kTB * kWL; cth = cal + kLrC; cL = cth + kLrC; cA = cL + kLrC; tiles = cA + 2 * kLrC;
    }
};

// Stages the chunk [t0, t0 + L) and builds its tables; ends with a barrier.
template <int D, bool SG>
__device__ __forceinline__ void chunk_setup(const ChunkLds<D> &m, const float *__restrict__ k_cache,
                                            const float *__restrict__ v_cache, const float *__restrict__ alpha_cache,
                                            const float *__restrict__ theta_cache, size_t tok0, int t0, int L, int tid) {
    constexpr int NT = 4 * D, V4 = D / 4, KL = D + 4;
    for (int e = tid; e < L * V4; e += NT) {
        const int li = e / V4, j = (e % V4) * 4;
        const size_t o = (tok0 + t0 + li) * D + j;
        const float4 k4 = *reinterpret_cast<const float4 *>(k_cache + o);
        const float4 v4 = *reinterpret_cast<const float4 *>(v_cache + o);
        *reinterpret_cast<float4 *>(m.KC + li * KL + j) = k4;
        *reinterpret_cast<float4 *>(m.XC + li * KL + j) =
            SG ? make_float4(k4.x - v4.x, k4.y - v4.y, k4.z - v4.z, k4.w - v4.w) : v4;
    }
    // rows behind a short chunk's last token enter the products of lowrank_tile times zero
    for (int e = L * KL + tid; e < kLrC * KL; e += NT) { m.KC[e] = 0.f; m.XC[e] = 0.f; }
    for (int e = tid; e < L; e += NT) { m.cal[e] = alpha_cache[tok0 + t0 + e]; m.cth[e] = theta_cache[tok0 + t0 + e]; }
    __syncthreads();
    if (tid < 64) {
        // lane t-1 builds row t of c (row L is c_L) from its diagonal leftwards:
        // c_{t,s} = th_s P, P = prod_{s<r<t} (1-a_r); P ends as A_t.  s runs in lock step
        // over the wave, so the gate reads are broadcasts that do not depend on the products.
        const int t = tid + 1;
        float P = 1.f;
#pragma unroll 8
        for (int s1 = kLrC - 1; s1 >= 0; s1--) {
            const float th_s = s1 < L ? m.cth[s1] : 0.f, keep_s = s1 < L ? 1.f - m.cal[s1] : 1.f;
            if (s1 < t && t <= L) {
                if (t < L) m.CT[t * kLrC + s1] = th_s * P;
                else m.cL[s1] = th_s * P;
                P *= keep_s;
            }
        }
        if (t <= L) m.cA[t] = P;
        if (t > L) m.cL[tid] = 0.f;  // c_Ls behind the chunk's last token (tid >= L)
        if (tid == 0) m.cA[0] = 1.f;
    }
    __syncthreads();
}

template <int D>
constexpr int chunk_lds_floats(int tiles) { return 2 * kLrC * (D + 4) + kLrC * kLrC + kTB * kWL + 5 * kLrC + tiles * kTB * (D + 4); }

// Chunk-parallel first pass of the backward (chunks of up to kLrC tokens): one workgroup per
// (chain, chunk).  Per token g = G x, p = G q, dp = F_mem^T dy, dq = G^T dp + H^T dy (and H x, H q
// without self-generated values) into rp [B, s, RS, D]; per chunk the transposed F_k, F_v, F_q
// (ftt [B, nc, 3, D, D]), the column sums of F_eta, F_alpha (csv [B, nc, 2, D]) and G_L, H_L
// (gl, hl [B, nc, D, D]; not for a chain's last chunk, whose boundary carries no gradient).
template <int D, bool SG>
__global__ __launch_bounds__(4 * D) void selfref_bwd_chunks_kernel(
    const float *__restrict__ emb, const float *__restrict__ d_y, const float *__restrict__ k_cache,
    const float *__restrict__ v_cache, const float *__restrict__ q_cache,
    const float *__restrict__ alpha_cache, const float *__restrict__ theta_cache,
    const float *__restrict__ frozen, float *__restrict__ rp, float *__restrict__ ftt, float *__restrict__ csv,
    float *__restrict__ gl, float *__restrict__ hl, int s, int C, int nc) {
    constexpr int NT = 4 * D, DD = D * D, V4 = D / 4, TL = D + 4, KL = D + 4, JT = D / 16, FL = D + 1;
    constexpr int RS = SG ? 4 : 6;
    extern __shared__ __align__(16) float chunk_lds[];
    const ChunkLds<D> m(chunk_lds);
    float *tX = m.tiles, *tQ = tX + kTB * TL, *tDY = tQ + kTB * TL, *tDP = tDY + kTB * TL;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, ml = lane & 15, kg = lane >> 4, wr = 16 * wave;
    const int ci = blockIdx.x % nc;
    const size_t b = blockIdx.x / nc, chunk = blockIdx.x, tok0 = b * (size_t)s;
    const int t0 = ci * C, L = min(C, s - t0);
    const float *fz = frozen + chunk * 6 * DD;

    {   // transposed F_k, F_v, F_q through LDS (row stride D + 1: both directions fall on 64 banks)
        float *Ft = chunk_lds;
#pragma unroll
        for (int comp = 0; comp < 3; comp++) {
            for (int e = tid; e < DD / 4; e += NT) {
                const int mr = e / V4, j = (e % V4) * 4;
                const float4 f = *reinterpret_cast<const float4 *>(fz + (size_t)comp * DD + mr * D + j);
                float *dst = Ft + (comp * D + mr) * FL + j;
                dst[0] = f.x; dst[1] = f.y; dst[2] = f.z; dst[3] = f.w;
            }
        }
        for (int e = tid; e < 2 * D; e += NT) {
            const float *src = fz + (size_t)(3 + e / D) * DD + (e % D);
            float a = 0.f;
#pragma unroll 8
            for (int c = 0; c < D; c++) a += src[c * D];
            csv[chunk * 2 * D + e] = a;
        }
        __syncthreads();
#pragma unroll
        for (int comp = 0; comp < 3; comp++) {
            for (int e = tid; e < DD / 4; e += NT) {
                const int rr = e / V4, c = (e % V4) * 4;
                const float *src = Ft + (comp * D + c) * FL + rr;
                *reinterpret_cast<float4 *>(ftt + (chunk * 3 + comp) * DD + rr * D + c) =
                    make_float4(src[0], src[FL], src[2 * FL], src[3 * FL]);
            }
        }
        __syncthreads();
    }
    chunk_setup<D, SG>(m, k_cache, v_cache, alpha_cache, theta_cache, tok0, t0, L, tid);

    const float *Fm = fz + 5 * DD;
    const int stt = tid / V4, sj = (tid % V4) * 4;
    const int ntile = (L + kTB - 1) / kTB;
    for (int tile = 0; tile < ntile; tile++) {
        const int tb = t0 + tile * kTB, nt = min(kTB, t0 + L - tb), li0 = tb - t0;
        __syncthreads();
        if (stt < nt) {
            const size_t o = (tok0 + tb + stt) * D + sj;
            *reinterpret_cast<float4 *>(tQ + stt * TL + sj) = *reinterpret_cast<const float4 *>(q_cache + o);
            *reinterpret_cast<float4 *>(tX + stt * TL + sj) = *reinterpret_cast<const float4 *>(emb + o);
            *reinterpret_cast<float4 *>(tDY + stt * TL + sj) = *reinterpret_cast<const float4 *>(d_y + o);
        }
        __syncthreads();
        float *rp_t = rp + (tok0 + tb) * RS * D;
        {   // dp_t = F_mem^T dy_t: wave w takes columns 16 w ..
            f32x4 o = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int k0 = 0; k0 < D; k0 += 4)
                o = __builtin_amdgcn_mfma_f32_16x16x4f32(tDY[ml * TL + k0 + kg], Fm[(k0 + kg) * D + wr + ml], o, 0, 0, 0);
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int tt = 4 * kg + v, j = wr + ml;
                tDP[tt * TL + j] = o[v];
                if (tt < nt) rp_t[((size_t)tt * RS + 3) * D + j] = o[v];
            }
        }
        // g = G x, p = G q
        lowrank_tile<D, true, false>(tX, m.KC, nullptr, nullptr, SG ? m.XC : m.KC, li0, nt, m.CT, m.cA, m.Wt, rp_t,
                                     (size_t)RS * D, tid);
        __syncthreads();
        lowrank_tile<D, true, false>(tQ, m.KC, nullptr, nullptr, SG ? m.XC : m.KC, li0, nt, m.CT, m.cA, m.Wt,
                                     rp_t + D, (size_t)RS * D, tid);
        __syncthreads();
        lowrank_tile<D, true, !SG>(tDP, SG ? m.XC : m.KC, tDY, m.XC, m.KC, li0, nt, m.CT, m.cA, m.Wt, rp_t + 2 * D,
                                   (size_t)RS * D, tid);
        if (!SG) {  // H x and H q for the scalar recurrence of the reverse sweep
            __syncthreads();
            lowrank_tile<D, false, true>(nullptr, nullptr, tX, m.KC, m.XC, li0, nt, m.CT, m.cA, m.Wt, rp_t + 4 * D,
                                         (size_t)RS * D, tid);
            __syncthreads();
            lowrank_tile<D, false, true>(nullptr, nullptr, tQ, m.KC, m.XC, li0, nt, m.CT, m.cA, m.Wt, rp_t + 5 * D,
                                         (size_t)RS * D, tid);
        }
    }
    if (ci < nc - 1) {
        // G_L = A_L I - sum_s c_Ls u_s k_s^T and H_L = sum_s c_Ls v_s k_s^T; wave w takes rows 16 w ..
        f32x4 g_acc[JT], h_acc[JT];
#pragma unroll
        for (int jt = 0; jt < JT; jt++) g_acc[jt] = h_acc[jt] = f32x4{0.f, 0.f, 0.f, 0.f};
        const float *UC = SG ? m.XC : m.KC;
        const int kend = (L + 3) & ~3;
        for (int k0 = 0; k0 < kend; k0 += 4) {
            const float cl = m.cL[k0 + kg];
            const float au = UC[(k0 + kg) * KL + wr + ml] * cl, avv = SG ? 0.f : m.XC[(k0 + kg) * KL + wr + ml] * cl;
#pragma unroll
            for (int jt = 0; jt < JT; jt++) {
                const float kb = m.KC[(k0 + kg) * KL + 16 * jt + ml];
                g_acc[jt] = __builtin_amdgcn_mfma_f32_16x16x4f32(au, kb, g_acc[jt], 0, 0, 0);
                if (!SG) h_acc[jt] = __builtin_amdgcn_mfma_f32_16x16x4f32(avv, kb, h_acc[jt], 0, 0, 0);
            }
        }
        const float aL = m.cA[L];
#pragma unroll
        for (int jt = 0; jt < JT; jt++) {
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int row = wr + 4 * kg + v, col = 16 * jt + ml;
                gl[chunk * DD + row * D + col] = (row == col ? aL : 0.f) - g_acc[jt][v];
                if (!SG) hl[chunk * DD + row * D + col] = h_acc[jt][v];
            }
        }
    }
}

// Chunk-parallel last pass on the same path: d_x_t = G_t^T dg_t + H_t^T dh_t, in place on d_emb, which
// holds dg [B, s, D] on entry (dh likewise in its own buffer without self-generated values).
template <int D, bool SG>
__global__ __launch_bounds__(4 * D) void selfref_bwd_dx_kernel(
    const float *__restrict__ k_cache, const float *__restrict__ v_cache, const float *__restrict__ alpha_cache,
    const float *__restrict__ theta_cache, float *d_emb, const float *__restrict__ dh, int s, int C, int nc) {
    constexpr int V4 = D / 4, TL = D + 4;
    extern __shared__ __align__(16) float chunk_lds[];
    const ChunkLds<D> m(chunk_lds);
    float *tDG = m.tiles, *tDH = tDG + kTB * TL;
    const int tid = threadIdx.x;
    const int ci = blockIdx.x % nc;
    const size_t b = blockIdx.x / nc, tok0 = b * (size_t)s;
    const int t0 = ci * C, L = min(C, s - t0);
    chunk_setup<D, SG>(m, k_cache, v_cache, alpha_cache, theta_cache, tok0, t0, L, tid);
    const int stt = tid / V4, sj = (tid % V4) * 4;
    const int ntile = (L + kTB - 1) / kTB;
    for (int tile = 0; tile < ntile; tile++) {
        const int tb = t0 + tile * kTB, nt = min(kTB, t0 + L - tb);
        __syncthreads();
        if (stt < nt) {
            const size_t o = (tok0 + tb + stt) * D + sj;
            *reinterpret_cast<float4 *>(tDG + stt * TL + sj) = *reinterpret_cast<const float4 *>(d_emb + o);
            if (!SG) *reinterpret_cast<float4 *>(tDH + stt * TL + sj) = *reinterpret_cast<const float4 *>(dh + o);
        }
        __syncthreads();
        lowrank_tile<D, true, !SG>(tDG, SG ? m.XC : m.KC, tDH, m.XC, m.KC, tb - t0, nt, m.CT, m.cA, m.Wt,
                                   d_emb + (tok0 + tb) * D, (size_t)D, tid);
    }
}

template <int D, bool SG, bool LR>
__global__ __launch_bounds__(4 * D) void selfref_bwd_kernel(
    const float *__restrict__ emb, const float *__restrict__ d_y, const float *__restrict__ k_cache,
    const float *__restrict__ v_cache, const float *__restrict__ q_cache,
    const float *__restrict__ alpha_cache, const float *__restrict__ theta_cache,
    const float *__restrict__ amean_cache, const float *__restrict__ emean_cache,
    const float *__restrict__ frozen, float *__restrict__ d_emb, float *__restrict__ d_mems,
    float *gtraj, float *htraj, float *rp, const float *__restrict__ ftt, const float *__restrict__ csv,
    float *__restrict__ dh_buf, int s, int C, int nc) {
    // LR: chunks of up to kLrC tokens.  selfref_bwd_chunks_kernel has filled rp, ftt, csv and put G_L, H_L
    // per chunk where the trajectory path keeps G_t, H_t per token (gtraj, htraj); this kernel leaves dg
    // in d_emb (dh in dh_buf) for selfref_bwd_dx_kernel.
    constexpr int CP = D / 4, NT = 4 * D, NW = (NT + 63) / 64, DD = D * D, V4 = D / 4, LD = D + 4, JT = D / 16;
    constexpr int TL = D + 4;  // row stride of the staged tiles
    constexpr int TILE_F = A_COUNT * kTB * TL, BND_F = 3 * D * LD;
    constexpr int RAW_F = TILE_F > BND_F ? TILE_F : BND_F;
    __shared__ __align__(16) float raw[RAW_F];
    __shared__ __align__(16) float wv[2][2][D];
    __shared__ __align__(16) float zp[2][2][NW][D];
    __shared__ __align__(16) float sp[2][NW][2];
    __shared__ __align__(16) float sc[4][kTB];
    __shared__ __align__(16) float av[2][D];
    __shared__ float dEA[2][kTB];  // de_t, da_t of the tile
    constexpr int RS = (LR && !SG) ? 6 : 4;  // vectors per token kept between the two passes of a chunk
#define T_(a, tt, i) raw[((a) * kTB + (tt)) * TL + (i)]

    const int tid = threadIdx.x, r = tid >> 2, cq = tid & 3, wave = tid >> 6, lane = tid & 63;
    const int c0 = cq * CP;
    const size_t b = blockIdx.x;
    const size_t tok0 = b * (size_t)s;
    float *gt_b = LR ? nullptr : gtraj + b * (size_t)C * DD;
    float *ht_b = (SG || LR) ? nullptr : htraj + b * (size_t)C * DD;
    float *rp_b = rp + tok0 * RS * D;
    float sig_base = 0.f, pend = 0.f;
    const int stt = tid / V4, sj = (tid % V4) * 4;  // staging slot: token, column

    // dF_k, dF_v, dF_q, dF_mem live in the accumulator layout of the matrix cores (wave w owns rows
    // 16 w .., lane (ml, kg) rows 4 kg + v of column 16 jt + ml); the equal rows of dF_eta, dF_alpha are
    // rows 0 and 1 of accEA, wave w holding columns 16 w .. (lanes kg = 0).
    const int ml = lane & 15, kg = lane >> 4, wr = 16 * wave;
    f32x4 dFm[4][JT], accEA = f32x4{0.f, 0.f, 0.f, 0.f};
    float dG[CP], dH[CP];
#pragma unroll
    for (int jt = 0; jt < JT; jt++) dFm[0][jt] = dFm[1][jt] = dFm[2][jt] = dFm[3][jt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < CP; i++) dG[i] = dH[i] = 0.f;

    // Inputs of the next tile of the reverse sweep, requested one tile ahead (low-rank path).
    float4 pf_k, pf_v, pf_q, pf_x, pf_dy, pf_g, pf_p, pf_dq, pf_dp, pf_hx, pf_hq, pf_s;
    pf_k = pf_v = pf_q = pf_x = pf_dy = pf_g = pf_p = pf_dq = pf_dp = pf_hx = pf_hq = pf_s = make_float4(0, 0, 0, 0);
#define SWEEP_REQUEST(tile_)                                                                        \
    {                                                                                               \
        const int tb_ = t0 + (tile_) * kTB, nt_ = min(kTB, t0 + L - tb_);                           \
        if (stt < nt_) {                                                                            \
            const size_t o_ = (tok0 + tb_ + stt) * D + sj;                                          \
            const float *rpt_ = rp_b + (size_t)(tb_ + stt) * RS * D + sj;                           \
            pf_k = *reinterpret_cast<const float4 *>(k_cache + o_);                                 \
            pf_v = *reinterpret_cast<const float4 *>(v_cache + o_);                                 \
            pf_q = *reinterpret_cast<const float4 *>(q_cache + o_);                                 \
            pf_x = *reinterpret_cast<const float4 *>(emb + o_);                                     \
            pf_dy = *reinterpret_cast<const float4 *>(d_y + o_);                                    \
            pf_g = *reinterpret_cast<const float4 *>(rpt_);                                         \
            pf_p = *reinterpret_cast<const float4 *>(rpt_ + D);                                     \
            pf_dq = *reinterpret_cast<const float4 *>(rpt_ + 2 * D);                                \
            pf_dp = *reinterpret_cast<const float4 *>(rpt_ + 3 * D);                                \
            if (!SG) {                                                                              \
                pf_hx = *reinterpret_cast<const float4 *>(rpt_ + 4 * D);                            \
                pf_hq = *reinterpret_cast<const float4 *>(rpt_ + 5 * D);                            \
            }                                                                                       \
        }                                                                                           \
        if (tid < nt_) {                                                                            \
            const size_t o_ = tok0 + tb_ + tid;                                                     \
            pf_s = make_float4(alpha_cache[o_], theta_cache[o_], amean_cache[o_], emean_cache[o_]); \
        }                                                                                           \
    }

    for (int ci = nc - 1; ci >= 0; ci--) {
        const int t0 = ci * C, L = min(C, s - t0);
        const float *fz = frozen + (b * nc + ci) * (size_t)6 * DD;
        // transposed register copies of F_k, F_v, F_q (F_mem on the trajectory path) and the column sums
        // of F_eta, F_alpha.  F_k, F_v, F_q pass through LDS (row stride D + 1: coalesced reads, and both
        // the writes and the transposed reads of a wave fall on 64 banks); the column sums reduce over
        // the rows of a wave in registers and over the waves through LDS.
        float FTk[CP], FTv[CP], FTq[CP], FTm[CP], csE = 0.f, csA = 0.f;
        if constexpr (LR) {  // prepared per chunk by selfref_bwd_chunks_kernel
            const size_t chunk = b * nc + ci;
            lds_read<CP>(FTk, ftt + (chunk * 3 + 0) * DD + r * D + c0);
            lds_read<CP>(FTv, ftt + (chunk * 3 + 1) * DD + r * D + c0);
            lds_read<CP>(FTq, ftt + (chunk * 3 + 2) * DD + r * D + c0);
            csE = csv[chunk * 2 * D + r];
            csA = csv[chunk * 2 * D + D + r];
        } else {
            constexpr int FL = D + 1;
            float *Ft = raw;
            float fe[CP], fa[CP], eo[CP / 4], ao[CP / 4];
            lds_read<CP>(fe, fz + 3 * DD + r * D + c0);
            lds_read<CP>(fa, fz + 4 * DD + r * D + c0);
#pragma unroll
            for (int comp = 0; comp < 3; comp++) {
                for (int e = tid; e < DD / 4; e += NT) {
                    const int m = e / V4, j = (e % V4) * 4;
                    const float4 f = *reinterpret_cast<const float4 *>(fz + (size_t)comp * DD + m * D + j);
                    float *dst = Ft + (comp * D + m) * FL + j;
                    dst[0] = f.x; dst[1] = f.y; dst[2] = f.z; dst[3] = f.w;
                }
            }
            rows_reduce_scatter<CP>(fe, eo);
            rows_reduce_scatter<CP>(fa, ao);
            const int rho = lane >> 4, zoff = c0 + (CP / 2) * (rho >> 1) + (CP / 4) * (rho & 1);
            if (((lane & 15) >> 2) == 0) {
#pragma unroll
                for (int i = 0; i < CP / 4; i++) { zp[0][0][wave][zoff + i] = eo[i]; zp[0][1][wave][zoff + i] = ao[i]; }
            }
            __syncthreads();
#pragma unroll
            for (int x = 0; x < NW; x++) { csE += zp[0][0][x][r]; csA += zp[0][1][x][r]; }
#pragma unroll
            for (int i = 0; i < CP; i++) {
                FTk[i] = Ft[(0 * D + c0 + i) * FL + r];
                FTv[i] = Ft[(1 * D + c0 + i) * FL + r];
                FTq[i] = Ft[(2 * D + c0 + i) * FL + r];
                FTm[i] = fz[5 * DD + (size_t)(c0 + i) * D + r];
            }
            __syncthreads();
        }
        // ---- first pass over the chunk: g = G x, p = G q, dp = F_mem^T dy, dq = G^T dp + H^T dy ----
        float G[CP], H[CP];
        const int ntile = (L + kTB - 1) / kTB;
        if constexpr (LR) {
            // g, p, dp, dq are in rp already; G_L, H_L of the chunk for the boundary and sigma_L
#pragma unroll
            for (int i = 0; i < CP; i++) G[i] = H[i] = 0.f;
            if (ci < nc - 1) {
                lds_read<CP>(G, gtraj + (b * nc + ci) * (size_t)DD + r * D + c0);
                if (!SG) lds_read<CP>(H, htraj + (b * nc + ci) * (size_t)DD + r * D + c0);
            }
        } else {
#pragma unroll
            for (int i = 0; i < CP; i++) { G[i] = (c0 + i == r) ? 1.f : 0.f; H[i] = 0.f; }
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

        }
        // ---- chunk boundary: gradients of F'_c = F_c G_L + H_L flow into dG_L, dH_L, dF_c ----
        __syncthreads();
        if (LR) SWEEP_REQUEST(ntile - 1)
        if (ci < nc - 1) {
            float *Fs = raw, *Bm = raw + D * LD, *GLT = raw + 2 * D * LD;
#pragma unroll
            for (int i = 0; i < CP; i++) GLT[(c0 + i) * LD + r] = G[i];
            if (kg == 0) { av[0][wr + ml] = accEA[0]; av[1][wr + ml] = accEA[1]; }
            __syncthreads();
            {   // rows of dF_eta, dF_alpha are all equal: rank-1 terms
                float eE[CP], eA[CP];
                lds_read<CP>(eE, &av[0][c0]);
                lds_read<CP>(eA, &av[1][c0]);
#pragma unroll
                for (int i = 0; i < CP; i++) {
                    dG[i] = csE * eE[i] + csA * eA[i];
                    dH[i] = eE[i] + eA[i];
                }
            }
            // The eight D x D products run on the matrix cores in fp32 (v_mfma_f32_16x16x4_f32: lane
            // (ml, kg) = (lane % 16, lane / 16) feeds A[ml][kg], B[kg][ml] and receives rows 4 kg + v of
            // column ml); wave w owns rows 16 w .. 16 w + 15 of both results, which are also the rows its
            // lanes keep in the row-quad layout, so values change layout through the wave's own rows of Bm
            // without a workgroup barrier.
            f32x4 accG[JT];
#pragma unroll
            for (int jt = 0; jt < JT; jt++) accG[jt] = f32x4{0.f, 0.f, 0.f, 0.f};
            // F_c travels global -> registers -> Fs; the next one is requested before the products of the
            // current one, so only the first request's latency is exposed.
            f32x4 fnext[JT];  // D*D/4 vectors of four over 4*D threads
#pragma unroll
            for (int i = 0; i < JT; i++) {
                const int e = tid + i * NT;
                fnext[i] = *reinterpret_cast<const f32x4 *>(fz + (e / V4) * D + (e % V4) * 4);
            }
#pragma unroll
            for (int comp = 0; comp < 4; comp++) {
                __syncthreads();
#pragma unroll
                for (int i = 0; i < JT; i++) {
                    const int e = tid + i * NT;
                    *reinterpret_cast<f32x4 *>(Fs + (e / V4) * LD + (e % V4) * 4) = fnext[i];
                }
                if (comp < 3) {
                    const float *nf = fz + (size_t)(comp < 2 ? comp + 1 : 5) * DD;
#pragma unroll
                    for (int i = 0; i < JT; i++) {
                        const int e = tid + i * NT;
                        fnext[i] = *reinterpret_cast<const f32x4 *>(nf + (e / V4) * D + (e % V4) * 4);
                    }
                }
#pragma unroll
                for (int jt = 0; jt < JT; jt++) {
#pragma unroll
                    for (int v = 0; v < 4; v++) Bm[(wr + 4 * kg + v) * LD + 16 * jt + ml] = dFm[comp][jt][v];
                }
                if (!SG) {  // the wave's own rows, back in the row-quad layout
                    float t[CP];
                    lds_read<CP>(t, Bm + r * LD + c0);
#pragma unroll
                    for (int i = 0; i < CP; i++) dH[i] += t[i];
                }
                __syncthreads();
                f32x4 accN[JT];
#pragma unroll
                for (int jt = 0; jt < JT; jt++) accN[jt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
                for (int k0 = 0; k0 < D; k0 += 4) {
                    const float a1 = Fs[(k0 + kg) * LD + wr + ml];   // (F_c^T)[row][k]
                    const float a2 = Bm[(wr + ml) * LD + k0 + kg];   // dF'_c[row][k]
#pragma unroll
                    for (int jt = 0; jt < JT; jt++) {
                        const float b1 = Bm[(k0 + kg) * LD + 16 * jt + ml];
                        const float b2 = GLT[(k0 + kg) * LD + 16 * jt + ml];
                        accG[jt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a1, b1, accG[jt], 0, 0, 0);
                        accN[jt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a2, b2, accN[jt], 0, 0, 0);
                    }
                }
#pragma unroll
                for (int jt = 0; jt < JT; jt++) dFm[comp][jt] = accN[jt];  // dF_c = dF'_c G_L^T
            }
            __syncthreads();  // every wave has read Bm
            {   // dG_L += sum_c F_c^T dF'_c, into the row-quad layout through the wave's own rows of Bm
#pragma unroll
                for (int jt = 0; jt < JT; jt++) {
#pragma unroll
                    for (int v = 0; v < 4; v++) Bm[(wr + 4 * kg + v) * LD + 16 * jt + ml] = accG[jt][v];
                }
                float t[CP];
                lds_read<CP>(t, Bm + r * LD + c0);
#pragma unroll
                for (int i = 0; i < CP; i++) dG[i] += t[i];
            }
            {   // accE <- G_L accE, accA <- G_L accA (column-indexed): rows 0 and 1 of one more product,
                // wave w computing columns 16 w .. 16 w + 15
                f32x4 accV = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
                for (int k0 = 0; k0 < D; k0 += 4) {
                    const float a = ml < 2 ? av[ml][k0 + kg] : 0.f;
                    accV = __builtin_amdgcn_mfma_f32_16x16x4f32(a, GLT[(k0 + kg) * LD + wr + ml], accV, 0, 0, 0);
                }
                accEA = accV;
            }
            __syncthreads();
        }

        if (LR) {
            // sigma_L = <G_L, dG_L> + <H_L, dH_L>, as per-lane partial sums that the first token of the
            // sweep reduces.  With sigma_t = <G_t, dG_t> + <H_t, dH_t> the two recurrences give
            //     (1-a_t) (<G_t, dG_{t+1}> + <H_t, dH_{t+1}>) = sigma_{t+1} + th_t (u.w - v.wh),
            //     sigma_t = that + dg.g + dp.p + dh.(H x) + dy.(H q).
            pend = dotn<CP>(G, dG);  // both are zero in a chain's last chunk
            if (!SG) pend += dotn<CP>(H, dH);
            sig_base = 0.f;
        }

        // ---- reverse sweep over the chunk ----
        for (int tile = ntile - 1; tile >= 0; tile--) {
            const int tb = t0 + tile * kTB, nt = min(kTB, t0 + L - tb);
            if (LR) {
                // the tile was requested a tile ago (the chunk's last tile before the boundary products)
                if (stt < nt) {
                    *reinterpret_cast<float4 *>(&T_(A_K, stt, sj)) = pf_k;
                    *reinterpret_cast<float4 *>(&T_(A_V, stt, sj)) = pf_v;
                    *reinterpret_cast<float4 *>(&T_(A_Q, stt, sj)) = pf_q;
                    *reinterpret_cast<float4 *>(&T_(A_X, stt, sj)) = pf_x;
                    *reinterpret_cast<float4 *>(&T_(A_DY, stt, sj)) = pf_dy;
                    *reinterpret_cast<float4 *>(&T_(A_G, stt, sj)) = pf_g;
                    *reinterpret_cast<float4 *>(&T_(A_P, stt, sj)) = pf_p;
                    *reinterpret_cast<float4 *>(&T_(A_DQ, stt, sj)) = pf_dq;
                    *reinterpret_cast<float4 *>(&T_(A_DP, stt, sj)) = pf_dp;
                    if (!SG) {
                        *reinterpret_cast<float4 *>(&T_(A_HX, stt, sj)) = pf_hx;
                        *reinterpret_cast<float4 *>(&T_(A_HQ, stt, sj)) = pf_hq;
                    }
                }
                if (tid < nt) {
                    sc[0][tid] = pf_s.x; sc[1][tid] = pf_s.y;
                    const float sa = sr_sigmoid(pf_s.z), keep_t = 1.f - pf_s.x;
                    // sigmoid'(mean) / d, here already over (1 - a_t): the sweep forms (1 - a_t) <G_t, dG_{t+1}>;
                    // a saturated gate (keep = 0) has no gradient
                    sc[2][tid] = keep_t > 0.f ? sa * (1.f - sa) * (1.f / D) / keep_t : 0.f;
                    sc[3][tid] = sr_sigmoid(pf_s.w) * (1.f / D);
                }
                __syncthreads();
                if (tile > 0) SWEEP_REQUEST(tile - 1)
            } else {
            if (stt < nt) {
                const size_t o = (tok0 + tb + stt) * D + sj;
                const float *rpt = rp_b + (size_t)(tb + stt) * RS * D + sj;
                *reinterpret_cast<float4 *>(&T_(A_K, stt, sj)) = *reinterpret_cast<const float4 *>(k_cache + o);
                *reinterpret_cast<float4 *>(&T_(A_V, stt, sj)) = *reinterpret_cast<const float4 *>(v_cache + o);
                *reinterpret_cast<float4 *>(&T_(A_Q, stt, sj)) = *reinterpret_cast<const float4 *>(q_cache + o);
                *reinterpret_cast<float4 *>(&T_(A_X, stt, sj)) = *reinterpret_cast<const float4 *>(emb + o);
                *reinterpret_cast<float4 *>(&T_(A_DY, stt, sj)) = *reinterpret_cast<const float4 *>(d_y + o);
                *reinterpret_cast<float4 *>(&T_(A_G, stt, sj)) = *reinterpret_cast<const float4 *>(rpt);
                *reinterpret_cast<float4 *>(&T_(A_P, stt, sj)) = *reinterpret_cast<const float4 *>(rpt + D);
                *reinterpret_cast<float4 *>(&T_(A_DQ, stt, sj)) = *reinterpret_cast<const float4 *>(rpt + 2 * D);
                *reinterpret_cast<float4 *>(&T_(A_DP, stt, sj)) = *reinterpret_cast<const float4 *>(rpt + 3 * D);
                if (LR && !SG) {
                    *reinterpret_cast<float4 *>(&T_(A_HX, stt, sj)) = *reinterpret_cast<const float4 *>(rpt + 4 * D);
                    *reinterpret_cast<float4 *>(&T_(A_HQ, stt, sj)) = *reinterpret_cast<const float4 *>(rpt + 5 * D);
                }
            }
            if (tid < nt) {
                const size_t o = tok0 + tb + tid;
                sc[0][tid] = alpha_cache[o]; sc[1][tid] = theta_cache[o];
                const float sa = sr_sigmoid(amean_cache[o]);
                sc[2][tid] = sa * (1.f - sa) * (1.f / D);           // sigmoid'(mean) / d
                sc[3][tid] = sr_sigmoid(emean_cache[o]) * (1.f / D);  // softplus'(mean) / d
            }
            }
            float Gt[CP], Ht[CP];
            if (!LR) {
                const int li = tb + nt - 1 - t0;
                lds_read<CP>(Gt, gt_b + (size_t)li * DD + r * D + c0);
                if (!SG) lds_read<CP>(Ht, ht_b + (size_t)li * DD + r * D + c0);
                __syncthreads();
            }
            for (int tt = nt - 1; tt >= 0; tt--) {
                const int pb = tt & 1, li = tb + tt - t0;
                float Gn[CP], Hn[CP];
                if (!LR && tt > 0) {
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
                float alp = LR ? pend : dotn<CP>(Gt, dG), thp = 0.25f * u_r * w;
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
                    if (!LR) alp += dotn<CP>(Ht, dH);
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
                if (LR) {
                    const float keepalp = fmaf(-th, dth, sig_base - dal);  // sigma_{t+1} + th (u.w - v.wh)
                    dal = -keepalp;  // times 1 / (1 - a_t), folded into sc[2]
                    sig_base = keepalp;
                }
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
                if (LR) {
                    pend = dg * T_(A_G, tt, r) + dp_r * T_(A_P, tt, r);
                    if (!SG) pend += dh * T_(A_HX, tt, r) + dy_r * T_(A_HQ, tt, r);
                    pend *= 0.25f;  // the four lanes of a row hold the same values
                }
                float xc[CP], qc[CP];
                lds_read<CP>(xc, &T_(A_X, tt, c0));
                lds_read<CP>(qc, &T_(A_Q, tt, c0));
                const float keep = 1.f - al;
#pragma unroll
                for (int i = 0; i < CP; i++) {
                    dG[i] = fmaf(dg, xc[i], fmaf(dp_r, qc[i], keep * dG[i]));
                    if (!SG) dH[i] = fmaf(dh, xc[i], fmaf(dy_r, qc[i], keep * dH[i]));
                }
                // dk_t, dv_t take the place of k_t, v_t (read by every wave before this token's barrier);
                // the outer products with g_t, p_t follow for the whole tile after the loop
                if (cq == 0) { T_(A_K, tt, r) = dk_r; T_(A_V, tt, r) = dv_r; }
                if (tid == 0) { dEA[0][tt] = de; dEA[1][tt] = da; }
                if (cq == 0) T_(A_DG, tt, r) = dg;
                if (!SG && cq == 1) T_(A_DH, tt, r) = dh;
                if (!LR && tt > 0) {
#pragma unroll
                    for (int i = 0; i < CP; i++) { Gt[i] = Gn[i]; if (!SG) Ht[i] = Hn[i]; }
                }
            }
            __syncthreads();
            // the tile's outer products: dF_k += dk g^T, dF_v += dv g^T, dF_q += dq g^T, dF_mem += dy p^T,
            // accE += sum_t de_t g_t, accA += sum_t da_t g_t (tokens are the contraction index)
#pragma unroll
            for (int k0 = 0; k0 < kTB; k0 += 4) {
                const int tk = k0 + kg;
                const bool ok = tk < nt;
                const float a_k = ok ? T_(A_K, tk, wr + ml) : 0.f, a_v = ok ? T_(A_V, tk, wr + ml) : 0.f;
                const float a_q = ok ? T_(A_DQ, tk, wr + ml) : 0.f, a_y = ok ? T_(A_DY, tk, wr + ml) : 0.f;
                const float a_e = (ok && ml < 2) ? dEA[ml][tk] : 0.f;
#pragma unroll
                for (int jt = 0; jt < JT; jt++) {
                    const float b_g = ok ? T_(A_G, tk, 16 * jt + ml) : 0.f, b_p = ok ? T_(A_P, tk, 16 * jt + ml) : 0.f;
                    dFm[0][jt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a_k, b_g, dFm[0][jt], 0, 0, 0);
                    dFm[1][jt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a_v, b_g, dFm[1][jt], 0, 0, 0);
                    dFm[2][jt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a_q, b_g, dFm[2][jt], 0, 0, 0);
                    dFm[3][jt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a_y, b_p, dFm[3][jt], 0, 0, 0);
                }
                accEA = __builtin_amdgcn_mfma_f32_16x16x4f32(a_e, ok ? T_(A_G, tk, wr + ml) : 0.f, accEA, 0, 0, 0);
            }
            // d_x_t = G_t^T dg_t + H_t^T dh_t
            if (LR) {
                if (stt < nt) {
                    const size_t o = (tok0 + tb + stt) * D + sj;
                    *reinterpret_cast<float4 *>(d_emb + o) = *reinterpret_cast<const float4 *>(&T_(A_DG, stt, sj));
                    if (!SG) *reinterpret_cast<float4 *>(dh_buf + o) = *reinterpret_cast<const float4 *>(&T_(A_DH, stt, sj));
                }
            } else if (stt < nt) {
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
    float *dmb = d_mems + b * 6 * DD;
#pragma unroll
    for (int comp = 0; comp < 4; comp++) {
        float *dst = dmb + (comp < 3 ? comp : 5) * DD;
#pragma unroll
        for (int jt = 0; jt < JT; jt++) {
#pragma unroll
            for (int v = 0; v < 4; v++) dst[(wr + 4 * kg + v) * D + 16 * jt + ml] = dFm[comp][jt][v];
        }
    }
    __syncthreads();
    if (kg == 0) { av[0][wr + ml] = accEA[0]; av[1][wr + ml] = accEA[1]; }
    __syncthreads();
    {
        float eE[CP], eA[CP];
        lds_read<CP>(eE, &av[0][c0]);
        lds_read<CP>(eA, &av[1][c0]);
        vec_store<CP>(dmb + 3 * DD + r * D + c0, eE);
        vec_store<CP>(dmb + 4 * DD + r * D + c0, eA);
    }
#undef T_
#undef SWEEP_REQUEST
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

struct BwdArgs {
    const float *emb, *dy, *kc, *vc, *qc, *al, *th, *am, *em, *frozen;
    float *d_emb, *d_mems;
    float *gtraj, *htraj;  // trajectory path: G_t, H_t of one chunk; low-rank path: G_L, H_L per chunk
    float *rp, *ftt, *csv, *dh;
    int batch, s, C, nc;
    bool sg, lowrank;
};

template <int D, bool SG>
void launch_bwd_sg(const BwdArgs &a) {
    const dim3 block(4 * D);
    auto set_lds = [](auto kernel, size_t bytes) {
        check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes), "dynamic LDS size");
    };
    if (a.lowrank) {
        const size_t lds1 = chunk_lds_floats<D>(4) * sizeof(float), lds3 = chunk_lds_floats<D>(2) * sizeof(float);
        set_lds(selfref_bwd_chunks_kernel<D, SG>, lds1);
        hipLaunchKernelGGL((selfref_bwd_chunks_kernel<D, SG>), dim3(a.batch * a.nc), block, lds1, stream(), a.emb,
                           a.dy, a.kc, a.vc, a.qc, a.al, a.th, a.frozen, a.rp, a.ftt, a.csv, a.gtraj, a.htraj, a.s,
                           a.C, a.nc);
        check_launch("selfref_bwd_chunks_kernel");
        {
            KernelTimer kt("selfref_bwd_kernel");
            hipLaunchKernelGGL((selfref_bwd_kernel<D, SG, true>), dim3(a.batch), block, 0, stream(), a.emb, a.dy,
                               a.kc, a.vc, a.qc, a.al, a.th, a.am, a.em, a.frozen, a.d_emb, a.d_mems, a.gtraj,
                               a.htraj, a.rp, a.ftt, a.csv, a.dh, a.s, a.C, a.nc);
            check_launch("selfref_bwd_kernel");
        }
        set_lds(selfref_bwd_dx_kernel<D, SG>, lds3);
        hipLaunchKernelGGL((selfref_bwd_dx_kernel<D, SG>), dim3(a.batch * a.nc), block, lds3, stream(), a.kc, a.vc,
                           a.al, a.th, a.d_emb, a.dh, a.s, a.C, a.nc);
        check_launch("selfref_bwd_dx_kernel");
    } else {
        KernelTimer kt("selfref_bwd_kernel");
        hipLaunchKernelGGL((selfref_bwd_kernel<D, SG, false>), dim3(a.batch), block, 0, stream(), a.emb, a.dy, a.kc,
                           a.vc, a.qc, a.al, a.th, a.am, a.em, a.frozen, a.d_emb, a.d_mems, a.gtraj, a.htraj, a.rp,
                           a.ftt, a.csv, a.dh, a.s, a.C, a.nc);
        check_launch("selfref_bwd_kernel");
    }
}

template <int D>
void launch_bwd(const BwdArgs &a) {
    if (a.sg) launch_bwd_sg<D, true>(a);
    else launch_bwd_sg<D, false>(a);
}

// head sizes of the tiled kernels; every other one takes the general kernels of selfref_generic.hip
bool tiled_head_size(int d) { return d == 16 || d == 32 || d == 64; }

bool check_args(const char *fn, int seq_len, int d, int batch, int chunk_size) {
    if (seq_len <= 0 || batch <= 0) { fail("%s: seq_len and batch_size must be positive", fn); return false; }
    if (chunk_size < 1) { fail("%s: chunk_size must be >= 1", fn); return false; }
    if (!tiled_head_size(d) && !selfref_generic_check(fn, d)) return false;
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
    if (!tiled_head_size(d)) {
        selfref_forward_generic(mems, embedded, y, k_cache, v_cache, q_cache, alpha_cache, theta_cache,
                                alpha_mean_cache, eta_mean_cache, frozen, seq_len, d, batch_size, C, nc, sg);
        return;
    }
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
    const ErrorScope es;
    if (!check_args("selfref_chunkwise_backward_f32_rocm", seq_len, d, batch_size, chunk_size)) return;
    const int C = chunk_size > seq_len ? seq_len : chunk_size;
    const int nc = (seq_len + chunk_size - 1) / chunk_size;
    const bool sg = self_generated_values != 0;
    if (!tiled_head_size(d)) {
        selfref_backward_generic(embedded, d_y, k_cache, v_cache, q_cache, alpha_cache, theta_cache, alpha_mean_cache,
                                 eta_mean_cache, frozen, d_embedded, d_mems, seq_len, d, batch_size, C, nc, sg);
        return;
    }
    const size_t dd = (size_t)d * d;
    const size_t traj_bytes = (size_t)batch_size * C * dd * sizeof(float);
    if (C > kLrC && traj_bytes > ((size_t)32 << 30)) {
        fail("selfref_chunkwise_backward_f32_rocm: chunk trajectory of %zu bytes exceeds the 32 GiB scratch limit",
             traj_bytes);
        return;
    }
    // Chunks of up to kLrC tokens take the low-rank path (no trajectory: G_L, H_L and the transposed
    // frozen matrices per chunk instead, six vectors per token without self-generated values).
    const bool lowrank = C <= kLrC;
    const size_t chunks = (size_t)batch_size * nc, tokens = (size_t)batch_size * seq_len;
    BwdArgs a{};
    a.emb = embedded; a.dy = d_y; a.kc = k_cache; a.vc = v_cache; a.qc = q_cache; a.al = alpha_cache;
    a.th = theta_cache; a.am = alpha_mean_cache; a.em = eta_mean_cache; a.frozen = frozen;
    a.d_emb = d_embedded; a.d_mems = d_mems;
    a.batch = batch_size; a.s = seq_len; a.C = C; a.nc = nc; a.sg = sg; a.lowrank = lowrank;
    a.gtraj = scratch(0, lowrank ? chunks * dd * sizeof(float) : traj_bytes);
    a.htraj = sg ? nullptr : scratch(1, lowrank ? chunks * dd * sizeof(float) : traj_bytes);
    a.rp = scratch(2, tokens * ((lowrank && !sg) ? 6 : 4) * d * sizeof(float));
    if (lowrank) {
        a.ftt = scratch(3, chunks * 3 * dd * sizeof(float));
        a.csv = scratch(4, chunks * 2 * d * sizeof(float));
        a.dh = sg ? nullptr : scratch(5, tokens * d * sizeof(float));
    }
    if (es.failed()) return;
    if (d == 16) launch_bwd<16>(a); else if (d == 32) launch_bwd<32>(a); else launch_bwd<64>(a);
}
