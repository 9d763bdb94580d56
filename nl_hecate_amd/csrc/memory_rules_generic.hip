// Exact and frozen-M0 Delta / Titans rule for ANY head size d >= 1, error clip and M-norm projection
// included: what serves the head sizes the register-resident kernels of memory_rules.hip are not
// instantiated for (the reference's kernels take any d: core/kernels/titans_forward.cu:83-210,
// titans_backward.cu:66-341; its own test uses d = 4, core/tests/test_cuda_titans.rs:99-128).
//
// One workgroup of 256 threads per chain; the d x d state lives in memory (the trajectory the caller
// asked for, or a work buffer) and is updated element-wise between barriers; the token's vectors and
// the per-row results live in LDS.  Row products (M k, dS k) take a wave per row with lanes along the
// row (contiguous reads); column products (M^T dy, dS^T e) take a thread per column with consecutive
// threads on consecutive addresses.  Same arithmetic as the tiled kernels, other summation orders.
// Not tuned: a head size that matters gets an instantiation in memory_rules.hip.
#include <hip/hip_runtime.h>

#include "lane_ops.h"
#include "rule_args.h"
#include "runtime.h"

namespace nlh {
namespace {

constexpr int kGThr = 256;
constexpr int kGWaves = kGThr / 64;

__device__ __forceinline__ bool mnorm_on(float m) { return m > 0.f && m < 1e30f; }

// sum over the workgroup; red: kGWaves floats of LDS; every thread calls it
__device__ __forceinline__ float block_sum(float x, float *red) {
    x = wave_allreduce(x);
    __syncthreads();                       // red may still be read from the previous use
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = x;
    __syncthreads();
    float s = 0.f;
#pragma unroll
    for (int w = 0; w < kGWaves; w++) s += red[w];
    return s;
}

// out[i] = sum_j A[i][j] x[j] (- sub[i]) for all rows: a wave per row
__device__ __forceinline__ void row_products(const float *A, const float *x, const float *sub, float *out, int d) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int i = wave; i < d; i += kGWaves) {
        float acc = 0.f;
        for (int j = lane; j < d; j += 64) acc = fmaf(A[(size_t)i * d + j], x[j], acc);
        acc = wave_allreduce(acc);
        if (lane == 0) out[i] = sub ? acc - sub[i] : acc;
    }
}

template <bool HAS_S, int STORE, bool FROZEN>
__global__ __launch_bounds__(kGThr) void rule_fwd_generic_kernel(FwdArgs a, int d, float *work_m, float *work_s,
                                                                  float *work_m0) {
    extern __shared__ float smem[];
    float *sk = smem, *sq = sk + d, *sv = sq + d, *se = sv + d, *red = se + d;
    const int chain = blockIdx.x, tid = threadIdx.x;
    const size_t dd = (size_t)d * d;
    const float *kb = a.k + (size_t)chain * a.input_stride * d, *vb = a.v + (size_t)chain * a.input_stride * d;
    const float *qb = a.q + (size_t)chain * a.input_stride * d;
    const float *ab = a.alpha + (size_t)chain * a.input_stride, *tb = a.theta + (size_t)chain * a.input_stride;
    const float *eb = HAS_S ? a.eta + (size_t)chain * a.input_stride : nullptr;
    float *yb = a.y + (size_t)chain * a.seq_len * d;
    float *mo = a.m_out + (size_t)chain * a.state_stride;
    float *so = HAS_S ? a.s_out + (size_t)chain * a.state_stride : nullptr;
    const float *mi = a.m_initial + (size_t)chain * a.m_stride;
    const float *si = HAS_S ? a.s_initial + (size_t)chain * a.m_stride : nullptr;
    // current state: slot t of the trajectory, or the work buffers
    float *cm = STORE == STORE_TRAJ ? mo : work_m + (size_t)chain * dd;
    float *cs = HAS_S ? (STORE == STORE_TRAJ ? so : work_s + (size_t)chain * dd) : nullptr;
    float *m0 = FROZEN ? work_m0 + (size_t)chain * dd : nullptr;
    for (size_t e = tid; e < dd; e += kGThr) {
        const float mv = mi[e];
        cm[e] = mv;
        if (STORE == STORE_CKPT) mo[e] = mv;
        if (FROZEN) m0[e] = mv;
        if (HAS_S) {
            const float svv = si[e];
            cs[e] = svv;
            if (STORE == STORE_CKPT) so[e] = svv;
        }
    }
    __syncthreads();
    const bool clip_on = a.error_clip > 0.f, mn_on = mnorm_on(a.m_norm_max);
    int ckpt_slot = 1;
    for (int t = 0; t < a.seq_len; t++) {
        for (int j = tid; j < d; j += kGThr) {
            sk[j] = kb[(size_t)t * d + j];
            sq[j] = qb[(size_t)t * d + j];
            sv[j] = vb[(size_t)t * d + j];
        }
        const float al = ab[t], th = tb[t], et = HAS_S ? eb[t] : 0.f, ret = 1.f - al;
        __syncthreads();
        row_products(FROZEN ? m0 : cm, sk, sv, se, d);   // e = M k - v
        __syncthreads();
        float scale = 1.f;
        if (clip_on) {
            float sq_sum = 0.f;
            for (int i = tid; i < d; i += kGThr) sq_sum = fmaf(se[i], se[i], sq_sum);
            const float nrm = sqrtf(block_sum(sq_sum, red));
            if (nrm > a.error_clip) scale = a.error_clip / nrm;
        }
        // state update, element-wise; the next state goes to slot t + 1 of a trajectory, else in place
        float *nm = STORE == STORE_TRAJ ? cm + dd : cm;
        float *ns = HAS_S ? (STORE == STORE_TRAJ ? cs + dd : cs) : nullptr;
        float fro = 0.f;
        for (size_t e = tid; e < dd; e += kGThr) {
            const int i = (int)(e / d), j = (int)(e % d);
            const float te = th * scale * se[i];
            float mv;
            if (HAS_S) {
                const float sn = et * cs[e] - te * sk[j];
                ns[e] = sn;
                mv = ret * cm[e] + sn;
            } else {
                mv = ret * cm[e] - te * sk[j];
            }
            nm[e] = mv;
            fro = fmaf(mv, mv, fro);
        }
        if (mn_on) {
            const float fn = sqrtf(block_sum(fro, red));   // includes the barrier that publishes nm
            if (fn > a.m_norm_max) {
                const float sc = a.m_norm_max / fn;
                for (size_t e = tid; e < dd; e += kGThr) nm[e] *= sc;
            }
        }
        __syncthreads();
        cm = nm;
        cs = ns;
        if ((STORE == STORE_CKPT || FROZEN) && (((t + 1) % a.ckpt_interval == 0) || (t + 1 == a.seq_len))) {
            for (size_t e = tid; e < dd; e += kGThr) {
                const float mv = cm[e];
                if (STORE == STORE_CKPT) {
                    mo[(size_t)ckpt_slot * dd + e] = mv;
                    if (HAS_S) so[(size_t)ckpt_slot * dd + e] = cs[e];
                }
                if (FROZEN) m0[e] = mv;
            }
            ckpt_slot++;
        }
        row_products(cm, sq, nullptr, yb + (size_t)t * d, d);   // y = M_{t+1} q
        __syncthreads();   // the vectors and (frozen) M0 are rewritten next
    }
}

template <bool HAS_S, bool FROZEN>
__global__ __launch_bounds__(kGThr) void rule_bwd_generic_kernel(BwdArgs a, int d, float *work_dm0) {
    extern __shared__ float smem[];
    float *sk = smem, *sq = sk + d, *sv = sq + d, *sdy = sv + d, *se = sdy + d, *sgk = se + d, *red = sgk + d;
    const int chain = blockIdx.x, tid = threadIdx.x;
    const size_t dd = (size_t)d * d;
    const int seq_len = a.seq_len, t_start = a.t_start, t_end = a.t_end;
    const size_t tok = (size_t)chain * seq_len;
    const float *kb = a.k + tok * d, *vb = a.v + tok * d, *qb = a.q + tok * d, *dyb = a.d_y + tok * d;
    const float *ab = a.alpha + tok, *tb = a.theta + tok, *eb = HAS_S ? a.eta + tok : nullptr;
    const float *ms = a.m_states + (size_t)chain * a.traj_stride;
    const float *ss = HAS_S ? a.s_states + (size_t)chain * a.traj_stride : nullptr;
    // d_M, d_S live in the output buffers and are updated in place
    float *dM = a.d_m_out + (size_t)chain * dd, *dS = HAS_S ? a.d_s_out + (size_t)chain * dd : nullptr;
    float *dM0 = FROZEN ? work_dm0 + (size_t)chain * dd : nullptr;
    for (size_t e = tid; e < dd; e += kGThr) {
        dM[e] = a.d_m_seed ? a.d_m_seed[(size_t)chain * dd + e] : 0.f;
        if (HAS_S) dS[e] = a.d_s_seed ? a.d_s_seed[(size_t)chain * dd + e] : 0.f;
        if (FROZEN) dM0[e] = 0.f;
    }
    __syncthreads();
    const bool clip_on = a.error_clip > 0.f;
    for (int t = t_end - 1; t >= t_start; t--) {
        const int lt = t - t_start;
        const float *Mt = ms + (size_t)lt * dd, *Mn = Mt + dd, *Mx = FROZEN ? ms : Mt;
        const float *St = HAS_S ? ss + (size_t)lt * dd : nullptr;
        for (int j = tid; j < d; j += kGThr) {
            sk[j] = kb[(size_t)t * d + j];
            sq[j] = qb[(size_t)t * d + j];
            sv[j] = vb[(size_t)t * d + j];
            sdy[j] = dyb[(size_t)t * d + j];
        }
        const float al = ab[t], th = tb[t], et = HAS_S ? eb[t] : 0.f, ret = 1.f - al;
        __syncthreads();
        // d_M += dy q^T, d_S += d_M; <M_t, d_M>, <S_t, d_S>
        float pa = 0.f, pe = 0.f;
        for (size_t e = tid; e < dd; e += kGThr) {
            const int i = (int)(e / d), j = (int)(e % d);
            const float g = dM[e] + sdy[i] * sq[j];
            dM[e] = g;
            pa = fmaf(Mt[e], g, pa);
            if (HAS_S) {
                const float gs = dS[e] + g;
                dS[e] = gs;
                pe = fmaf(St[e], gs, pe);
            }
        }
        pa = block_sum(pa, red);
        if (HAS_S) pe = block_sum(pe, red);
        __syncthreads();   // d_M, d_S of every thread are visible
        const float *G = HAS_S ? dS : dM;
        row_products(Mx, sk, sv, se, d);       // e = M k - v
        row_products(G, sk, nullptr, sgk, d);  // G k
        // d_q = M_{t+1}^T dy: a thread per column
        for (int j = tid; j < d; j += kGThr) {
            float acc = 0.f;
            for (int i = 0; i < d; i++) acc = fmaf(Mn[(size_t)i * d + j], sdy[i], acc);
            a.d_q[(tok + t) * d + j] = acc;
        }
        __syncthreads();
        if (clip_on) {
            float sq_sum = 0.f;
            for (int i = tid; i < d; i += kGThr) sq_sum = fmaf(se[i], se[i], sq_sum);
            const float nrm = sqrtf(block_sum(sq_sum, red));
            if (nrm > a.error_clip) {
                const float sc = a.error_clip / nrm;
                for (int i = tid; i < d; i += kGThr) se[i] *= sc;
            }
            __syncthreads();
        }
        float pt = 0.f;
        for (int i = tid; i < d; i += kGThr) {
            pt = fmaf(se[i], sgk[i], pt);
            a.d_v[(tok + t) * d + i] = th * sgk[i];     // d_v = -d_err, d_err = -theta G k
        }
        pt = block_sum(pt, red);
        if (tid == 0) {
            a.d_alpha[tok + t] = -pa;
            a.d_theta[tok + t] = -pt;
            if (HAS_S) a.d_eta[tok + t] = pe;
        }
        // d_k = -theta G^T e + M^T d_err: a thread per column
        for (int j = tid; j < d; j += kGThr) {
            float acc = 0.f;
            for (int i = 0; i < d; i++)
                acc = fmaf(-th * se[i], G[(size_t)i * d + j], fmaf(-th * sgk[i], Mx[(size_t)i * d + j], acc));
            a.d_k[(tok + t) * d + j] = acc;
        }
        __syncthreads();   // G was read by every thread; now it changes
        for (size_t e = tid; e < dd; e += kGThr) {
            const int i = (int)(e / d), j = (int)(e % d);
            const float derr = -th * sgk[i];
            if (HAS_S) dS[e] *= et;
            if (FROZEN) {
                dM[e] *= ret;
                dM0[e] = fmaf(derr, sk[j], dM0[e]);
            } else {
                dM[e] = fmaf(ret, dM[e], derr * sk[j]);
            }
        }
        __syncthreads();
    }
    if (FROZEN)
        for (size_t e = tid; e < dd; e += kGThr) dM[e] += dM0[e];
}

}  // namespace

void launch_fwd_generic(const FwdArgs &a, int d, int batch, bool has_s, int store, bool frozen) {
    const ErrorScope es;
    const size_t dd = (size_t)d * d, lds = (4 * (size_t)d + kGWaves) * sizeof(float);
    if (lds > 64 * 1024) { fail("memory rule: d=%d is beyond the general kernels' LDS vectors (d <= 4000).", d); return; }
    float *wm = store != STORE_TRAJ ? scratch(16, (size_t)batch * dd * sizeof(float)) : nullptr;
    float *ws = (store != STORE_TRAJ && has_s) ? scratch(17, (size_t)batch * dd * sizeof(float)) : nullptr;
    float *w0 = frozen ? scratch(18, (size_t)batch * dd * sizeof(float)) : nullptr;
    if (es.failed()) return;
    KernelTimer kt("rule_fwd_generic_kernel");
#define NLH_GF(HS, ST, FZ)                                                                                   \
    hipLaunchKernelGGL((rule_fwd_generic_kernel<HS, ST, FZ>), dim3(batch), dim3(kGThr), lds, stream(), a, d, \
                       wm, ws, w0)
#define NLH_GF_ST(HS, FZ)                                      \
    do {                                                       \
        if (store == STORE_TRAJ) NLH_GF(HS, STORE_TRAJ, FZ);   \
        else if (store == STORE_CKPT) NLH_GF(HS, STORE_CKPT, FZ); \
        else NLH_GF(HS, STORE_NONE, FZ);                       \
    } while (0)
    if (has_s) { if (frozen) NLH_GF_ST(true, true); else NLH_GF_ST(true, false); }
    else { if (frozen) NLH_GF_ST(false, true); else NLH_GF_ST(false, false); }
#undef NLH_GF_ST
#undef NLH_GF
    check_launch("rule_fwd_generic_kernel");
}

void launch_bwd_generic(const BwdArgs &a, int d, bool has_s, bool frozen) {
    const ErrorScope es;
    const size_t dd = (size_t)d * d, lds = (6 * (size_t)d + kGWaves) * sizeof(float);
    if (lds > 64 * 1024) { fail("memory rule: d=%d is beyond the general kernels' LDS vectors (d <= 2700).", d); return; }
    float *w0 = frozen ? scratch(19, (size_t)a.batch * dd * sizeof(float)) : nullptr;
    if (es.failed()) return;
    KernelTimer kt("rule_bwd_generic_kernel");
#define NLH_GB(HS, FZ) \
    hipLaunchKernelGGL((rule_bwd_generic_kernel<HS, FZ>), dim3(a.batch), dim3(kGThr), lds, stream(), a, d, w0)
    if (has_s) { if (frozen) NLH_GB(true, true); else NLH_GB(true, false); }
    else { if (frozen) NLH_GB(false, true); else NLH_GB(false, false); }
#undef NLH_GB
    check_launch("rule_bwd_generic_kernel");
}

}  // namespace nlh
