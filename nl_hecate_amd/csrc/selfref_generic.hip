// HOPE self-referential memory for any head size d >= 1 (the tiled kernels of selfref.hip cover
// d = 16, 32, 64): the update equations as the reference writes them
// (core/src/chunkwise_self_ref.rs:52-222 forward, :236-317 dgd_frozen_backward, :336-620 backward),
// one workgroup per chain, the six memories and their adjoints in global memory, per-token vectors
// in LDS.  Rows are dotted by a wave (lanes along the columns: coalesced), column sums by a thread
// per column.  Same caches and snapshots as the tiled kernels, so either forward serves either
// backward.  Not tuned: this is the path that makes the head sizes of the reference's own tests
// (d = 4) and odd sizes run, not the production shape.
#include "lane_ops.h"
#include "runtime.h"
#include "selfref_generic.h"

namespace nlh {
namespace {

constexpr int kT = 256, kW = kT / 64;

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

__device__ __forceinline__ float row_dot(const float *__restrict__ row, const float *__restrict__ x, int d) {
    float acc = 0.f;
    for (int j = threadIdx.x & 63; j < d; j += 64) acc = fmaf(row[j], x[j], acc);
    return wave_allreduce(acc);
}

__global__ __launch_bounds__(kT) void selfref_fwd_generic_kernel(
    float *__restrict__ mems, const float *__restrict__ emb, float *__restrict__ y, float *__restrict__ kc,
    float *__restrict__ vc, float *__restrict__ qc, float *__restrict__ al, float *__restrict__ th,
    float *__restrict__ am, float *__restrict__ em, float *__restrict__ frozen, int s, int d, int C, int nc, int sg) {
    extern __shared__ float sh[];
    float *x = sh, *k = x + d, *v = k + d, *q = v + d, *er = q + d, *ar = er + d;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, b = blockIdx.x;
    const size_t dd = (size_t)d * d;
    float *M = mems + (size_t)b * 6 * dd;
    for (int t = 0; t < s; t++) {
        const size_t tok = (size_t)b * s + t;
        float *F = frozen + ((size_t)b * nc + t / C) * 6 * dd;
        if (t % C == 0)
            for (size_t i = tid; i < 6 * dd; i += kT) F[i] = M[i];
        for (int j = tid; j < d; j += kT) x[j] = emb[tok * d + j];
        __syncthreads();
        // k, v, q, eta_raw, alpha_raw = M_c x with the current memories
        for (int r = wave; r < 5 * d; r += kW) {
            const int c = r / d, i = r - c * d;
            const float a = row_dot(M + c * dd + (size_t)i * d, x, d);
            if (lane == 0) (c == 0 ? k : c == 1 ? v : c == 2 ? q : c == 3 ? er : ar)[i] = a;
        }
        __syncthreads();
        float se = 0.f, sa = 0.f;
        for (int j = lane; j < d; j += 64) { se += er[j]; sa += ar[j]; }
        const float emean = wave_allreduce(se) / (float)d, amean = wave_allreduce(sa) / (float)d;
        const float alpha = sr_sigmoid(amean), theta = sr_softplus(emean), keep = 1.f - alpha;
        if (tid == 0) { al[tok] = alpha; th[tok] = theta; am[tok] = amean; em[tok] = emean; }
        for (int j = tid; j < d; j += kT) { kc[tok * d + j] = k[j]; vc[tok * d + j] = v[j]; qc[tok * d + j] = q[j]; }
        // per row: the read of m_mem before its update, the error against the frozen snapshot, the update
        for (int r = wave; r < 6 * d; r += kW) {
            const int c = r / d, i = r - c * d;
            float *row = M + c * dd + (size_t)i * d;
            const float *fr = F + c * dd + (size_t)i * d;
            float e = 0.f, tv = 0.f, yy = 0.f;
            for (int j = lane; j < d; j += 64) {
                const float f = fr[j];
                e = fmaf(f, k[j], e);
                if (sg) tv = fmaf(f, v[j], tv);
                if (c == 5) yy = fmaf(row[j], q[j], yy);
            }
            e = wave_allreduce(e);
            if (sg) tv = wave_allreduce(tv);
            if (c == 5) {
                yy = wave_allreduce(yy);
                if (lane == 0) y[tok * d + i] = yy;
            }
            const float scaled = theta * (e - (sg ? tv : v[i]));
            for (int j = lane; j < d; j += 64) row[j] = keep * row[j] - scaled * k[j];
        }
        __syncthreads();
    }
}

// The reverse sweep of one chain.  The states at the token starts of a chunk are replayed from the
// chunk's snapshot and the cached k, v, alpha, theta into traj ([C, 6, d*d] per chain; index 0 is the
// snapshot itself and is not stored); d_mems holds dM while the sweep runs, dfz the gradient that
// reaches the snapshot of the current chunk.
__global__ __launch_bounds__(kT) void selfref_bwd_generic_kernel(
    const float *__restrict__ emb, const float *__restrict__ dy_all, const float *__restrict__ kc,
    const float *__restrict__ vc, const float *__restrict__ qc, const float *__restrict__ al,
    const float *__restrict__ th, const float *__restrict__ am, const float *__restrict__ em,
    const float *__restrict__ frozen, float *__restrict__ d_emb, float *__restrict__ d_mems,
    float *__restrict__ traj_all, float *__restrict__ dfz_all, int s, int d, int C, int nc, int sg) {
    extern __shared__ float sh[];
    float *x = sh, *k = x + d, *v = k + d, *q = v + d, *dy = q + d;
    float *err = dy + d, *dmk = err + 6 * d;           // [6][d] each
    float *dq = dmk + 6 * d, *dkt = dq + d, *dvt = dkt + d;
    float *red = dvt + d;                              // [2][kW]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, b = blockIdx.x;
    const size_t dd = (size_t)d * d, n6 = 6 * dd;
    float *dm = d_mems + (size_t)b * n6, *dfz = dfz_all + (size_t)b * n6, *traj = traj_all + (size_t)b * C * n6;
    for (size_t i = tid; i < n6; i += kT) { dm[i] = 0.f; dfz[i] = 0.f; }
    __syncthreads();
    for (int ci = nc - 1; ci >= 0; ci--) {
        const int t0 = ci * C, len = min(C, s - t0);
        const float *F = frozen + ((size_t)b * nc + ci) * n6;
        if (ci < nc - 1) {   // the later chunk's snapshot was this chunk's final state
            for (size_t i = tid; i < n6; i += kT) { dm[i] += dfz[i]; dfz[i] = 0.f; }
            __syncthreads();
        }
        // replay: state at the start of token tt + 1 from the state at the start of token tt
        for (int tt = 0; tt + 1 < len; tt++) {
            const size_t tok = (size_t)b * s + t0 + tt;
            for (int j = tid; j < d; j += kT) { k[j] = kc[tok * d + j]; v[j] = vc[tok * d + j]; }
            const float keep = 1.f - al[tok], theta = th[tok];
            __syncthreads();
            for (int r = wave; r < 6 * d; r += kW) {
                const float *fr = F + (size_t)r * d;
                const float e = row_dot(fr, k, d);
                const float tgt = sg ? row_dot(fr, v, d) : v[r % d];
                if (lane == 0) err[r] = theta * (e - tgt);
            }
            __syncthreads();
            const float *src = tt == 0 ? F : traj + (size_t)tt * n6;
            float *dst = traj + (size_t)(tt + 1) * n6;
            for (int r = wave; r < 6 * d; r += kW) {
                const float se = err[r];
                for (int j = lane; j < d; j += 64) dst[(size_t)r * d + j] = keep * src[(size_t)r * d + j] - se * k[j];
            }
            __syncthreads();
        }
        for (int tt = len - 1; tt >= 0; tt--) {
            const size_t tok = (size_t)b * s + t0 + tt;
            const float *mt = tt == 0 ? F : traj + (size_t)tt * n6;
            for (int j = tid; j < d; j += kT) {
                x[j] = emb[tok * d + j]; k[j] = kc[tok * d + j]; v[j] = vc[tok * d + j]; q[j] = qc[tok * d + j];
                dy[j] = dy_all[tok * d + j];
            }
            const float alpha = al[tok], theta = th[tok], keep = 1.f - alpha;
            __syncthreads();
            // per row of every memory: the error against the snapshot and dM k
            for (int r = wave; r < 6 * d; r += kW) {
                const float *fr = F + (size_t)r * d;
                const float e = row_dot(fr, k, d);
                const float tgt = sg ? row_dot(fr, v, d) : v[r % d];
                const float mk = row_dot(dm + (size_t)r * d, k, d);
                if (lane == 0) { err[r] = e - tgt; dmk[r] = mk; }
            }
            __syncthreads();
            // per column: d_q = M_mem^T dy, the k and v gradients of the six updates, and this
            // thread's share of the two inner products behind the gate gradients
            float pa = 0.f, pt = 0.f;
            for (int j = tid; j < d; j += kT) {
                float sq = 0.f;
                for (int i = 0; i < d; i++) sq = fmaf(mt[5 * dd + (size_t)i * d + j], dy[i], sq);
                float dk = 0.f, dv = 0.f;
                for (int c = 5; c >= 0; c--) {   // the reference's order: mem, alpha, eta, q, v, k
                    const float *fc = F + c * dd, *gc = dm + c * dd, *mc = mt + c * dd;
                    float s1 = 0.f, s2 = 0.f, sv = 0.f;
                    for (int i = 0; i < d; i++) {
                        const float f = fc[(size_t)i * d + j], g = gc[(size_t)i * d + j], mk = dmk[c * d + i];
                        s1 = fmaf(f, mk, s1);
                        s2 = fmaf(err[c * d + i], g, s2);
                        pa = fmaf(mc[(size_t)i * d + j], g, pa);
                        if (sg) sv = fmaf(f, mk, sv);
                    }
                    dk -= theta * (s1 + s2);
                    pt = fmaf(s2, k[j], pt);
                    dv += sg ? theta * sv : theta * dmk[c * d + j];
                }
                dq[j] = sq; dkt[j] = dk; dvt[j] = dv;
            }
            pa = wave_allreduce(pa);
            pt = wave_allreduce(pt);
            if (lane == 0) { red[wave] = pa; red[kW + wave] = pt; }
            __syncthreads();
            float dalpha_tot = 0.f, dtheta_tot = 0.f;
            for (int w = 0; w < kW; w++) { dalpha_tot -= red[w]; dtheta_tot -= red[kW + w]; }
            const float sa = sr_sigmoid(am[tok]);
            const float dalpha_pd = dalpha_tot * sa * (1.f - sa) / (float)d;
            const float deta_pd = dtheta_tot * sr_sigmoid(em[tok]) / (float)d;
            // d_x = sum over the five read memories of M_c,t^T g_c
            for (int j = tid; j < d; j += kT) {
                float dx = 0.f;
                for (int c = 0; c < 5; c++) {
                    const float *mc = mt + c * dd;
                    for (int i = 0; i < d; i++) {
                        const float g = c == 0 ? dkt[i] : c == 1 ? dvt[i] : c == 2 ? dq[i] : c == 3 ? deta_pd : dalpha_pd;
                        dx = fmaf(mc[(size_t)i * d + j], g, dx);
                    }
                }
                d_emb[tok * d + j] = dx;
            }
            // per element: what reaches the snapshot, the retention chain, the reads of this token
            for (int r = wave; r < 6 * d; r += kW) {
                const int c = r / d, i = r - c * d;
                const float mk = theta * dmk[r];
                const float g = c == 0 ? dkt[i] : c == 1 ? dvt[i] : c == 2 ? dq[i] : c == 3 ? deta_pd : c == 4 ? dalpha_pd : dy[i];
                const float *u = c == 5 ? q : x;
                for (int j = lane; j < d; j += 64) {
                    const size_t e = (size_t)r * d + j;
                    dfz[e] += sg ? mk * (v[j] - k[j]) : -mk * k[j];
                    dm[e] = fmaf(keep, dm[e], g * u[j]);
                }
            }
            __syncthreads();
        }
    }
    for (size_t i = tid; i < n6; i += kT) dm[i] += dfz[i];
}

}  // namespace

size_t selfref_generic_lds_bytes(int d) { return ((size_t)20 * d + 2 * kW) * sizeof(float); }

bool selfref_generic_check(const char *fn, int d) {
    if (d < 1 || d > kSelfrefGenericMaxD) {
        fail("%s: d=%d is beyond the general kernels (1 .. %d)", fn, d, kSelfrefGenericMaxD);
        return false;
    }
    return true;
}

void selfref_forward_generic(float *mems, const float *emb, float *y, float *kc, float *vc, float *qc, float *al,
                             float *th, float *am, float *em, float *frozen, int s, int d, int batch, int C, int nc,
                             bool sg) {
    KernelTimer kt("selfref_fwd_generic_kernel");
    hipLaunchKernelGGL(selfref_fwd_generic_kernel, dim3(batch), dim3(kT), 6 * (size_t)d * sizeof(float), stream(), mems,
                       emb, y, kc, vc, qc, al, th, am, em, frozen, s, d, C, nc, sg ? 1 : 0);
    check_launch("selfref_fwd_generic_kernel");
}

void selfref_backward_generic(const float *emb, const float *dy, const float *kc, const float *vc, const float *qc,
                              const float *al, const float *th, const float *am, const float *em,
                              const float *frozen, float *d_emb, float *d_mems, int s, int d, int batch, int C,
                              int nc, bool sg) {
    const ErrorScope es;
    const size_t n6 = 6 * (size_t)d * d;
    const size_t traj_bytes = (size_t)batch * C * n6 * sizeof(float);
    if (traj_bytes > ((size_t)32 << 30)) {
        fail("selfref_chunkwise_backward_f32_rocm: chunk trajectory of %zu bytes exceeds the 32 GiB scratch limit",
             traj_bytes);
        return;
    }
    float *traj = scratch(0, traj_bytes), *dfz = scratch(1, (size_t)batch * n6 * sizeof(float));
    if (es.failed()) return;
    KernelTimer kt("selfref_bwd_generic_kernel");
    hipLaunchKernelGGL(selfref_bwd_generic_kernel, dim3(batch), dim3(kT), selfref_generic_lds_bytes(d), stream(), emb,
                       dy, kc, vc, qc, al, th, am, em, frozen, d_emb, d_mems, traj, dfz, s, d, C, nc, sg ? 1 : 0);
    check_launch("selfref_bwd_generic_kernel");
}

}  // namespace nlh
