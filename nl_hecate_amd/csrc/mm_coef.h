// Gate coefficients of the chunkwise matrix forms on the fp32 matrix cores: the vectors a, beta, h and the tables
// c, bb, r of one chunk of up to 64 tokens, built in LDS by the first waves of a 512-thread workgroup.
#pragma once
#include <hip/hip_runtime.h>

#include "mm_tiles.h"

namespace nlh {
namespace mmt {

// Gate coefficients of one chunk (L <= 64 tokens), all in LDS.
struct Coef {
    float al[CW], th[CW], et[CW];   // gates (eta = 0 for the Delta rule), zero beyond L
    float a[CW], beta[CW], h[CW];   // a_t, beta_t, h_t
    float cl[CW], bl[CW];           // c[L-1,j], bb[j,L-1]
};

// Gates of token (lane % 64) of a chunk, one register each; zero beyond L (eta = 0 without S).
struct Gates { float al, th, et; };
__device__ __forceinline__ Gates fetch_gates(const float *alpha, const float *theta, const float *eta, int L,
                                             bool has_s) {
    const int t = threadIdx.x & 63;
    Gates g;
    g.al = t < L ? alpha[t] : 0.f;
    g.th = t < L ? theta[t] : 0.f;
    g.et = (t < L && has_s) ? eta[t] : 0.f;
    return g;
}
__device__ __forceinline__ void load_gates(Coef &cf, const Gates &g) {
    const int t = threadIdx.x;
    if (t < CW) { cf.al[t] = g.al; cf.th[t] = g.th; cf.et[t] = g.et; }
}

__device__ __forceinline__ float lane_bcast(float x, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), lane));
}

// Column j of c, bb, r (thread j of waves 0, 2, 3), optionally stored: Cc[t][j], Bb[j][t], Rr[j][t]
// (stride LDM; entries outside j <= t < L are zero), plus the vectors (wave 1).  The gates
// are read from global memory into one register per lane and broadcast per step, so the
// sequential loops carry no memory latency.  Needs a barrier afterwards.
__device__ __forceinline__ void coefficients(Coef &cf, const Gates &g, int L, float *Cc, float *Bb, float *Rr) {
    const int j = threadIdx.x & 63, w = threadIdx.x >> 6;
    if (w >= 4) return;
    const float keep_j = 1.f - g.al;   // 1 beyond L
    const float eta_j = g.et;          // 0 beyond L
    const bool jv = j < L;
    if (w == 0) {
        // branch-free: tokens after j update the running products; lanes t >= L broadcast
        // keep = 1, eta = 0, which leaves cc unchanged
        float b = 1.f, cc = 1.f, blv = 0.f;
#pragma unroll 16
        for (int t = 0; t < CW; t++) {
            const float keep = lane_bcast(keep_j, t), et = lane_bcast(eta_j, t);
            const bool after = t > j;
            b *= after ? et : 1.f;
            cc = after ? fmaf(keep, cc, b) : cc;
            blv = (t == L - 1) ? b : blv;
            if (Cc) Cc[t * LDM + j] = (jv && t >= j && t < L) ? cc : 0.f;
        }
        cf.cl[j] = jv ? cc : 0.f;
        cf.bl[j] = jv ? blv : 0.f;
    } else if (w == 1) {
        // a_t, beta_t, h_t: every lane runs the same scalar recurrence, lane t keeps step t
        float a = 1.f, h = 1.f, beta = 0.f, ka = 0.f, kb = 0.f, kh = 0.f;
#pragma unroll 8
        for (int t = 0; t < CW; t++) {
            const float keep = lane_bcast(keep_j, t), et = lane_bcast(eta_j, t);
            a *= keep;
            h *= et;
            beta = keep * beta + h;
            if (t == j) { ka = a; kb = beta; kh = h; }
        }
        cf.a[j] = j < L ? ka : 0.f;
        cf.beta[j] = j < L ? kb : 0.f;
        cf.h[j] = j < L ? kh : 0.f;
    } else if (w == 2) {
        if (!Bb) return;
        float b = 1.f;
#pragma unroll 16
        for (int t = 0; t < CW; t++) {
            const float et = lane_bcast(eta_j, t);
            b *= t > j ? et : 1.f;
            Bb[j * LDM + t] = (jv && t >= j && t < L) ? b : 0.f;
        }
    } else {
        if (!Rr) return;
        float rr = 1.f;
#pragma unroll 16
        for (int t = 0; t < CW; t++) {
            const float keep = lane_bcast(keep_j, t);
            rr *= t > j ? keep : 1.f;
            Rr[j * LDM + t] = (jv && t >= j && t < L) ? rr : 0.f;
        }
    }
}

}  // namespace mmt
}  // namespace nlh
