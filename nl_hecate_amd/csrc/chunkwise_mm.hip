// Frozen-M0 chunkwise Titans / Delta rule in matrix form on the fp32 matrix
// cores (v_mfma_f32_32x32x2_f32), head size 64, chunks of up to 64 tokens.
//
// Semantics are those of core/kernels/titans_chunkwise_forward.cu and
// titans_chunkwise_backward.cu (errors of a chunk taken against the chunk-start
// M0; S and M then evolve per token; y_t reads M after token t's update) with
// error_clip and the M-norm projection off.  Because e_t = M0 k_t - v_t does not
// depend on the evolving state, the token recurrence inside a chunk is linear
// with scalar coefficients and unrolls into dense products.  With
//   r[j,t]  = prod_{i=j+1..t} (1-alpha_i)        bb[j,t] = prod_{i=j+1..t} eta_i
//   c[t,j]  = sum_{m=j..t} r[m,t] bb[j,m]        (weight of token j's rank-1 term in M_t)
//   a_t = prod_{i<=t}(1-alpha_i),  h_t = prod_{i<=t} eta_i,  beta_t = sum_{m<=t} r[m,t] h_m
// the state after token t is
//   M_t = a_t M0 + beta_t S0 - sum_{j<=t} theta_j c[t,j] e_j k_j^T
//   S_t = h_t S0           - sum_{j<=t} theta_j bb[j,t] e_j k_j^T
// so  Y = a.(Q M0^T) + beta.(Q S0^T) + (W . (Q K^T)) E,   W[t,j] = -theta_j c[t,j] (j <= t),
// and the end-of-chunk state is an affine map of (M0, S0) whose matrices depend
// on the chunk's K, V and gates only:
//   M' = M0 (a_L I + K^T diag(wM) K) + beta_L S0 - (V.wM)^T K,   wM_j = -theta_j c[L-1,j]
//   S' = M0 (        K^T diag(wS) K) + h_L    S0 - (V.wS)^T K,   wS_j = -theta_j bb[j,L-1]
// Three passes: (1) per chunk, in parallel, the four 64x64 matrices of that map;
// (2) a short sequential scan over chunks (two 32x64x64 products per step and
// row block) that writes the chunk-start states; (3) per chunk, in parallel, Y.
// The backward has the same shape: the adjoint scan uses the same (symmetric)
// matrices, and everything else is chunk-local.
//
// Delta rule = the same formulas with eta = 0 and S0 = 0.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/nl_hecate_ffi.h"
#include "rule_common.h"
#include "runtime.h"

namespace nlh {
namespace {

using f32x16 = __attribute__((ext_vector_type(16))) float;

constexpr int CW = 64;          // tokens per chunk tile
constexpr int HD = 64;          // head size
constexpr int LDM = 65;         // LDS row stride in floats (odd: conflict-free rows and columns)
constexpr int MAT = 64 * LDM;   // floats per 64x64 LDS matrix
constexpr int kThr = 256;       // 4 waves, one 32x32 output tile each

__device__ __forceinline__ float to_f32(float x) { return x; }
__device__ __forceinline__ float to_f32(uint16_t u) { return __uint_as_float((uint32_t)u << 16); }

// Stage a row-major [nrows <= 64][64] global tile into LDS; rows >= nrows are zero.
template <class T>
__device__ __forceinline__ void stage(float *dst, const T *src, int nrows) {
    for (int e = threadIdx.x * 4; e < 64 * 64; e += kThr * 4) {
        const int rr = e >> 6, cc = e & 63;
        float x0 = 0.f, x1 = 0.f, x2 = 0.f, x3 = 0.f;
        if (rr < nrows) {
            if constexpr (sizeof(T) == 4) {
                const float4 t = *reinterpret_cast<const float4 *>(src + rr * 64 + cc);
                x0 = t.x; x1 = t.y; x2 = t.z; x3 = t.w;
            } else {
                const uint2 t = *reinterpret_cast<const uint2 *>(src + rr * 64 + cc);
                x0 = __uint_as_float(t.x << 16); x1 = __uint_as_float(t.x & 0xffff0000u);
                x2 = __uint_as_float(t.y << 16); x3 = __uint_as_float(t.y & 0xffff0000u);
            }
        }
        float *p = dst + rr * LDM + cc;
        p[0] = x0; p[1] = x1; p[2] = x2; p[3] = x3;
    }
}

// One wave: acc (32x32) += sum_k a(m,k) b(k,n), m,n in [0,32), k in [0,K).
// Operand layout of v_mfma_f32_32x32x2_f32: lane l supplies A[l%32][l/32] and B[l/32][l%32].
template <class FA, class FB>
__device__ __forceinline__ void mma32(f32x16 &acc, int K, FA a, FB b) {
    const int l = threadIdx.x & 63, mn = l & 31, hf = l >> 5;
#pragma unroll 8
    for (int k = 0; k < K; k += 2)
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a(mn, k + hf), b(k + hf, mn), acc, 0, 0, 0);
}
// Accumulator element i of lane l is C[8*(i/4) + 4*(l/32) + i%4][l%32].
__device__ __forceinline__ int c_row(int i) { return 8 * (i >> 2) + 4 * ((threadIdx.x & 63) >> 5) + (i & 3); }
__device__ __forceinline__ int c_col() { return threadIdx.x & 31; }
__device__ __forceinline__ f32x16 zero16() {
    f32x16 z;
#pragma unroll
    for (int i = 0; i < 16; i++) z[i] = 0.f;
    return z;
}

// Gate coefficients of one chunk (L <= 64 tokens), all in LDS.
struct Coef {
    float al[CW], th[CW], et[CW];   // gates (eta = 0 for the Delta rule), zero beyond L
    float a[CW], beta[CW], h[CW];   // a_t, beta_t, h_t
    float cl[CW], bl[CW];           // c[L-1,j], bb[j,L-1]
};

__device__ __forceinline__ void load_gates(Coef &cf, const float *alpha, const float *theta, const float *eta,
                                           int L, bool has_s) {
    const int t = threadIdx.x;
    if (t < CW) {
        cf.al[t] = t < L ? alpha[t] : 0.f;
        cf.th[t] = t < L ? theta[t] : 0.f;
        cf.et[t] = (t < L && has_s) ? eta[t] : 0.f;
    }
}

// Column j of r, bb, c (thread j), optionally stored: Cc[t][j], Bb[j][t], Rr[j][t]
// (stride LDM; entries outside j <= t < L are zero), plus the vectors.
// Call after load_gates + barrier; needs a barrier afterwards.
__device__ __forceinline__ void coefficients(Coef &cf, int L, float *Cc, float *Bb, float *Rr) {
    const int j = threadIdx.x;
    if (j < CW) {
        float rr = 1.f, b = 1.f, cc = 1.f;
        for (int t = 0; t < CW; t++) {
            float vr = 0.f, vb = 0.f, vc = 0.f;
            if (t >= j && t < L && j < L) {
                if (t > j) {
                    const float keep = 1.f - cf.al[t];
                    rr *= keep;
                    b *= cf.et[t];
                    cc = keep * cc + b;
                }
                vr = rr; vb = b; vc = cc;
            }
            if (Cc) Cc[t * LDM + j] = vc;
            if (Bb) Bb[j * LDM + t] = vb;
            if (Rr) Rr[j * LDM + t] = vr;
        }
        cf.cl[j] = j < L ? cc : 0.f;
        cf.bl[j] = j < L ? b : 0.f;
    } else if (j == CW) {
        float a = 1.f, h = 1.f, beta = 0.f;
        for (int t = 0; t < CW; t++) {
            if (t < L) {
                const float keep = 1.f - cf.al[t];
                a *= keep;
                h *= cf.et[t];
                beta = keep * beta + h;
            }
            cf.a[t] = t < L ? a : 0.f;
            cf.beta[t] = t < L ? beta : 0.f;
            cf.h[t] = t < L ? h : 0.f;
        }
    }
}

// Per-chunk scratch written by the local passes and read by the scans:
//   loc  [chain][chunk][4][64*64]: T_a, T_b, C_1, C_2      locs [chain][chunk][4]: a_L, beta_L, h_L
constexpr size_t kLocMats = 4;

// ── pass 1 (forward) / shared with the backward: chunk-local matrices ───────
// T_a = a_L I + K^T diag(wM) K,  T_b = K^T diag(wS) K  (both symmetric);
// forward also C_1 = -(V.wM)^T K, C_2 = -(V.wS)^T K.
template <class TIn>
__global__ __launch_bounds__(kThr) void cw_local_fwd_kernel(const TIn *__restrict__ k, const TIn *__restrict__ v,
                                                            const float *__restrict__ alpha,
                                                            const float *__restrict__ theta,
                                                            const float *__restrict__ eta, float *__restrict__ loc,
                                                            float *__restrict__ locs, int s, int C, int nc,
                                                            int has_s) {
    __shared__ float Ks[MAT], Vs[MAT];
    __shared__ Coef cf;
    __shared__ float wM[CW], wS[CW];
    const int chain = blockIdx.x / nc, ci = blockIdx.x % nc, t0 = ci * C, L = min(C, s - t0);
    const size_t tok = (size_t)chain * s + t0;
    stage(Ks, k + tok * HD, L);
    stage(Vs, v + tok * HD, L);
    load_gates(cf, alpha + tok, theta + tok, eta + tok, L, has_s != 0);
    __syncthreads();
    coefficients(cf, L, nullptr, nullptr, nullptr);
    __syncthreads();
    if (threadIdx.x < CW) {
        wM[threadIdx.x] = -cf.th[threadIdx.x] * cf.cl[threadIdx.x];
        wS[threadIdx.x] = -cf.th[threadIdx.x] * cf.bl[threadIdx.x];
    }
    const float aL = cf.a[L - 1], betaL = cf.beta[L - 1], hL = cf.h[L - 1];
    if (threadIdx.x == 0) {
        float *sc = locs + ((size_t)chain * nc + ci) * 4;
        sc[0] = aL; sc[1] = betaL; sc[2] = hL; sc[3] = 0.f;
    }
    __syncthreads();
    const int w = threadIdx.x >> 6, m0 = 32 * (w >> 1), n0 = 32 * (w & 1);
    float *out = loc + ((size_t)chain * nc + ci) * kLocMats * HD * HD;
    auto bK = [&](int kk, int n) { return Ks[kk * LDM + n0 + n]; };
#pragma unroll 1
    for (int o = 0; o < 4; o++) {
        const float *Am = o < 2 ? Ks : Vs;
        const float *wv = (o & 1) ? wS : wM;
        f32x16 acc = zero16();
        mma32(acc, 64, [&](int m, int kk) { return Am[kk * LDM + m0 + m] * wv[kk]; }, bK);
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int row = m0 + c_row(i), col = n0 + c_col();
            float x = o < 2 ? acc[i] : -acc[i];
            if (o == 0 && row == col) x += aL;
            out[(size_t)o * HD * HD + row * HD + col] = x;
        }
    }
}

// ── pass 2: scan over chunks, one workgroup per (chain, 32-row block) ────────
// FWD:  X1' = X1 T_a + s1 X2 + C_1,  X2' = X1 T_b + s2 X2 + C_2,  (s1, s2) = (beta_L, h_L)
//       states[chain][c+1] = f(states[chain][c]), slot 0 = initial state
// BWD:  X1' = X1 T_a + X2 T_b + C_1, X2' = s1 X1 + s2 X2 + C_2
//       states[chain][c] = g(states[chain][c+1]), slot nc = 0
template <bool FWD>
__global__ __launch_bounds__(kThr) void cw_scan_kernel(const float *__restrict__ init1,
                                                       const float *__restrict__ init2,
                                                       const float *__restrict__ loc,
                                                       const float *__restrict__ locs, float *__restrict__ st1,
                                                       float *__restrict__ st2, int nc, int has_s) {
    __shared__ float X1[32 * LDM], X2[32 * LDM], Ta[MAT], Tb[MAT], part[2][32 * 33];
    const int chain = blockIdx.x >> 1, r0 = 32 * (blockIdx.x & 1);
    const int w = threadIdx.x >> 6, n0 = 32 * (w & 1), which = w >> 1;
    float *s1p = st1 + (size_t)chain * (nc + 1) * HD * HD, *s2p = st2 ? st2 + (size_t)chain * (nc + 1) * HD * HD : nullptr;
    // initial state of this row block
    for (int e = threadIdx.x; e < 32 * 64; e += kThr) {
        const int rr = e >> 6, cc = e & 63;
        float x1 = 0.f, x2 = 0.f;
        if (FWD) {
            x1 = init1[(size_t)chain * HD * HD + (r0 + rr) * HD + cc];
            if (has_s) x2 = init2[(size_t)chain * HD * HD + (r0 + rr) * HD + cc];
        }
        X1[rr * LDM + cc] = x1; X2[rr * LDM + cc] = x2;
        const size_t slot = FWD ? 0 : nc;
        s1p[slot * HD * HD + (r0 + rr) * HD + cc] = x1;
        if (s2p) s2p[slot * HD * HD + (r0 + rr) * HD + cc] = x2;
    }
    for (int step = 0; step < nc; step++) {
        const int ci = FWD ? step : nc - 1 - step;
        const float *lc = loc + ((size_t)chain * nc + ci) * kLocMats * HD * HD;
        const float *sc = locs + ((size_t)chain * nc + ci) * 4;
        __syncthreads();  // previous step's readers of Ta/Tb and writers of X1/X2 are done
        stage(Ta, lc, 64);
        stage(Tb, lc + HD * HD, 64);
        const float s1 = sc[1], s2 = sc[2];
        __syncthreads();
        f32x16 acc = zero16();
        float out[16];
        if (FWD) {
            const float *T = which ? Tb : Ta;
            mma32(acc, 64, [&](int m, int kk) { return X1[m * LDM + kk]; },
                  [&](int kk, int n) { return T[kk * LDM + n0 + n]; });
            const float *Cm = lc + (2 + which) * HD * HD;
            const float sx = which ? s2 : s1;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int row = c_row(i), col = n0 + c_col();
                out[i] = acc[i] + sx * X2[row * LDM + col] + Cm[(r0 + row) * HD + col];
            }
        } else {
            const float *Xs = which ? X2 : X1;
            const float *T = which ? Tb : Ta;
            mma32(acc, 64, [&](int m, int kk) { return Xs[m * LDM + kk]; },
                  [&](int kk, int n) { return T[kk * LDM + n0 + n]; });
            if (which) {
#pragma unroll
                for (int i = 0; i < 16; i++) part[w & 1][c_row(i) * 33 + c_col()] = acc[i];
                const float *Cm = lc + 3 * HD * HD;
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const int row = c_row(i), col = n0 + c_col();
                    out[i] = s1 * X1[row * LDM + col] + s2 * X2[row * LDM + col] + Cm[(r0 + row) * HD + col];
                }
            }
        }
        __syncthreads();  // all reads of the old X1/X2 are done; partial products are in LDS
        if (!FWD && !which) {
            const float *Cm = lc + 2 * HD * HD;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int row = c_row(i), col = n0 + c_col();
                out[i] = acc[i] + part[w & 1][row * 33 + c_col()] + Cm[(r0 + row) * HD + col];
            }
        }
        float *Xd = which ? X2 : X1;
        float *gd = which ? s2p : s1p;
        const size_t slot = FWD ? ci + 1 : ci;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int row = c_row(i), col = n0 + c_col();
            Xd[row * LDM + col] = out[i];
            if (gd) gd[slot * HD * HD + (r0 + row) * HD + col] = out[i];
        }
    }
}

// ── pass 3 (forward): outputs of one chunk ──────────────────────────────────
template <class TIn>
__global__ __launch_bounds__(kThr) void cw_out_fwd_kernel(const TIn *__restrict__ k, const TIn *__restrict__ v,
                                                          const TIn *__restrict__ q,
                                                          const float *__restrict__ alpha,
                                                          const float *__restrict__ theta,
                                                          const float *__restrict__ eta,
                                                          const float *__restrict__ m_states,
                                                          const float *__restrict__ s_states,
                                                          float *__restrict__ y, int s, int C, int nc, int has_s) {
    extern __shared__ float smem[];
    float *Ks = smem, *Qs = Ks + MAT, *Es = Qs + MAT, *Ms = Es + MAT, *Ss = Ms + MAT, *Cc = Ss + MAT, *Pw = Cc + MAT;
    __shared__ Coef cf;
    const int chain = blockIdx.x / nc, ci = blockIdx.x % nc, t0 = ci * C, L = min(C, s - t0);
    const size_t tok = (size_t)chain * s + t0;
    stage(Ks, k + tok * HD, L);
    stage(Qs, q + tok * HD, L);
    stage(Es, v + tok * HD, L);
    stage(Ms, m_states + ((size_t)chain * (nc + 1) + ci) * HD * HD, 64);
    if (has_s) stage(Ss, s_states + ((size_t)chain * (nc + 1) + ci) * HD * HD, 64);
    load_gates(cf, alpha + tok, theta + tok, eta + tok, L, has_s != 0);
    __syncthreads();
    coefficients(cf, L, Cc, nullptr, nullptr);
    __syncthreads();
    const int w = threadIdx.x >> 6, m0 = 32 * (w >> 1), n0 = 32 * (w & 1);
    {
        // E[t][i] = sum_k K[t][k] M0[i][k] - V[t][i]   (in place over V: tiles are disjoint per wave)
        f32x16 e = zero16(), p = zero16();
        mma32(e, 64, [&](int m, int kk) { return Ks[(m0 + m) * LDM + kk]; },
              [&](int kk, int n) { return Ms[(n0 + n) * LDM + kk]; });
        // P[t][j] = sum_k Q[t][k] K[j][k]
        mma32(p, 64, [&](int m, int kk) { return Qs[(m0 + m) * LDM + kk]; },
              [&](int kk, int n) { return Ks[(n0 + n) * LDM + kk]; });
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int row = m0 + c_row(i), col = n0 + c_col();
            Es[row * LDM + col] = e[i] - Es[row * LDM + col];
            // W[t][j] = -theta_j c[t][j]; Cc is zero outside j <= t < L
            Pw[row * LDM + col] = -cf.th[col] * Cc[row * LDM + col] * p[i];
        }
    }
    __syncthreads();
    f32x16 y0 = zero16(), y1 = zero16(), y2 = zero16();
    mma32(y0, 64, [&](int m, int kk) { return Qs[(m0 + m) * LDM + kk]; },
          [&](int kk, int n) { return Ms[(n0 + n) * LDM + kk]; });
    if (has_s)
        mma32(y1, 64, [&](int m, int kk) { return Qs[(m0 + m) * LDM + kk]; },
              [&](int kk, int n) { return Ss[(n0 + n) * LDM + kk]; });
    mma32(y2, 64, [&](int m, int kk) { return Pw[(m0 + m) * LDM + kk]; },
          [&](int kk, int n) { return Es[kk * LDM + n0 + n]; });
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const int row = m0 + c_row(i), col = n0 + c_col();
        if (row < L) y[(tok + row) * HD + col] = cf.a[row] * y0[i] + cf.beta[row] * y1[i] + y2[i];
    }
}

constexpr size_t kOutFwdLds = 7 * MAT * sizeof(float);

struct Scratch {
    float *loc, *locs;
};
Scratch local_scratch(int batch, int nc) {
    Scratch sc;
    sc.loc = scratch(3, (size_t)batch * nc * kLocMats * HD * HD * sizeof(float));
    sc.locs = scratch(4, (size_t)batch * nc * 4 * sizeof(float));
    return sc;
}

bool check_mm_args(const char *fn, int seq_len, int d, int batch, int chunk_size) {
    if (seq_len <= 0 || batch <= 0) { fail("%s: seq_len and batch_size must be positive", fn); return false; }
    if (d != HD) { fail("%s: d=%d unsupported (the matrix-core path is built for d=64)", fn, d); return false; }
    if (chunk_size < 1 || chunk_size > CW) {
        fail("%s: chunk_size=%d unsupported (1..64)", fn, chunk_size);
        return false;
    }
    return true;
}

template <class TIn>
void forward_mm(const char *fn, const TIn *k, const TIn *v, const TIn *q, const float *alpha, const float *theta,
                const float *eta, const float *m_initial, const float *s_initial, float *m_states, float *s_states,
                float *y, int seq_len, int d, int batch, int chunk_size, bool has_s) {
    if (!check_mm_args(fn, seq_len, d, batch, chunk_size)) return;
    const int nc = ceil_div(seq_len, chunk_size);
    Scratch sc = local_scratch(batch, nc);
    if (failed()) return;
    static bool attr_set = false;
    if (!attr_set) {
        check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(cw_out_fwd_kernel<float>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)kOutFwdLds), "LDS size");
        check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(cw_out_fwd_kernel<uint16_t>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)kOutFwdLds), "LDS size");
        attr_set = true;
    }
    hipLaunchKernelGGL((cw_local_fwd_kernel<TIn>), dim3(batch * nc), dim3(kThr), 0, stream(), k, v, alpha, theta,
                       eta, sc.loc, sc.locs, seq_len, chunk_size, nc, (int)has_s);
    check_launch("cw_local_fwd_kernel");
    hipLaunchKernelGGL((cw_scan_kernel<true>), dim3(batch * 2), dim3(kThr), 0, stream(), m_initial, s_initial,
                       sc.loc, sc.locs, m_states, has_s ? s_states : nullptr, nc, (int)has_s);
    check_launch("cw_scan_kernel");
    hipLaunchKernelGGL((cw_out_fwd_kernel<TIn>), dim3(batch * nc), dim3(kThr), kOutFwdLds, stream(), k, v, q, alpha,
                       theta, eta, m_states, s_states, y, seq_len, chunk_size, nc, (int)has_s);
    check_launch("cw_out_fwd_kernel");
}

}  // namespace
}  // namespace nlh

using namespace nlh;

extern "C" void titans_chunkwise_forward_bf16_rocm(const uint16_t *k_mem, const uint16_t *v_mem,
                                                   const uint16_t *q_mem, const float *alpha, const float *theta,
                                                   const float *eta, const float *m_initial,
                                                   const float *s_initial, float *m_chunk_states,
                                                   float *s_chunk_states, float *y, int seq_len, int d,
                                                   int batch_size, int chunk_size) {
    forward_mm<uint16_t>("titans_chunkwise_forward_bf16_rocm", k_mem, v_mem, q_mem, alpha, theta, eta, m_initial,
                         s_initial, m_chunk_states, s_chunk_states, y, seq_len, d, batch_size, chunk_size, true);
}

extern "C" void titans_chunkwise_forward_mm_f32_rocm(const float *k_mem, const float *v_mem, const float *q_mem,
                                                     const float *alpha, const float *theta, const float *eta,
                                                     const float *m_initial, const float *s_initial,
                                                     float *m_chunk_states, float *s_chunk_states, float *y,
                                                     int seq_len, int d, int batch_size, int chunk_size) {
    forward_mm<float>("titans_chunkwise_forward_mm_f32_rocm", k_mem, v_mem, q_mem, alpha, theta, eta, m_initial,
                      s_initial, m_chunk_states, s_chunk_states, y, seq_len, d, batch_size, chunk_size, true);
}
