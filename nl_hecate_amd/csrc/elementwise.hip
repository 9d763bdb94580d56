// Glue kernels either side of the memory rules: activations, gating, bf16
// conversion, gate projections and their backward, row L2 normalisation, head
// transposes, Frobenius clamps.  All are HBM-bound streaming kernels: 16-byte
// accesses where the buffers allow it, one wave per row for row reductions
// (wave-level DPP sums, no LDS tree), grid sized to a few workgroups per CU.
#include <hip/hip_runtime.h>
#include <limits.h>
#include <math.h>

#include "../../include/nl_hecate_ffi.h"
#include "lane_ops.h"
#include "runtime.h"

namespace nlh {

constexpr int kEwThreads = 256;
constexpr int kMaxBlocks = 256 * 8;  // 8 workgroups per CU

static inline int ew_blocks(long long work_items) {
    long long b = (work_items + kEwThreads - 1) / kEwThreads;
    return (int)(b < 1 ? 1 : (b > kMaxBlocks ? kMaxBlocks : b));
}

static inline bool aligned16(const void *p) { return (((uintptr_t)p) & 15) == 0; }

// out[i] = f(i) over n elements; 4 elements per thread-iteration when VEC.
template <bool VEC, typename F>
__global__ void map_kernel(int n, F f) {
    const int stride = gridDim.x * blockDim.x;
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (VEC) {
        const int n4 = n >> 2;
        for (int j = i; j < n4; j += stride) f.vec4(j);
        for (int j = (n4 << 2) + i; j < n; j += stride) f.one(j);
    } else {
        for (; i < n; i += stride) f.one(i);
    }
}

template <typename F>
static void launch_map(int n, bool vec_ok, F f, const char *name) {
    if (n <= 0) return;
    if (vec_ok)
        hipLaunchKernelGGL((map_kernel<true, F>), dim3(ew_blocks((n + 3) / 4)), dim3(kEwThreads), 0, stream(), n, f);
    else
        hipLaunchKernelGGL((map_kernel<false, F>), dim3(ew_blocks(n)), dim3(kEwThreads), 0, stream(), n, f);
    check_launch(name);
}

__device__ __forceinline__ float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }
// softplus with the kernels' threshold (core/kernels/elementwise.cu:38-45)
__device__ __forceinline__ float softplusf_(float x) { return x > 20.0f ? x : logf(1.0f + expf(x)); }

// round-to-nearest-even f32 -> bf16 (NaN stays NaN), as __float2bfloat16
__device__ __forceinline__ unsigned short f32_to_bf16_rne(float f) {
    unsigned u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (unsigned short)((u >> 16) | 0x40);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (unsigned short)(u >> 16);
}
__device__ __forceinline__ float bf16_to_f32(unsigned short h) { return __uint_as_float(((unsigned)h) << 16); }

#define F4(p, j) (reinterpret_cast<const float4 *>(p)[j])
#define F4W(p, j) (reinterpret_cast<float4 *>(p)[j])

struct SigmoidF {
    const float *x; float *o;
    __device__ void one(int i) const { o[i] = sigmoidf_(x[i]); }
    __device__ void vec4(int j) const {
        float4 a = F4(x, j);
        F4W(o, j) = make_float4(sigmoidf_(a.x), sigmoidf_(a.y), sigmoidf_(a.z), sigmoidf_(a.w));
    }
};
struct SoftplusF {
    const float *x; float *o;
    __device__ void one(int i) const { o[i] = softplusf_(x[i]); }
    __device__ void vec4(int j) const {
        float4 a = F4(x, j);
        F4W(o, j) = make_float4(softplusf_(a.x), softplusf_(a.y), softplusf_(a.z), softplusf_(a.w));
    }
};
struct MulF {
    const float *a, *b; float *o;
    __device__ void one(int i) const { o[i] = a[i] * b[i]; }
    __device__ void vec4(int j) const {
        float4 x = F4(a, j), y = F4(b, j);
        F4W(o, j) = make_float4(x.x * y.x, x.y * y.y, x.z * y.z, x.w * y.w);
    }
};
struct GatingBwdF {  // d_a = d_out*b, d_b = d_out*a
    const float *d, *a, *b; float *da, *db;
    __device__ void one(int i) const { float g = d[i]; da[i] = g * b[i]; db[i] = g * a[i]; }
    __device__ void vec4(int j) const {
        float4 g = F4(d, j), x = F4(a, j), y = F4(b, j);
        F4W(da, j) = make_float4(g.x * y.x, g.y * y.y, g.z * y.z, g.w * y.w);
        F4W(db, j) = make_float4(g.x * x.x, g.y * x.y, g.z * x.z, g.w * x.w);
    }
};
struct SigmoidBwdF {  // d_x = d_gate * g * (1-g)
    const float *d, *g; float *o;
    __device__ static float f(float d, float g) { return d * g * (1.0f - g); }
    __device__ void one(int i) const { o[i] = f(d[i], g[i]); }
    __device__ void vec4(int j) const {
        float4 a = F4(d, j), b = F4(g, j);
        F4W(o, j) = make_float4(f(a.x, b.x), f(a.y, b.y), f(a.z, b.z), f(a.w, b.w));
    }
};
struct ToBf16F {
    const float *s; unsigned short *o;
    __device__ void one(int i) const { o[i] = f32_to_bf16_rne(s[i]); }
    __device__ void vec4(int j) const {
        float4 a = F4(s, j);
        ushort4 r;
        r.x = f32_to_bf16_rne(a.x); r.y = f32_to_bf16_rne(a.y);
        r.z = f32_to_bf16_rne(a.z); r.w = f32_to_bf16_rne(a.w);
        reinterpret_cast<ushort4 *>(o)[j] = r;
    }
};
struct FromBf16F {
    const unsigned short *s; float *o;
    __device__ void one(int i) const { o[i] = bf16_to_f32(s[i]); }
    __device__ void vec4(int j) const {
        ushort4 a = reinterpret_cast<const ushort4 *>(s)[j];
        F4W(o, j) = make_float4(bf16_to_f32(a.x), bf16_to_f32(a.y), bf16_to_f32(a.z), bf16_to_f32(a.w));
    }
};
struct SaxpyF {
    float alpha; const float *x; float *y;
    __device__ void one(int i) const { y[i] += alpha * x[i]; }
    __device__ void vec4(int j) const {
        float4 a = F4(x, j), b = F4(y, j);
        F4W(y, j) = make_float4(b.x + alpha * a.x, b.y + alpha * a.y, b.z + alpha * a.z, b.w + alpha * a.w);
    }
};
struct ClampF {
    float *x; float lo, hi;
    __device__ float f(float v) const { return fmaxf(lo, fminf(hi, v)); }
    __device__ void one(int i) const { x[i] = f(x[i]); }
    __device__ void vec4(int j) const {
        float4 a = F4(x, j);
        F4W(x, j) = make_float4(f(a.x), f(a.y), f(a.z), f(a.w));
    }
};
struct ClampMaskF {  // zero d_theta where theta sits on a clamp bound
    const float *t; float *d; float lo, hi;
    __device__ void one(int i) const { float v = t[i]; if (v <= lo || v >= hi) d[i] = 0.0f; }
    __device__ void vec4(int j) const {
        float4 a = F4(t, j), g = F4(d, j);
        if (a.x <= lo || a.x >= hi) g.x = 0.f;
        if (a.y <= lo || a.y >= hi) g.y = 0.f;
        if (a.z <= lo || a.z >= hi) g.z = 0.f;
        if (a.w <= lo || a.w >= hi) g.w = 0.f;
        F4W(d, j) = g;
    }
};

// ── per-token gate: act(k.w[:d] + v.w[d:] + bias), one wave per token ───────
__global__ void gate_compute_kernel(const float *__restrict__ k, const float *__restrict__ v,
                                    const float *__restrict__ w, const float *__restrict__ bias,
                                    float *__restrict__ out, int n_tok, int d, int activation) {
    const int lane = threadIdx.x & 63;
    const int wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int nwaves = (gridDim.x * blockDim.x) >> 6;
    const float b = bias[0];
    for (int t = wave; t < n_tok; t += nwaves) {
        const float *kr = k + (size_t)t * d, *vr = v + (size_t)t * d;
        float sum = 0.f;
        for (int i = lane; i < d; i += 64) sum += kr[i] * w[i] + vr[i] * w[d + i];
        sum = wave_allreduce(sum) + b;
        if (lane == 0) out[t] = activation == 0 ? sigmoidf_(sum) : softplusf_(sum);
    }
}

// ── the glue of one memory level's forward in one pass over the tokens ──────
// gpu_memory_forward (core/src/gpu_forward.rs:1197 ff.) runs, per level: row L2 norm of k and q, three
// gate projections on the normalised k and v, the head split of k, v, q and the per-head copies of the
// gates: eleven launches that each stream [n, d] tensors.  Here one wave owns a token: it normalises k
// and q in place (the backward needs them), writes the norms and the token-major gates, and emits the
// head-major tensors directly (as bf16 when KV16: what the matrix-core chunkwise rule takes).  Sums run
// over the same lane pattern as the separate kernels, so the results are the same numbers.
template <bool KV16>
__global__ void memory_inputs_fused_kernel(float *__restrict__ k, const float *__restrict__ v, float *__restrict__ q,
                                           const float *__restrict__ w_alpha, const float *__restrict__ b_alpha,
                                           const float *__restrict__ w_theta, const float *__restrict__ b_theta,
                                           const float *__restrict__ w_eta, const float *__restrict__ b_eta,
                                           float *__restrict__ k_norms, float *__restrict__ q_norms,
                                           float *__restrict__ alpha, float *__restrict__ theta, float *__restrict__ eta,
                                           void *__restrict__ kh, void *__restrict__ vh, void *__restrict__ qh,
                                           float *__restrict__ ah, float *__restrict__ th, float *__restrict__ eh,
                                           int bs, int s, int nh, int hd, float eps) {
    const int lane = threadIdx.x & 63, d = nh * hd;
    const int wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6, nwaves = (gridDim.x * blockDim.x) >> 6;
    const float ba = b_alpha[0], bt = b_theta[0], be = b_eta[0];
    for (int tok = wave; tok < bs * s; tok += nwaves) {
        float *kr = k + (size_t)tok * d, *qr = q + (size_t)tok * d;
        const float *vr = v + (size_t)tok * d;
        float sk = 0.f, sq = 0.f;
        for (int i = lane; i < d; i += 64) { const float a = kr[i], c = qr[i]; sk += a * a; sq += c * c; }
        const float kn = sqrtf(wave_allreduce(sk)), qn = sqrtf(wave_allreduce(sq));
        const float ki = 1.0f / fmaxf(kn, eps), qi = 1.0f / fmaxf(qn, eps);
        const int b = tok / s, t = tok % s;
        float ga = 0.f, gt = 0.f, ge = 0.f;
        for (int i = lane; i < d; i += 64) {
            const float kk = kr[i] * ki, qq = qr[i] * qi, vv = vr[i];
            kr[i] = kk;
            qr[i] = qq;
            ga += kk * w_alpha[i] + vv * w_alpha[d + i];
            gt += kk * w_theta[i] + vv * w_theta[d + i];
            ge += kk * w_eta[i] + vv * w_eta[d + i];
            const size_t o = (((size_t)b * nh + i / hd) * s + t) * hd + i % hd;
            if (KV16) {
                reinterpret_cast<__bf16 *>(kh)[o] = (__bf16)kk;
                reinterpret_cast<__bf16 *>(vh)[o] = (__bf16)vv;
                reinterpret_cast<__bf16 *>(qh)[o] = (__bf16)qq;
            } else {
                reinterpret_cast<float *>(kh)[o] = kk;
                reinterpret_cast<float *>(vh)[o] = vv;
                reinterpret_cast<float *>(qh)[o] = qq;
            }
        }
        const float al = sigmoidf_(wave_allreduce(ga) + ba), tht = softplusf_(wave_allreduce(gt) + bt);
        const float et = sigmoidf_(wave_allreduce(ge) + be);
        if (lane == 0) { k_norms[tok] = kn; q_norms[tok] = qn; alpha[tok] = al; theta[tok] = tht; eta[tok] = et; }
        for (int h = lane; h < nh; h += 64) {
            const size_t o = ((size_t)b * nh + h) * s + t;
            ah[o] = al; th[o] = tht; eh[o] = et;
        }
    }
}

// The glue of the level's backward between the rule and the projections: head sums of the gate
// gradients, head merge of d_k, d_v, d_q and the backward of the two row normalisations
// (gpu_memory_backward, core/src/gpu_backward.rs:2047 ff.: eight launches), one wave per token.
__global__ void memory_grads_fused_kernel(const float *__restrict__ dkh, const float *__restrict__ dvh,
                                          const float *__restrict__ dqh, const float *__restrict__ dah,
                                          const float *__restrict__ dth, const float *__restrict__ deh,
                                          const float *__restrict__ k_norm, const float *__restrict__ q_norm,
                                          const float *__restrict__ k_norms, const float *__restrict__ q_norms,
                                          float *__restrict__ dk_in, float *__restrict__ dv, float *__restrict__ dq_in,
                                          float *__restrict__ d_alpha, float *__restrict__ d_theta,
                                          float *__restrict__ d_eta, int bs, int s, int nh, int hd, float eps) {
    const int lane = threadIdx.x & 63, d = nh * hd;
    const int wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6, nwaves = (gridDim.x * blockDim.x) >> 6;
    for (int tok = wave; tok < bs * s; tok += nwaves) {
        const int b = tok / s, t = tok % s;
        if (lane < 3) {   // sum_heads: serial over the heads, as the separate kernel
            const float *src = lane == 0 ? dah : (lane == 1 ? dth : deh);
            float acc = 0.f;
            for (int h = 0; h < nh; h++) acc += src[((size_t)b * nh + h) * s + t];
            (lane == 0 ? d_alpha : (lane == 1 ? d_theta : d_eta))[tok] = acc;
        }
        const float *kx = k_norm + (size_t)tok * d, *qx = q_norm + (size_t)tok * d;
        float dk_dot = 0.f, dq_dot = 0.f;
        for (int i = lane; i < d; i += 64) {
            const size_t o = (((size_t)b * nh + i / hd) * s + t) * hd + i % hd;
            dk_dot += dkh[o] * kx[i];
            dq_dot += dqh[o] * qx[i];
        }
        dk_dot = wave_allreduce(dk_dot);
        dq_dot = wave_allreduce(dq_dot);
        const float kn = k_norms[tok], qn = q_norms[tok];
        const float ki = 1.0f / fmaxf(kn, eps), qi = 1.0f / fmaxf(qn, eps), inv_eps = 1.0f / eps;
        for (int i = lane; i < d; i += 64) {
            const size_t o = (((size_t)b * nh + i / hd) * s + t) * hd + i % hd;
            const float gk = dkh[o], gq = dqh[o];
            dk_in[(size_t)tok * d + i] = kn >= eps ? (gk - kx[i] * dk_dot) * ki : gk * inv_eps;
            dq_in[(size_t)tok * d + i] = qn >= eps ? (gq - qx[i] * dq_dot) * qi : gq * inv_eps;
            dv[(size_t)tok * d + i] = dvh[o];
        }
    }
}

// ── gate backward: d_w[2D] and d_b for alpha / theta / eta ──────────────────
// Stage 1: each workgroup owns a token range and every thread a set of the 2D
// columns; stage 2 sums the per-workgroup partials in a fixed order.
constexpr int kGateTok = 64;  // tokens per workgroup in stage 1

__global__ void gate_backward_stage1(const float *__restrict__ d_alpha, const float *__restrict__ alpha,
                                     const float *__restrict__ d_theta, const float *__restrict__ theta,
                                     const float *__restrict__ d_eta, const float *__restrict__ eta,
                                     const float *__restrict__ k, const float *__restrict__ v,
                                     float *__restrict__ part, int T, int D, int has_theta, int has_eta) {
    __shared__ float sg[3][kGateTok];
    const int t0 = blockIdx.x * kGateTok, tn = min(kGateTok, T - t0);
    const int twoD = 2 * D;
    for (int j = threadIdx.x; j < tn; j += blockDim.x) {
        const int t = t0 + j;
        const float a = alpha[t];
        sg[0][j] = d_alpha[t] * a * (1.0f - a);
        sg[1][j] = has_theta ? d_theta[t] * (1.0f - expf(-theta[t])) : 0.f;  // softplus' from its output
        float e = has_eta ? eta[t] : 0.f;
        sg[2][j] = has_eta ? d_eta[t] * e * (1.0f - e) : 0.f;
    }
    __syncthreads();
    float *pb = part + (size_t)blockIdx.x * 3 * (twoD + 1);
    for (int i = threadIdx.x; i < twoD; i += blockDim.x) {
        const float *x = i < D ? k + (size_t)t0 * D + i : v + (size_t)t0 * D + (i - D);
        float wa = 0.f, wt = 0.f, we = 0.f;
        for (int j = 0; j < tn; j++) {
            const float xv = x[(size_t)j * D];
            wa += sg[0][j] * xv;
            wt += sg[1][j] * xv;
            we += sg[2][j] * xv;
        }
        pb[i] = wa;
        pb[(twoD + 1) + i] = wt;
        pb[2 * (twoD + 1) + i] = we;
    }
    if (threadIdx.x < 3) {
        float s = 0.f;
        for (int j = 0; j < tn; j++) s += sg[threadIdx.x][j];
        pb[threadIdx.x * (twoD + 1) + twoD] = s;
    }
}

// 64 columns per workgroup, 4 thread groups each summing a quarter of the partial blocks,
// combined in a fixed order.
__global__ __launch_bounds__(256) void gate_backward_stage2(const float *__restrict__ part, int nblk, int twoD,
                                                            float *d_w_alpha, float *d_b_alpha, float *d_w_theta,
                                                            float *d_b_theta, float *d_w_eta, float *d_b_eta,
                                                            int has_theta, int has_eta) {
    __shared__ float red[4][3][64];
    const int col = threadIdx.x & 63, seg = threadIdx.x >> 6;
    const int i = blockIdx.x * 64 + col;
    float s[3] = {0.f, 0.f, 0.f};
    if (i <= twoD) {
        const int per = (nblk + 3) / 4, b0 = seg * per, b1 = min(nblk, b0 + per);
        for (int b = b0; b < b1; b++) {
            const float *pb = part + (size_t)b * 3 * (twoD + 1);
            s[0] += pb[i];
            s[1] += pb[(twoD + 1) + i];
            s[2] += pb[2 * (twoD + 1) + i];
        }
    }
    red[seg][0][col] = s[0]; red[seg][1][col] = s[1]; red[seg][2][col] = s[2];
    __syncthreads();
    if (seg != 0 || i > twoD) return;
#pragma unroll
    for (int g = 1; g < 4; g++) { s[0] += red[g][0][col]; s[1] += red[g][1][col]; s[2] += red[g][2][col]; }
    if (i < twoD) {
        d_w_alpha[i] = s[0];
        if (has_theta) d_w_theta[i] = s[1];
        if (has_eta) d_w_eta[i] = s[2];
    } else {
        d_b_alpha[0] = s[0];
        if (has_theta) d_b_theta[0] = s[1];
        if (has_eta) d_b_eta[0] = s[2];
    }
}

// ── row L2 normalisation, one wave per row ──────────────────────────────────
__global__ void l2_normalize_rows_kernel(float *__restrict__ x, float *__restrict__ norms, int n_rows,
                                         int d, float eps) {
    const int lane = threadIdx.x & 63;
    const int wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int nwaves = (gridDim.x * blockDim.x) >> 6;
    for (int r = wave; r < n_rows; r += nwaves) {
        float *row = x + (size_t)r * d;
        float s = 0.f;
        for (int j = lane; j < d; j += 64) { float v = row[j]; s += v * v; }
        const float norm = sqrtf(wave_allreduce(s));
        const float inv = 1.0f / fmaxf(norm, eps);
        if (lane == 0) norms[r] = norm;
        for (int j = lane; j < d; j += 64) row[j] *= inv;
    }
}

__global__ void l2_normalize_backward_kernel(const float *__restrict__ d_out, const float *__restrict__ xn,
                                             const float *__restrict__ norms, float *__restrict__ d_in,
                                             int n_rows, int d, float eps) {
    const int lane = threadIdx.x & 63;
    const int wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int nwaves = (gridDim.x * blockDim.x) >> 6;
    for (int r = wave; r < n_rows; r += nwaves) {
        const float *g = d_out + (size_t)r * d, *x = xn + (size_t)r * d;
        float *o = d_in + (size_t)r * d;
        const float norm = norms[r];
        float dot = 0.f;
        for (int j = lane; j < d; j += 64) dot += g[j] * x[j];
        dot = wave_allreduce(dot);
        if (norm >= eps) {
            const float inv = 1.0f / fmaxf(norm, eps);
            for (int j = lane; j < d; j += 64) o[j] = (g[j] - x[j] * dot) * inv;
        } else {  // forward was x/eps: linear
            const float inv_eps = 1.0f / eps;
            for (int j = lane; j < d; j += 64) o[j] = g[j] * inv_eps;
        }
    }
}

// ── head layout: [bs, s, nh, hd] <-> [bs, nh, s, hd] ───────────────────────
template <bool FORWARD, bool VEC>
__global__ void transpose_heads_kernel(const float *__restrict__ in, float *__restrict__ out,
                                       long long total, int s, int nh, int hd) {
    constexpr int V = VEC ? 4 : 1;
    const long long stride = (long long)gridDim.x * blockDim.x;
    const int hdv = hd / V;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total / V; i += stride) {
        // i indexes the [bs, s, nh, hd/V] order
        const int j = (int)(i % hdv);
        const int h = (int)((i / hdv) % nh);
        const long long bt = i / ((long long)hdv * nh);
        const int t = (int)(bt % s);
        const long long b = bt / s;
        const long long tok_major = i;
        const long long head_major = ((b * nh + h) * s + t) * hdv + j;
        if (VEC) {
            if (FORWARD) F4W(out, head_major) = F4(in, tok_major);
            else F4W(out, tok_major) = F4(in, head_major);
        } else {
            if (FORWARD) out[head_major] = in[tok_major];
            else out[tok_major] = in[head_major];
        }
    }
}

__global__ void broadcast_heads_kernel(const float *__restrict__ in, float *__restrict__ out,
                                       long long total, int s, int nh) {
    const long long stride = (long long)gridDim.x * blockDim.x;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int t = (int)(i % s);
        const long long b = i / ((long long)s * nh);
        out[i] = in[b * s + t];
    }
}

__global__ void sum_heads_kernel(const float *__restrict__ in, float *__restrict__ out, long long total,
                                 int s, int nh) {
    const long long stride = (long long)gridDim.x * blockDim.x;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int t = (int)(i % s);
        const long long b = i / s;
        float acc = 0.f;
        for (int h = 0; h < nh; h++) acc += in[(b * nh + h) * s + t];
        out[i] = acc;
    }
}

__global__ void broadcast_fill_kernel(float *__restrict__ dst, const float *__restrict__ src, int dd,
                                      int n_slots) {
    const long long b = blockIdx.y, t = blockIdx.x;
    const float *s = src + b * dd;
    float *o = dst + (b * n_slots + t) * dd;
    for (int i = threadIdx.x; i < dd; i += blockDim.x) o[i] = s[i];
}

// ── Frobenius clamp of carried-forward M: one workgroup per matrix ─────────
__global__ void m_norm_clamp_kernel(float *m, int dd, float m_norm_max) {
    __shared__ float part[kEwThreads / 64];
    float *mb = m + (size_t)blockIdx.x * dd;
    float s = 0.f;
    for (int i = threadIdx.x; i < dd; i += blockDim.x) { float v = mb[i]; s += v * v; }
    s = wave_allreduce(s);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = s;
    __syncthreads();
    float tot = 0.f;
    for (int w = 0; w < (int)(blockDim.x >> 6); w++) tot += part[w];
    const float fnorm = sqrtf(tot);
    if (fnorm > m_norm_max) {
        const float sc = m_norm_max / fnorm;
        for (int i = threadIdx.x; i < dd; i += blockDim.x) mb[i] *= sc;
    }
}

// |M k - v|_2 for one d x d matrix (core/kernels/elementwise.cu:297)
__global__ void dgd_delta_norm_kernel(const float *__restrict__ M, const float *__restrict__ k,
                                      const float *__restrict__ v, float *norm_out, int d) {
    __shared__ float part[kEwThreads / 64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    float sq = 0.f;
    for (int r = wave; r < d; r += nw) {
        float p = 0.f;
        for (int j = lane; j < d; j += 64) p += M[(size_t)r * d + j] * k[j];
        p = wave_allreduce(p);
        const float e = p - v[r];
        sq += e * e;  // identical in all lanes of the wave
    }
    if (lane == 0) part[wave] = sq;
    __syncthreads();
    if (threadIdx.x == 0) {
        float t = 0.f;
        for (int w = 0; w < nw; w++) t += part[w];
        norm_out[0] = sqrtf(t);
    }
}

}  // namespace nlh

using namespace nlh;

extern "C" {

void sigmoid_cuda(const float *x, float *out, int n) {
    launch_map(n, aligned16(x) && aligned16(out), SigmoidF{x, out}, "sigmoid");
}
void softplus_cuda(const float *x, float *out, int n) {
    launch_map(n, aligned16(x) && aligned16(out), SoftplusF{x, out}, "softplus");
}
void elemwise_mul_cuda(const float *a, const float *b, float *out, int n) {
    launch_map(n, aligned16(a) && aligned16(b) && aligned16(out), MulF{a, b, out}, "elemwise_mul");
}
void gating_backward_cuda(const float *d_out, const float *a, const float *b, float *d_a, float *d_b, int n) {
    launch_map(n, aligned16(d_out) && aligned16(a) && aligned16(b) && aligned16(d_a) && aligned16(d_b),
               GatingBwdF{d_out, a, b, d_a, d_b}, "gating_backward");
}
void sigmoid_backward_cuda(const float *d_gate, const float *gate, float *d_x, int n) {
    launch_map(n, aligned16(d_gate) && aligned16(gate) && aligned16(d_x), SigmoidBwdF{d_gate, gate, d_x},
               "sigmoid_backward");
}
void f32_to_bf16_cuda(const float *src, uint16_t *dst, int n) {
    launch_map(n, aligned16(src) && ((((uintptr_t)dst) & 7) == 0), ToBf16F{src, dst}, "f32_to_bf16");
}
void bf16_to_f32_cuda(const uint16_t *src, float *dst, int n) {
    launch_map(n, aligned16(dst) && ((((uintptr_t)src) & 7) == 0), FromBf16F{src, dst}, "bf16_to_f32");
}
// Operand packing of the split-bf16 GEMMs: row r of out is [hi(src0 .. src{count-1}) | lo(..) | hi(..)],
// 3*count*d bf16 values, where x = hi + lo with hi = bf16(x), lo = bf16(x - hi).
struct SplitSrcs { const float *p[4]; };
__global__ void split_pack_bf16_kernel(SplitSrcs src, int count, uint16_t *__restrict__ out, long long n, int d) {
    const int d4 = d / 4;
    const long long total = n * count * d4;
    for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < total;
         e += (long long)gridDim.x * blockDim.x) {
        const int c4 = (int)(e % d4), sidx = (int)((e / d4) % count);
        const long long r = e / ((long long)d4 * count);
        const float4 x = *reinterpret_cast<const float4 *>(src.p[sidx] + r * d + c4 * 4);
        const __bf16 h0 = (__bf16)x.x, h1 = (__bf16)x.y, h2 = (__bf16)x.z, h3 = (__bf16)x.w;
        const __bf16 l0 = (__bf16)(x.x - (float)h0), l1 = (__bf16)(x.y - (float)h1), l2 = (__bf16)(x.z - (float)h2),
                     l3 = (__bf16)(x.w - (float)h3);
        typedef __bf16 bf4 __attribute__((ext_vector_type(4)));
        uint16_t *o = out + r * (3LL * count * d) + (long long)sidx * d + c4 * 4;
        const bf4 hv = {h0, h1, h2, h3}, lv = {l0, l1, l2, l3};
        *reinterpret_cast<bf4 *>(o) = hv;
        *reinterpret_cast<bf4 *>(o + (long long)count * d) = lv;
        *reinterpret_cast<bf4 *>(o + 2LL * count * d) = hv;
    }
}
void split_pack_bf16_rocm(const float *const *srcs, int count, uint16_t *out, long long n, int d) {
    if (n <= 0) return;
    if (count < 1 || count > 4 || d <= 0 || d % 4) {
        fail("split_pack_bf16_rocm: count=%d must be 1..4 and d=%d a multiple of 4.", count, d);
        return;
    }
    SplitSrcs s{};
    for (int i = 0; i < count; i++) s.p[i] = srcs[i];
    hipLaunchKernelGGL(split_pack_bf16_kernel, dim3(ew_blocks(n * count * (d / 4))), dim3(kEwThreads), 0, stream(), s,
                       count, out, n, d);
    check_launch("split_pack_bf16_kernel");
}
void saxpy_cuda(float alpha, const float *x, float *y, int n) {
    launch_map(n, aligned16(x) && aligned16(y), SaxpyF{alpha, x, y}, "saxpy");
}
void clamp_f32_cuda(float *inout, int n, float lo, float hi) {
    launch_map(n, aligned16(inout), ClampF{inout, lo, hi}, "clamp_f32");
}
void theta_clamp_mask_cuda(const float *theta, float *d_theta, int n, float lo, float hi) {
    launch_map(n, aligned16(theta) && aligned16(d_theta), ClampMaskF{theta, d_theta, lo, hi}, "theta_clamp_mask");
}

void gate_compute_cuda(const float *k_mem, const float *v_mem, const float *w_gate,
                       const float *bias_ptr, float *gate_out, int seq_len, int d, int activation) {
    if (seq_len <= 0 || d <= 0) return;
    hipLaunchKernelGGL(gate_compute_kernel, dim3(ew_blocks((long long)seq_len * 64)), dim3(kEwThreads), 0,
                       stream(), k_mem, v_mem, w_gate, bias_ptr, gate_out, seq_len, d, activation);
    check_launch("gate_compute_kernel");
}

void memory_inputs_fused_rocm(float *k_mem, const float *v_mem, float *q_mem, const float *w_alpha,
                              const float *b_alpha, const float *w_theta, const float *b_theta, const float *w_eta,
                              const float *b_eta, float *k_norms, float *q_norms, float *alpha, float *theta,
                              float *eta, void *k_heads, void *v_heads, void *q_heads, float *alpha_heads,
                              float *theta_heads, float *eta_heads, int bs, int s, int nh, int hd, float eps,
                              int heads_bf16) {
    const long long n = (long long)bs * s;
    if (n <= 0 || nh <= 0 || hd <= 0) return;
    const dim3 grid(ew_blocks(n * 64)), blk(kEwThreads);
    if (heads_bf16)
        hipLaunchKernelGGL(memory_inputs_fused_kernel<true>, grid, blk, 0, stream(), k_mem, v_mem, q_mem, w_alpha,
                           b_alpha, w_theta, b_theta, w_eta, b_eta, k_norms, q_norms, alpha, theta, eta, k_heads, v_heads,
                           q_heads, alpha_heads, theta_heads, eta_heads, bs, s, nh, hd, eps);
    else
        hipLaunchKernelGGL(memory_inputs_fused_kernel<false>, grid, blk, 0, stream(), k_mem, v_mem, q_mem, w_alpha,
                           b_alpha, w_theta, b_theta, w_eta, b_eta, k_norms, q_norms, alpha, theta, eta, k_heads, v_heads,
                           q_heads, alpha_heads, theta_heads, eta_heads, bs, s, nh, hd, eps);
    check_launch("memory_inputs_fused_kernel");
}

void memory_grads_fused_rocm(const float *d_k_heads, const float *d_v_heads, const float *d_q_heads,
                             const float *d_alpha_heads, const float *d_theta_heads, const float *d_eta_heads,
                             const float *k_norm, const float *q_norm, const float *k_norms, const float *q_norms,
                             float *d_k_in, float *d_v, float *d_q_in, float *d_alpha, float *d_theta, float *d_eta,
                             int bs, int s, int nh, int hd, float eps) {
    const long long n = (long long)bs * s;
    if (n <= 0 || nh <= 0 || hd <= 0) return;
    hipLaunchKernelGGL(memory_grads_fused_kernel, dim3(ew_blocks(n * 64)), dim3(kEwThreads), 0, stream(), d_k_heads,
                       d_v_heads, d_q_heads, d_alpha_heads, d_theta_heads, d_eta_heads, k_norm, q_norm, k_norms, q_norms,
                       d_k_in, d_v, d_q_in, d_alpha, d_theta, d_eta, bs, s, nh, hd, eps);
    check_launch("memory_grads_fused_kernel");
}

void gate_backward_cuda(const float *d_alpha, const float *alpha, const float *d_theta,
                        const float *theta, const float *d_eta, const float *eta,
                        const float *k_mem, const float *v_mem,
                        float *d_w_alpha, float *d_b_alpha, float *d_w_theta, float *d_b_theta,
                        float *d_w_eta, float *d_b_eta, int T, int D, int has_theta, int has_eta) {
    const ErrorScope es;
    if (D <= 0) { fail("gate_backward_cuda: D=%d must be > 0.", D); return; }
    const int twoD = 2 * D;
    const int nblk = T > 0 ? ceil_div(T, kGateTok) : 0;
    float *part = scratch(10, (size_t)(nblk > 0 ? nblk : 1) * 3 * (twoD + 1) * sizeof(float));
    if (es.failed()) return;
    if (nblk > 0) {
        hipLaunchKernelGGL(gate_backward_stage1, dim3(nblk), dim3(kEwThreads), 0, stream(), d_alpha, alpha,
                           d_theta, theta, d_eta, eta, k_mem, v_mem, part, T, D, has_theta, has_eta);
        check_launch("gate_backward_stage1");
    }
    hipLaunchKernelGGL(gate_backward_stage2, dim3(ceil_div(twoD + 1, 64)), dim3(256), 0,
                       stream(), part, nblk, twoD, d_w_alpha, d_b_alpha, d_w_theta, d_b_theta, d_w_eta,
                       d_b_eta, has_theta, has_eta);
    check_launch("gate_backward_stage2");
}

void l2_normalize_rows_f32_cuda(float *x, float *norms, int n_rows, int d, float eps) {
    if (n_rows <= 0 || d <= 0) return;
    hipLaunchKernelGGL(l2_normalize_rows_kernel, dim3(ew_blocks((long long)n_rows * 64)), dim3(kEwThreads),
                       0, stream(), x, norms, n_rows, d, eps);
    check_launch("l2_normalize_rows_kernel");
}

void l2_normalize_backward_f32_cuda(const float *d_out, const float *x_norm, const float *norms,
                                    float *d_in, int n_rows, int d, float eps) {
    if (n_rows <= 0 || d <= 0) return;
    hipLaunchKernelGGL(l2_normalize_backward_kernel, dim3(ew_blocks((long long)n_rows * 64)),
                       dim3(kEwThreads), 0, stream(), d_out, x_norm, norms, d_in, n_rows, d, eps);
    check_launch("l2_normalize_backward_kernel");
}

void transpose_heads_f32_cuda(const float *input, float *output, int bs, int s, int nh, int hd, int forward) {
    const long long total = (long long)bs * s * nh * hd;
    if (total <= 0) return;
    const bool vec = (hd % 4 == 0) && aligned16(input) && aligned16(output);
    const dim3 grid(ew_blocks(vec ? total / 4 : total)), blk(kEwThreads);
    if (forward) {
        if (vec) hipLaunchKernelGGL((transpose_heads_kernel<true, true>), grid, blk, 0, stream(), input, output, total, s, nh, hd);
        else hipLaunchKernelGGL((transpose_heads_kernel<true, false>), grid, blk, 0, stream(), input, output, total, s, nh, hd);
    } else {
        if (vec) hipLaunchKernelGGL((transpose_heads_kernel<false, true>), grid, blk, 0, stream(), input, output, total, s, nh, hd);
        else hipLaunchKernelGGL((transpose_heads_kernel<false, false>), grid, blk, 0, stream(), input, output, total, s, nh, hd);
    }
    check_launch("transpose_heads_kernel");
}

void broadcast_heads_f32_cuda(const float *input, float *output, int bs, int s, int nh) {
    const long long total = (long long)bs * nh * s;
    if (total <= 0) return;
    hipLaunchKernelGGL(broadcast_heads_kernel, dim3(ew_blocks(total)), dim3(kEwThreads), 0, stream(), input,
                       output, total, s, nh);
    check_launch("broadcast_heads_kernel");
}

void sum_heads_f32_cuda(const float *input, float *output, int bs, int s, int nh) {
    const long long total = (long long)bs * s;
    if (total <= 0) return;
    hipLaunchKernelGGL(sum_heads_kernel, dim3(ew_blocks(total)), dim3(kEwThreads), 0, stream(), input,
                       output, total, s, nh);
    check_launch("sum_heads_kernel");
}

int broadcast_fill_f32_cuda(float *dst, const float *src, int dd, int n_slots, int n_batch) {
    if ((long long)n_batch * dd > INT_MAX) {
        fprintf(stderr, "broadcast_fill_f32_cuda: overflow (n_batch=%d, n_slots=%d, dd=%d)\n", n_batch,
                n_slots, dd);
        return 1;
    }
    if (dd <= 0 || n_slots <= 0 || n_batch <= 0) return 0;
    hipLaunchKernelGGL(broadcast_fill_kernel, dim3(n_slots, n_batch), dim3(dd < 256 ? dd : 256), 0, stream(),
                       dst, src, dd, n_slots);
    return hipGetLastError() == hipSuccess ? 0 : 2;
}

void m_norm_clamp_f32_cuda(float *m, int d, float m_norm_max) { m_norm_clamp_batch_f32_cuda(m, d, 1, m_norm_max); }

void m_norm_clamp_batch_f32_cuda(float *m, int d, int batch_size, float m_norm_max) {
    if (m_norm_max <= 0.0f || m_norm_max >= 1e30f) return;
    if (batch_size <= 0 || d <= 0) return;
    hipLaunchKernelGGL(m_norm_clamp_kernel, dim3(batch_size), dim3(kEwThreads), 0, stream(), m, d * d,
                       m_norm_max);
    check_launch("m_norm_clamp_kernel");
}

void dgd_delta_norm_cuda(const float *m, const float *k, const float *v, float *norm_out, int d) {
    if (d <= 0) return;
    hipLaunchKernelGGL(dgd_delta_norm_kernel, dim3(1), dim3(kEwThreads), 0, stream(), m, k, v, norm_out, d);
    check_launch("dgd_delta_norm_kernel");
}

}  // extern "C"
