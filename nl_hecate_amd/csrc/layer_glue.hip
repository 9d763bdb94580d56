// The glue of one layer step around the rule kernels and the library GEMMs, written so that every
// [tokens, d] tensor is read once and written once: operand packing for the split-bf16 GEMMs with
// row strides and column offsets (several producers fill column slabs of ONE operand, so a group of
// projections is one GEMM), the level's forward glue on strided projection outputs, and the level's
// backward glue that emits the packed GEMM operand and the gate weight partial sums directly.
// HBM-bound streaming kernels: one wave per token, a token's rows in registers as float4.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>

#include "../../include/nl_hecate_ffi.h"
#include "lane_ops.h"
#include "runtime.h"

namespace nlh {

namespace {

constexpr int kThr = 256;
constexpr int kWavesWg = kThr / 64;
typedef __bf16 bf4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float sigmoid_(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float softplus_(float x) { return x > 20.0f ? x : logf(1.0f + expf(x)); }
__device__ __forceinline__ float dot4(const float4 &a, const float4 &b) {
    return a.x * b.x + a.y * b.y + a.z * b.z + a.w * b.w;
}
__device__ __forceinline__ void fma4(float4 &acc, float s, const float4 &x) {
    acc.x = fmaf(s, x.x, acc.x); acc.y = fmaf(s, x.y, acc.y); acc.z = fmaf(s, x.z, acc.z); acc.w = fmaf(s, x.w, acc.w);
}
__device__ __forceinline__ bf4 hi4(const float4 &x) { return bf4{(__bf16)x.x, (__bf16)x.y, (__bf16)x.z, (__bf16)x.w}; }
__device__ __forceinline__ bf4 lo4(const float4 &x, const bf4 &h) {
    return bf4{(__bf16)(x.x - (float)h[0]), (__bf16)(x.y - (float)h[1]), (__bf16)(x.z - (float)h[2]),
               (__bf16)(x.w - (float)h[3])};
}
// x = hi + lo in bf16; hi goes to two column positions of the row (one when off_h2 < 0), lo to one
__device__ __forceinline__ void store_split(uint16_t *row, long long col, long long off_h1, long long off_l,
                                            long long off_h2, const float4 &x) {
    const bf4 h = hi4(x), l = lo4(x, h);
    *reinterpret_cast<bf4 *>(row + off_h1 + col) = h;
    *reinterpret_cast<bf4 *>(row + off_l + col) = l;
    if (off_h2 >= 0) *reinterpret_cast<bf4 *>(row + off_h2 + col) = h;
}

struct SplitSrcs4 { const float *p[4]; };

__global__ void split_pack_ld_kernel(SplitSrcs4 src, int count, long long src_ld, uint16_t *__restrict__ out,
                                     long long n, int d, long long out_ld, long long off_h1, long long off_l,
                                     long long off_h2) {
    const int d4 = d / 4;
    const long long total = n * count * d4;
    for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < total;
         e += (long long)gridDim.x * blockDim.x) {
        const int c4 = (int)(e % d4), sidx = (int)((e / d4) % count);
        const long long r = e / ((long long)d4 * count);
        const float4 x = *reinterpret_cast<const float4 *>(src.p[sidx] + r * src_ld + c4 * 4);
        store_split(out + r * out_ld, (long long)sidx * d + c4 * 4, off_h1, off_l, off_h2, x);
    }
}

// pack [rows, d] fp32 -> wb [rows, 3d] = (Wh | Wl | Wh) per row and wstack [3 * rows_stack, d] =
// (Wh[:rows_stack] ; Wh[:rows_stack] ; Wl[:rows_stack])
__global__ void split_pack_weights_kernel(const float *__restrict__ pack, int rows, int rows_stack, int d,
                                          uint16_t *__restrict__ wb, uint16_t *__restrict__ wstack) {
    const int d4 = d / 4;
    const long long total = (long long)rows * d4;
    for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < total;
         e += (long long)gridDim.x * blockDim.x) {
        const int c = (int)(e % d4) * 4;
        const long long r = e / d4;
        const float4 x = *reinterpret_cast<const float4 *>(pack + r * d + c);
        const bf4 h = hi4(x), l = lo4(x, h);
        uint16_t *o = wb + r * 3 * d + c;
        *reinterpret_cast<bf4 *>(o) = h;
        *reinterpret_cast<bf4 *>(o + d) = l;
        *reinterpret_cast<bf4 *>(o + 2 * d) = h;
        if (r < rows_stack) {
            *reinterpret_cast<bf4 *>(wstack + r * d + c) = h;
            *reinterpret_cast<bf4 *>(wstack + ((long long)rows_stack + r) * d + c) = h;
            *reinterpret_cast<bf4 *>(wstack + (2LL * rows_stack + r) * d + c) = l;
        }
    }
}

// Forward glue of one level on projection outputs with row stride ld (columns of a wider GEMM output):
// k and q normalised (in place when write_back; otherwise the raw rows stay and the backward divides by the
// stored norms again), gates, head-major bf16 / fp32 k, v, q and per-head gate copies.
// NIT float4 per lane and tensor: d <= 256 * NIT.
template <int NIT, bool KV16>
__global__ __launch_bounds__(kThr) void level_inputs_kernel(
    float *__restrict__ k, const float *__restrict__ v, float *__restrict__ q, long long ld,
    const float *__restrict__ w_alpha, const float *__restrict__ b_alpha, const float *__restrict__ w_theta,
    const float *__restrict__ b_theta, const float *__restrict__ w_eta, const float *__restrict__ b_eta,
    float *__restrict__ k_norms, float *__restrict__ q_norms, float *__restrict__ alpha, float *__restrict__ theta,
    float *__restrict__ eta, void *__restrict__ kh, void *__restrict__ vh, void *__restrict__ qh,
    float *__restrict__ ah, float *__restrict__ th, float *__restrict__ eh, int bs, int s, int nh, int hd, float eps,
    int write_back) {
    const int lane = threadIdx.x & 63, d = nh * hd, d4 = d / 4;
    const int wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6, nwaves = (gridDim.x * blockDim.x) >> 6;
    const float ba = b_alpha[0], bt = b_theta[0], be = b_eta[0];
    float4 wa[2][NIT], wt[2][NIT], we[2][NIT];
#pragma unroll
    for (int it = 0; it < NIT; it++) {
        const int i4 = lane + 64 * it;
        const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
        const bool on = i4 < d4;
        wa[0][it] = on ? *reinterpret_cast<const float4 *>(w_alpha + 4 * i4) : z;
        wa[1][it] = on ? *reinterpret_cast<const float4 *>(w_alpha + d + 4 * i4) : z;
        wt[0][it] = on ? *reinterpret_cast<const float4 *>(w_theta + 4 * i4) : z;
        wt[1][it] = on ? *reinterpret_cast<const float4 *>(w_theta + d + 4 * i4) : z;
        we[0][it] = on ? *reinterpret_cast<const float4 *>(w_eta + 4 * i4) : z;
        we[1][it] = on ? *reinterpret_cast<const float4 *>(w_eta + d + 4 * i4) : z;
    }
    for (int tok = wave; tok < bs * s; tok += nwaves) {
        float *kr = k + (size_t)tok * ld, *qr = q + (size_t)tok * ld;
        const float *vr = v + (size_t)tok * ld;
        float4 kk[NIT], qq[NIT], vv[NIT];
        float sk = 0.f, sq = 0.f;
#pragma unroll
        for (int it = 0; it < NIT; it++) {
            const int i4 = lane + 64 * it;
            kk[it] = qq[it] = vv[it] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (i4 < d4) {
                kk[it] = *reinterpret_cast<const float4 *>(kr + 4 * i4);
                qq[it] = *reinterpret_cast<const float4 *>(qr + 4 * i4);
                vv[it] = *reinterpret_cast<const float4 *>(vr + 4 * i4);
            }
            sk += dot4(kk[it], kk[it]);
            sq += dot4(qq[it], qq[it]);
        }
        const float kn = sqrtf(wave_allreduce(sk)), qn = sqrtf(wave_allreduce(sq));
        const float ki = 1.0f / fmaxf(kn, eps), qi = 1.0f / fmaxf(qn, eps);
        const int b = tok / s, t = tok % s;
        float ga = 0.f, gt = 0.f, ge = 0.f;
#pragma unroll
        for (int it = 0; it < NIT; it++) {
            const int i4 = lane + 64 * it;
            if (i4 >= d4) continue;
            kk[it].x *= ki; kk[it].y *= ki; kk[it].z *= ki; kk[it].w *= ki;
            qq[it].x *= qi; qq[it].y *= qi; qq[it].z *= qi; qq[it].w *= qi;
            if (write_back) {
                *reinterpret_cast<float4 *>(kr + 4 * i4) = kk[it];
                *reinterpret_cast<float4 *>(qr + 4 * i4) = qq[it];
            }
            ga += dot4(kk[it], wa[0][it]) + dot4(vv[it], wa[1][it]);
            gt += dot4(kk[it], wt[0][it]) + dot4(vv[it], wt[1][it]);
            ge += dot4(kk[it], we[0][it]) + dot4(vv[it], we[1][it]);
            const int i = 4 * i4;
            const size_t o = (((size_t)b * nh + i / hd) * s + t) * hd + i % hd;
            if (KV16) {
                *reinterpret_cast<bf4 *>(reinterpret_cast<uint16_t *>(kh) + o) = hi4(kk[it]);
                *reinterpret_cast<bf4 *>(reinterpret_cast<uint16_t *>(vh) + o) = hi4(vv[it]);
                *reinterpret_cast<bf4 *>(reinterpret_cast<uint16_t *>(qh) + o) = hi4(qq[it]);
            } else {
                *reinterpret_cast<float4 *>(reinterpret_cast<float *>(kh) + o) = kk[it];
                *reinterpret_cast<float4 *>(reinterpret_cast<float *>(vh) + o) = vv[it];
                *reinterpret_cast<float4 *>(reinterpret_cast<float *>(qh) + o) = qq[it];
            }
        }
        const float al = sigmoid_(wave_allreduce(ga) + ba), tht = softplus_(wave_allreduce(gt) + bt);
        const float et = sigmoid_(wave_allreduce(ge) + be);
        if (lane == 0) { k_norms[tok] = kn; q_norms[tok] = qn; alpha[tok] = al; theta[tok] = tht; eta[tok] = et; }
        for (int h = lane; h < nh; h += 64) {
            const size_t o = ((size_t)b * nh + h) * s + t;
            ah[o] = al; th[o] = tht; eh[o] = et;
        }
    }
}

// Backward glue of one level.  Per token: head sums of the gate gradients, head merge of d_k, d_v, d_q,
// backward of the two row normalisations; the three token-major gradients go out as the split-bf16 GEMM
// operand (d_k at column 0, d_v at d, d_q at 2d of the slab; hi twice, lo once), never as fp32.  The
// gate projections' weight and bias gradients (sums over tokens of dpre x [k | v]) are accumulated per
// wave in registers and leave as one partial row per workgroup.
template <int NIT>
__global__ __launch_bounds__(kThr) void level_grads_packed_kernel(
    const float *__restrict__ dkh, const float *__restrict__ dvh, const float *__restrict__ dqh,
    const float *__restrict__ dah, const float *__restrict__ dth, const float *__restrict__ deh,
    const float *__restrict__ kx, const float *__restrict__ vx, const float *__restrict__ qx, long long ld,
    const float *__restrict__ k_norms, const float *__restrict__ q_norms, const float *__restrict__ alpha,
    const float *__restrict__ theta, const float *__restrict__ eta, uint16_t *__restrict__ P, long long p_ld,
    long long off_h1, long long off_l, long long off_h2, float *__restrict__ part, int bs, int s, int nh, int hd,
    float eps, int inputs_raw) {
    extern __shared__ float red[];   // [3][2d + 1]
    const int lane = threadIdx.x & 63, wave_l = threadIdx.x >> 6, d = nh * hd, d4 = d / 4;
    const int wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6, nwaves = (gridDim.x * blockDim.x) >> 6;
    const float inv_eps = 1.0f / eps;
    float4 acc[3][2][NIT];
    float accb[3] = {0.f, 0.f, 0.f};
#pragma unroll
    for (int g = 0; g < 3; g++)
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int it = 0; it < NIT; it++) acc[g][h][it] = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int tok = wave; tok < bs * s; tok += nwaves) {
        const int b = tok / s, t = tok % s;
        float da = 0.f, dt = 0.f, de = 0.f;
        for (int h = lane; h < nh; h += 64) {
            const size_t o = ((size_t)b * nh + h) * s + t;
            da += dah[o]; dt += dth[o]; de += deh[o];
        }
        da = wave_allreduce(da); dt = wave_allreduce(dt); de = wave_allreduce(de);
        {   // through the gate activations, from their outputs
            const float a = alpha[tok], th = theta[tok], e = eta[tok];
            da *= a * (1.0f - a);
            dt *= 1.0f - expf(-th);
            de *= e * (1.0f - e);
        }
        accb[0] += da; accb[1] += dt; accb[2] += de;
        const float *kr = kx + (size_t)tok * ld, *qr = qx + (size_t)tok * ld, *vr = vx + (size_t)tok * ld;
        const float kn = k_norms[tok], qn = q_norms[tok];
        const float ki = 1.0f / fmaxf(kn, eps), qi = 1.0f / fmaxf(qn, eps);
        float4 kk[NIT], qq[NIT], gk[NIT], gv[NIT], gq[NIT];
        float dk_dot = 0.f, dq_dot = 0.f;
#pragma unroll
        for (int it = 0; it < NIT; it++) {
            const int i4 = lane + 64 * it;
            kk[it] = qq[it] = gk[it] = gv[it] = gq[it] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (i4 < d4) {
                const int i = 4 * i4;
                const size_t o = (((size_t)b * nh + i / hd) * s + t) * hd + i % hd;
                kk[it] = *reinterpret_cast<const float4 *>(kr + i);
                qq[it] = *reinterpret_cast<const float4 *>(qr + i);
                if (inputs_raw) {   // the same products as the forward's normalisation
                    kk[it].x *= ki; kk[it].y *= ki; kk[it].z *= ki; kk[it].w *= ki;
                    qq[it].x *= qi; qq[it].y *= qi; qq[it].z *= qi; qq[it].w *= qi;
                }
                const float4 vv = *reinterpret_cast<const float4 *>(vr + i);
                gk[it] = *reinterpret_cast<const float4 *>(dkh + o);
                gv[it] = *reinterpret_cast<const float4 *>(dvh + o);
                gq[it] = *reinterpret_cast<const float4 *>(dqh + o);
                fma4(acc[0][0][it], da, kk[it]); fma4(acc[0][1][it], da, vv);
                fma4(acc[1][0][it], dt, kk[it]); fma4(acc[1][1][it], dt, vv);
                fma4(acc[2][0][it], de, kk[it]); fma4(acc[2][1][it], de, vv);
            }
            dk_dot += dot4(gk[it], kk[it]);
            dq_dot += dot4(gq[it], qq[it]);
        }
        dk_dot = wave_allreduce(dk_dot);
        dq_dot = wave_allreduce(dq_dot);
        uint16_t *prow = P + (size_t)tok * p_ld;
#pragma unroll
        for (int it = 0; it < NIT; it++) {
            const int i4 = lane + 64 * it;
            if (i4 >= d4) continue;
            float4 a, c;
            if (kn >= eps) {
                a.x = (gk[it].x - kk[it].x * dk_dot) * ki; a.y = (gk[it].y - kk[it].y * dk_dot) * ki;
                a.z = (gk[it].z - kk[it].z * dk_dot) * ki; a.w = (gk[it].w - kk[it].w * dk_dot) * ki;
            } else {
                a.x = gk[it].x * inv_eps; a.y = gk[it].y * inv_eps; a.z = gk[it].z * inv_eps; a.w = gk[it].w * inv_eps;
            }
            if (qn >= eps) {
                c.x = (gq[it].x - qq[it].x * dq_dot) * qi; c.y = (gq[it].y - qq[it].y * dq_dot) * qi;
                c.z = (gq[it].z - qq[it].z * dq_dot) * qi; c.w = (gq[it].w - qq[it].w * dq_dot) * qi;
            } else {
                c.x = gq[it].x * inv_eps; c.y = gq[it].y * inv_eps; c.z = gq[it].z * inv_eps; c.w = gq[it].w * inv_eps;
            }
            store_split(prow, 4 * i4, off_h1, off_l, off_h2, a);
            store_split(prow, (long long)d + 4 * i4, off_h1, off_l, off_h2, gv[it]);
            store_split(prow, 2LL * d + 4 * i4, off_h1, off_l, off_h2, c);
        }
    }
    // the workgroup's partial row: the waves add their sums into LDS one after the other (fixed order)
    const int stride = 2 * d + 1;
    for (int w = 0; w < kWavesWg; w++) {
        if (wave_l == w) {
#pragma unroll
            for (int g = 0; g < 3; g++) {
#pragma unroll
                for (int h = 0; h < 2; h++)
#pragma unroll
                    for (int it = 0; it < NIT; it++) {
                        const int i4 = lane + 64 * it;
                        if (i4 >= d4) continue;
                        float *r = red + g * stride + h * d + 4 * i4;
                        const float4 a = acc[g][h][it];
                        if (w == 0) { r[0] = a.x; r[1] = a.y; r[2] = a.z; r[3] = a.w; }
                        else { r[0] += a.x; r[1] += a.y; r[2] += a.z; r[3] += a.w; }
                    }
                if (lane == 0) {
                    if (w == 0) red[g * stride + 2 * d] = accb[g];
                    else red[g * stride + 2 * d] += accb[g];
                }
            }
        }
        __syncthreads();
    }
    float *pb = part + (size_t)blockIdx.x * 3 * stride;
    for (int i = threadIdx.x; i < 3 * stride; i += kThr) pb[i] = red[i];
}

// Sums the workgroups' partial rows [nblk][3][2d + 1] in a fixed order: a workgroup per (64 columns, gate),
// 16 thread groups that each take every 16th row, combined in order.
__global__ __launch_bounds__(1024) void gate_partials_reduce_kernel(const float *__restrict__ part, int nblk, int twoD,
                                                                    float *d_w_alpha, float *d_b_alpha, float *d_w_theta,
                                                                    float *d_b_theta, float *d_w_eta, float *d_b_eta) {
    __shared__ float red[16][64];
    const int col = threadIdx.x & 63, seg = threadIdx.x >> 6, g = blockIdx.y;
    const int i = blockIdx.x * 64 + col;
    const size_t stride = (size_t)twoD + 1;
    float sum = 0.f;
    if (i <= twoD)
        for (int b = seg; b < nblk; b += 16) sum += part[((size_t)b * 3 + g) * stride + i];
    red[seg][col] = sum;
    __syncthreads();
    if (seg != 0 || i > twoD) return;
#pragma unroll
    for (int q = 1; q < 16; q++) sum += red[q][col];
    float *w = g == 0 ? d_w_alpha : (g == 1 ? d_w_theta : d_w_eta);
    float *bias = g == 0 ? d_b_alpha : (g == 1 ? d_b_theta : d_b_eta);
    if (i < twoD) w[i] = sum;
    else bias[0] = sum;
}

// gate = sigmoid(scale * sum_l y_l); gated = attn * gate, with attn in bf16 and 4 elements per thread; gated
// leaves as fp32 and / or as the packed left operand (hi | hi | lo) [n / d, 3d] of the output projection
struct LevelY { const float *y[8]; };
__global__ void combine_gate_bf16_kernel(LevelY lv, int k, float scale, const uint16_t *__restrict__ attn,
                                         float *__restrict__ gate, float *__restrict__ gated,
                                         uint16_t *__restrict__ gated_packed, int d, long long n4) {
    const long long stride = (long long)gridDim.x * blockDim.x;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride) {
        float4 sum = *reinterpret_cast<const float4 *>(lv.y[0] + 4 * i);
        for (int l = 1; l < k; l++) {
            const float4 y = *reinterpret_cast<const float4 *>(lv.y[l] + 4 * i);
            sum.x += y.x; sum.y += y.y; sum.z += y.z; sum.w += y.w;
        }
        const bf4 a = *reinterpret_cast<const bf4 *>(attn + 4 * i);
        float4 g, o;
        g.x = sigmoid_(sum.x * scale); g.y = sigmoid_(sum.y * scale);
        g.z = sigmoid_(sum.z * scale); g.w = sigmoid_(sum.w * scale);
        o.x = (float)a[0] * g.x; o.y = (float)a[1] * g.y; o.z = (float)a[2] * g.z; o.w = (float)a[3] * g.w;
        *reinterpret_cast<float4 *>(gate + 4 * i) = g;
        if (gated) *reinterpret_cast<float4 *>(gated + 4 * i) = o;
        if (gated_packed) {
            const long long e = 4 * i, row = e / d;
            store_split(gated_packed + row * 3 * d, e - row * d, 0, 2LL * d, d, o);
        }
    }
}

// d_attn = d_gated*gate; d_y = d_gated*attn*gate*(1-gate)*scale, attn in bf16
__global__ void gate_backward_bf16_kernel(const float *__restrict__ d_gated, const uint16_t *__restrict__ attn,
                                          const float *__restrict__ gate, float scale, float *__restrict__ d_attn,
                                          float *__restrict__ d_y, long long n4) {
    const long long stride = (long long)gridDim.x * blockDim.x;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride) {
        const float4 dg = *reinterpret_cast<const float4 *>(d_gated + 4 * i);
        const float4 g = *reinterpret_cast<const float4 *>(gate + 4 * i);
        const bf4 a = *reinterpret_cast<const bf4 *>(attn + 4 * i);
        float4 da, dy;
        da.x = dg.x * g.x; da.y = dg.y * g.y; da.z = dg.z * g.z; da.w = dg.w * g.w;
        dy.x = dg.x * (float)a[0] * g.x * (1.0f - g.x) * scale; dy.y = dg.y * (float)a[1] * g.y * (1.0f - g.y) * scale;
        dy.z = dg.z * (float)a[2] * g.z * (1.0f - g.z) * scale; dy.w = dg.w * (float)a[3] * g.w * (1.0f - g.w) * scale;
        *reinterpret_cast<float4 *>(d_attn + 4 * i) = da;
        *reinterpret_cast<float4 *>(d_y + 4 * i) = dy;
    }
}

inline int stream_blocks(long long items, int cap) {
    long long b = (items + kThr - 1) / kThr;
    return (int)(b < 1 ? 1 : (b > cap ? cap : b));
}
inline bool al16(const void *p) { return (((uintptr_t)p) & 15) == 0; }
inline bool al8(const void *p) { return (((uintptr_t)p) & 7) == 0; }

}  // namespace
}  // namespace nlh

using namespace nlh;

extern "C" {

void split_pack_bf16_ld_rocm(const float *const *srcs, int count, long long src_ld, uint16_t *out, long long n, int d,
                             long long out_ld, long long off_h1, long long off_l, long long off_h2) {
    if (n <= 0) return;
    if (count < 1 || count > 4 || d <= 0 || d % 4 || src_ld % 4 || out_ld % 4 || off_h1 % 4 || off_l % 4 || (off_h2 >= 0 && off_h2 % 4) ||
        !al8(out)) {
        fail("split_pack_bf16_ld_rocm: count=%d must be 1..4, d=%d, the strides and the offsets multiples of 4.", count, d);
        return;
    }
    SplitSrcs4 s{};
    for (int i = 0; i < count; i++) {
        if (!al16(srcs[i])) { fail("split_pack_bf16_ld_rocm: source %d is not 16-byte aligned.", i); return; }
        s.p[i] = srcs[i];
    }
    KernelTimer kt("split_pack_ld_kernel");
    hipLaunchKernelGGL(split_pack_ld_kernel, dim3(stream_blocks(n * count * (d / 4), 2048)), dim3(kThr), 0, stream(), s,
                       count, src_ld, out, n, d, out_ld, off_h1, off_l, off_h2);
    check_launch("split_pack_ld_kernel");
}

void split_pack_weights_rocm(const float *pack, int rows, int rows_stack, int d, uint16_t *wb, uint16_t *wstack) {
    if (rows <= 0) return;
    if (d <= 0 || d % 4 || rows_stack < 0 || rows_stack > rows || !al16(pack) || !al8(wb) || !al8(wstack)) {
        fail("split_pack_weights_rocm: d=%d must be a multiple of 4, rows_stack=%d in [0, rows=%d], buffers aligned.", d,
             rows_stack, rows);
        return;
    }
    KernelTimer kt("split_pack_weights_kernel");
    hipLaunchKernelGGL(split_pack_weights_kernel, dim3(stream_blocks((long long)rows * (d / 4), 2048)), dim3(kThr), 0,
                       stream(), pack, rows, rows_stack, d, wb, wstack);
    check_launch("split_pack_weights_kernel");
}

void level_inputs_fused_rocm(float *k_mem, const float *v_mem, float *q_mem, long long ld, const float *w_alpha,
                             const float *b_alpha, const float *w_theta, const float *b_theta, const float *w_eta,
                             const float *b_eta, float *k_norms, float *q_norms, float *alpha, float *theta, float *eta,
                             void *k_heads, void *v_heads, void *q_heads, float *alpha_heads, float *theta_heads,
                             float *eta_heads, int bs, int s, int nh, int hd, float eps, int heads_bf16,
                             int normalise_in_place) {
    const long long n = (long long)bs * s;
    if (n <= 0 || nh <= 0 || hd <= 0) return;
    const int d = nh * hd;
    if (hd % 4 || d > 1024 || ld % 4 || ld < d || !al16(k_mem) || !al16(v_mem) || !al16(q_mem) || !al16(w_alpha) ||
        !al16(w_theta) || !al16(w_eta) || !al16(k_heads) || !al16(v_heads) || !al16(q_heads)) {
        fail("level_inputs_fused_rocm: needs head_dim=%d a multiple of 4, nh*hd=%d <= 1024, ld=%lld a multiple of 4 and "
             ">= nh*hd, and 16-byte aligned buffers.", hd, d, ld);
        return;
    }
    const dim3 grid(stream_blocks(n * 64, 2048)), blk(kThr);
    KernelTimer kt("level_inputs_kernel");
#define NLH_LI(NIT, KV)                                                                                              \
    hipLaunchKernelGGL((level_inputs_kernel<NIT, KV>), grid, blk, 0, stream(), k_mem, v_mem, q_mem, ld, w_alpha,      \
                       b_alpha, w_theta, b_theta, w_eta, b_eta, k_norms, q_norms, alpha, theta, eta, k_heads, v_heads, \
                       q_heads, alpha_heads, theta_heads, eta_heads, bs, s, nh, hd, eps, normalise_in_place)
    if (d <= 256) { if (heads_bf16) NLH_LI(1, true); else NLH_LI(1, false); }
    else if (d <= 512) { if (heads_bf16) NLH_LI(2, true); else NLH_LI(2, false); }
    else { if (heads_bf16) NLH_LI(4, true); else NLH_LI(4, false); }
#undef NLH_LI
    check_launch("level_inputs_kernel");
}

void level_grads_packed_rocm(const float *d_k_heads, const float *d_v_heads, const float *d_q_heads,
                             const float *d_alpha_heads, const float *d_theta_heads, const float *d_eta_heads,
                             const float *k_norm, const float *v_mem, const float *q_norm, long long ld,
                             const float *k_norms, const float *q_norms, const float *alpha, const float *theta,
                             const float *eta, uint16_t *p_out, long long p_ld, long long off_h1, long long off_l,
                             long long off_h2, float *d_w_alpha, float *d_b_alpha, float *d_w_theta, float *d_b_theta,
                             float *d_w_eta, float *d_b_eta, int bs, int s, int nh, int hd, float eps, int inputs_raw) {
    const ErrorScope es;
    const long long n = (long long)bs * s;
    if (n <= 0 || nh <= 0 || hd <= 0) return;
    const int d = nh * hd;
    if (hd % 4 || d > 1024 || ld % 4 || ld < d || p_ld % 4 || off_h1 % 4 || off_l % 4 || (off_h2 >= 0 && off_h2 % 4) || !al16(d_k_heads) ||
        !al16(d_v_heads) || !al16(d_q_heads) || !al16(k_norm) || !al16(v_mem) || !al16(q_norm) || !al8(p_out)) {
        fail("level_grads_packed_rocm: needs head_dim=%d a multiple of 4, nh*hd=%d <= 1024, strides and offsets multiples "
             "of 4, ld=%lld >= nh*hd, and aligned buffers.", hd, d, ld);
        return;
    }
    const int nblk = stream_blocks(n * 64, 512);
    const size_t row = 3 * (2 * (size_t)d + 1);
    float *part = scratch(10, (size_t)nblk * row * sizeof(float));
    if (es.failed()) return;
    {
        KernelTimer kt("level_grads_packed_kernel");
#define NLH_LG(NIT)                                                                                                  \
    hipLaunchKernelGGL((level_grads_packed_kernel<NIT>), dim3(nblk), dim3(kThr), row * sizeof(float), stream(),       \
                       d_k_heads, d_v_heads, d_q_heads, d_alpha_heads, d_theta_heads, d_eta_heads, k_norm, v_mem, q_norm, \
                       ld, k_norms, q_norms, alpha, theta, eta, p_out, p_ld, off_h1, off_l, off_h2, part, bs, s, nh, hd, eps, \
                       inputs_raw)
        if (d <= 256) NLH_LG(1);
        else if (d <= 512) NLH_LG(2);
        else NLH_LG(4);
#undef NLH_LG
        check_launch("level_grads_packed_kernel");
    }
    KernelTimer kt("gate_partials_reduce_kernel");
    hipLaunchKernelGGL(gate_partials_reduce_kernel, dim3(ceil_div(2 * d + 1, 64), 3), dim3(1024), 0, stream(), part, nblk,
                       2 * d, d_w_alpha, d_b_alpha, d_w_theta, d_b_theta, d_w_eta, d_b_eta);
    check_launch("gate_partials_reduce_kernel");
}

void cms_combine_gate_bf16_rocm(const float *const *y_levels, int k, const uint16_t *attn_out, float *gate, float *gated,
                                uint16_t *gated_packed, int d, long long n) {
    if (k < 1 || k > 8) { fail("cms_combine_gate_bf16_rocm: k=%d must be in [1, 8].", k); return; }
    if (n <= 0) return;
    if (n % 4 || !al8(attn_out) || !al16(gate) || !al16(gated) || !al8(gated_packed) ||
        (gated_packed && (d <= 0 || d % 4 || n % d))) {
        fail("cms_combine_gate_bf16_rocm: n=%lld must be a multiple of 4 (and of d=%d, itself a multiple of 4, for the "
             "packed output) and the buffers aligned.", n, d);
        return;
    }
    LevelY lv{};
    for (int l = 0; l < k; l++) {
        if (!al16(y_levels[l])) { fail("cms_combine_gate_bf16_rocm: level %d is not 16-byte aligned.", l); return; }
        lv.y[l] = y_levels[l];
    }
    const float scale = k > 2 ? 1.0f / sqrtf((float)k) : 1.0f;
    KernelTimer kt("combine_gate_bf16_kernel");
    hipLaunchKernelGGL(combine_gate_bf16_kernel, dim3(stream_blocks(n / 4, 4096)), dim3(kThr), 0, stream(), lv, k, scale,
                       attn_out, gate, gated, gated_packed, d, n / 4);
    check_launch("combine_gate_bf16_kernel");
}

void cms_gate_backward_bf16_rocm(const float *d_gated, const uint16_t *attn_out, const float *gate, int k, float *d_attn,
                                 float *d_y_combined, long long n) {
    if (n <= 0) return;
    if (n % 4 || !al16(d_gated) || !al8(attn_out) || !al16(gate) || !al16(d_attn) || !al16(d_y_combined)) {
        fail("cms_gate_backward_bf16_rocm: n=%lld must be a multiple of 4 and the buffers aligned.", n);
        return;
    }
    const float scale = k > 2 ? 1.0f / sqrtf((float)k) : 1.0f;
    KernelTimer kt("gate_backward_bf16_kernel");
    hipLaunchKernelGGL(gate_backward_bf16_kernel, dim3(stream_blocks(n / 4, 4096)), dim3(kThr), 0, stream(), d_gated,
                       attn_out, gate, scale, d_attn, d_y_combined, n / 4);
    check_launch("gate_backward_bf16_kernel");
}

}  // extern "C"
