// Sliding-window attention, forward and backward (bf16 storage, f32 math).
//
// Contract (core/kernels/swa_forward.cu, swa_backward.cu): q/k/v/out are
// [batch, seq, heads*hd] bf16; the forward also emits the normalised attention
// weights [batch, heads, seq, n_persistent + window] as bf16 and the backward
// differentiates through those ROUNDED weights.  Query t sees the prefix keys
// [0, min(t+1, n_persistent)) and the local keys [ls, t], ls = max(t+1-window,
// n_persistent); weight slot of prefix key p is p, of local key ls+w is
// n_persistent+w; unused slots hold 0.
//
// This version: one wavefront per query (forward, backward pass 1) and one per
// key (backward pass 2).  Scores put keys on lanes (each lane walks its key row
// with 16-byte loads), value sums put head dimensions on lanes.  The backward
// has no atomics: pass 1 writes d_q and the per-slot score gradients, pass 2
// gathers d_k / d_v per key in a fixed order, so results are reproducible.
#include <hip/hip_runtime.h>
#include <float.h>
#include <math.h>

#include "../../include/nl_hecate_ffi.h"
#include "lane_ops.h"
#include "runtime.h"
#include "swa_mfma.h"

namespace nlh {

constexpr int kSwaWaves = 4;

__device__ __forceinline__ float bf2f(unsigned short h) { return __uint_as_float(((unsigned)h) << 16); }
__device__ __forceinline__ unsigned short f2bf(float f) {
    unsigned u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (unsigned short)((u >> 16) | 0x40);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (unsigned short)(u >> 16);
}

// Orders one wave's LDS writes before reads by its other lanes.
__device__ __forceinline__ void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

struct SwaGeom { int n_p, ls, ll; };
__device__ __forceinline__ SwaGeom swa_geom(int t, int window, int n_persistent) {
    SwaGeom g;
    g.n_p = min(t + 1, n_persistent);
    if (t >= n_persistent) {
        g.ls = max(t + 1 - window, n_persistent);
        g.ll = t + 1 - g.ls;
    } else {
        g.ls = 0;
        g.ll = 0;
    }
    return g;
}

// dot of a bf16 row (global) with an f32 vector held in LDS
__device__ __forceinline__ float dot_row_bf16(const unsigned short *__restrict__ row,
                                              const float *__restrict__ vec, int hd) {
    float acc = 0.f;
    if ((hd & 7) == 0 && ((((uintptr_t)row) & 15) == 0)) {
        for (int c = 0; c < hd; c += 8) {
            const uint4 p = *reinterpret_cast<const uint4 *>(row + c);
            const float4 a = *reinterpret_cast<const float4 *>(vec + c);
            const float4 b = *reinterpret_cast<const float4 *>(vec + c + 4);
            acc += __uint_as_float(p.x << 16) * a.x + __uint_as_float(p.x & 0xffff0000u) * a.y;
            acc += __uint_as_float(p.y << 16) * a.z + __uint_as_float(p.y & 0xffff0000u) * a.w;
            acc += __uint_as_float(p.z << 16) * b.x + __uint_as_float(p.z & 0xffff0000u) * b.y;
            acc += __uint_as_float(p.w << 16) * b.z + __uint_as_float(p.w & 0xffff0000u) * b.w;
        }
    } else {
        for (int c = 0; c < hd; c++) acc += bf2f(row[c]) * vec[c];
    }
    return acc;
}

// LDS per wave: vec[hd] (q or dO as f32) + sc[aw] (scores / weights)
__global__ __launch_bounds__(kSwaWaves * 64) void swa_forward_kernel(
    const unsigned short *__restrict__ q, const unsigned short *__restrict__ k,
    const unsigned short *__restrict__ v, unsigned short *__restrict__ out,
    unsigned short *__restrict__ attn_w, int seq_len, int num_heads, int head_dim, int window,
    int n_persistent, long long n_queries) {
    extern __shared__ __align__(16) float smem[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int aw = n_persistent + window;
    const int per_wave = ((head_dim + 3) & ~3) + aw;
    float *vec = smem + (size_t)wave * per_wave;
    float *sc = vec + ((head_dim + 3) & ~3);
    const long long qi = (long long)blockIdx.x * kSwaWaves + wave;  // (b, h, t) flattened
    if (qi >= n_queries) return;
    const int t = (int)(qi % seq_len);
    const int h = (int)((qi / seq_len) % num_heads);
    const long long b = qi / ((long long)seq_len * num_heads);
    const int td = num_heads * head_dim;
    const unsigned short *qb = q + (b * seq_len + t) * td + h * head_dim;
    const unsigned short *kb = k + b * seq_len * td + h * head_dim;
    const unsigned short *vb = v + b * seq_len * td + h * head_dim;
    const SwaGeom g = swa_geom(t, window, n_persistent);
    const float scale = 1.0f / sqrtf((float)head_dim);

    for (int d = lane; d < head_dim; d += 64) vec[d] = bf2f(qb[d]);
    wave_sync();
    // scores, one key per lane per round
    float mx = -INFINITY;
    for (int s = lane; s < aw; s += 64) {
        const bool valid = s < n_persistent ? s < g.n_p : (s - n_persistent) < g.ll;
        float x = -INFINITY;
        if (valid) {
            const int key = s < n_persistent ? s : g.ls + (s - n_persistent);
            x = dot_row_bf16(kb + (size_t)key * td, vec, head_dim) * scale;
        }
        sc[s] = x;
        mx = fmaxf(mx, x);
    }
    for (int m = 1; m < 64; m <<= 1) mx = fmaxf(mx, __shfl_xor(mx, m, 64));
    float sum = 0.f;
    for (int s = lane; s < aw; s += 64) {
        const float x = sc[s];
        const float e = x == -INFINITY ? 0.f : expf(x - mx);
        sc[s] = e;
        sum += e;
    }
    sum = wave_allreduce(sum);
    const float inv = 1.0f / sum;
    unsigned short *wr = attn_w + ((b * num_heads + h) * seq_len + t) * (long long)aw;
    for (int s = lane; s < aw; s += 64) {
        const float w = sc[s] * inv;
        sc[s] = w;
        wr[s] = f2bf(w);
    }
    wave_sync();
    // out[d] = sum_s w_s v[key_s][d]  (unrounded weights, as the reference)
    for (int d = lane; d < head_dim; d += 64) {
        float acc = 0.f;
        for (int s = 0; s < g.n_p; s++) acc += sc[s] * bf2f(vb[(size_t)s * td + d]);
        for (int w = 0; w < g.ll; w++) acc += sc[n_persistent + w] * bf2f(vb[(size_t)(g.ls + w) * td + d]);
        out[(b * seq_len + t) * td + h * head_dim + d] = f2bf(acc);
    }
}

// Backward pass 1, one wave per query: dW_s = dO . V[key_s]; D = sum_s w_s dW_s;
// dS_s = w_s (dW_s - D) * scale -> ds_out; d_q = sum_s dS_s K[key_s].
__global__ __launch_bounds__(kSwaWaves * 64) void swa_backward_query_kernel(
    const unsigned short *__restrict__ k, const unsigned short *__restrict__ v,
    const unsigned short *__restrict__ attn_w, const float *__restrict__ d_out,
    float *__restrict__ d_q, float *__restrict__ ds_out, int seq_len, int num_heads, int head_dim,
    int window, int n_persistent, long long n_queries) {
    extern __shared__ __align__(16) float smem[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int aw = n_persistent + window;
    const int per_wave = ((head_dim + 3) & ~3) + aw;
    float *vec = smem + (size_t)wave * per_wave;
    float *sc = vec + ((head_dim + 3) & ~3);
    const long long qi = (long long)blockIdx.x * kSwaWaves + wave;
    if (qi >= n_queries) return;
    const int t = (int)(qi % seq_len);
    const int h = (int)((qi / seq_len) % num_heads);
    const long long b = qi / ((long long)seq_len * num_heads);
    const int td = num_heads * head_dim;
    const size_t qo = (size_t)(b * seq_len + t) * td + h * head_dim;
    const unsigned short *kb = k + b * seq_len * td + h * head_dim;
    const unsigned short *vb = v + b * seq_len * td + h * head_dim;
    const unsigned short *wr = attn_w + ((b * num_heads + h) * seq_len + t) * (long long)aw;
    float *dsr = ds_out + ((b * num_heads + h) * seq_len + t) * (long long)aw;
    const SwaGeom g = swa_geom(t, window, n_persistent);
    const float scale = 1.0f / sqrtf((float)head_dim);

    for (int d = lane; d < head_dim; d += 64) vec[d] = d_out[qo + d];
    wave_sync();
    float dot_pw = 0.f;
    for (int s = lane; s < aw; s += 64) {
        const bool valid = s < n_persistent ? s < g.n_p : (s - n_persistent) < g.ll;
        float dw = 0.f;
        if (valid) {
            const int key = s < n_persistent ? s : g.ls + (s - n_persistent);
            dw = dot_row_bf16(vb + (size_t)key * td, vec, head_dim);
        }
        sc[s] = dw;
        dot_pw += bf2f(wr[s]) * dw;
    }
    dot_pw = wave_allreduce(dot_pw);
    for (int s = lane; s < aw; s += 64) {
        const float ds = bf2f(wr[s]) * (sc[s] - dot_pw) * scale;
        sc[s] = ds;
        dsr[s] = ds;
    }
    wave_sync();
    for (int d = lane; d < head_dim; d += 64) {
        float acc = 0.f;
        for (int s = 0; s < g.n_p; s++) acc += sc[s] * bf2f(kb[(size_t)s * td + d]);
        for (int w = 0; w < g.ll; w++) acc += sc[n_persistent + w] * bf2f(kb[(size_t)(g.ls + w) * td + d]);
        d_q[qo + d] = acc;
    }
}

// Backward pass 2, one wave per key j: gathers over the queries that see j.
//   d_v[j] += sum_t w[t, slot(t,j)] dO[t];  d_k[j] += sum_t dS[t, slot(t,j)] q[t]
// Queries that see key j: prefix key (j < n_persistent): every t >= j;
// local key: t in [j, j + window - 1] (with t >= n_persistent).
__global__ __launch_bounds__(kSwaWaves * 64) void swa_backward_key_kernel(
    const unsigned short *__restrict__ q, const unsigned short *__restrict__ attn_w,
    const float *__restrict__ d_out, const float *__restrict__ ds, float *__restrict__ d_k,
    float *__restrict__ d_v, int seq_len, int num_heads, int head_dim, int window, int n_persistent,
    long long n_keys) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const long long ki = (long long)blockIdx.x * kSwaWaves + wave;
    if (ki >= n_keys) return;
    const int j = (int)(ki % seq_len);
    const int h = (int)((ki / seq_len) % num_heads);
    const long long b = ki / ((long long)seq_len * num_heads);
    const int td = num_heads * head_dim, aw = n_persistent + window;
    const bool prefix = j < n_persistent;
    const int t_lo = prefix ? j : max(j, n_persistent);
    const int t_hi = prefix ? seq_len - 1 : min(seq_len - 1, j + window - 1);
    const unsigned short *wb = attn_w + ((b * num_heads + h) * seq_len) * (long long)aw;
    const float *dsb = ds + ((b * num_heads + h) * seq_len) * (long long)aw;
    for (int d0 = 0; d0 < head_dim; d0 += 64) {
        const int d = d0 + lane;
        float av = 0.f, ak = 0.f;
        for (int t = t_lo; t <= t_hi; t++) {
            int slot;
            if (prefix) slot = j;
            else slot = n_persistent + (j - max(t + 1 - window, n_persistent));
            const float w = bf2f(wb[(long long)t * aw + slot]);
            const float dsv = dsb[(long long)t * aw + slot];
            if (d < head_dim) {
                const size_t o = (size_t)(b * seq_len + t) * td + h * head_dim + d;
                av += w * d_out[o];
                ak += dsv * bf2f(q[o]);
            }
        }
        if (d < head_dim) {
            const size_t o = (size_t)(b * seq_len + j) * td + h * head_dim + d;
            d_v[o] += av;
            d_k[o] += ak;
        }
    }
}

// Decode-time attention of the newest token against a KV cache
// (core/kernels/swa_forward.cu:187-291): same two-range mask as the full kernel
// for query position cache_len-1, no attention weights kept.  One workgroup per
// head; a thread scores whole keys (no per-key reduction), then the block
// normalises and gathers.
constexpr int kDecThreads = 256;
__global__ __launch_bounds__(kDecThreads) void swa_single_token_kernel(
    const unsigned short *__restrict__ q, const unsigned short *__restrict__ k_cache,
    const unsigned short *__restrict__ v_cache, unsigned short *__restrict__ out, int cache_len, int num_heads,
    int head_dim, int window, int n_persistent) {
    extern __shared__ float dsm[];
    float *qf = dsm, *sc = dsm + head_dim, *red = sc + n_persistent + window;  // red [kDecThreads]
    __shared__ float wred[kDecThreads / 64];
    const int h = blockIdx.x, tid = threadIdx.x, total = num_heads * head_dim, hoff = h * head_dim;
    const int aw = n_persistent + window;
    const SwaGeom g = swa_geom(cache_len - 1, window, n_persistent);
    for (int d = tid; d < head_dim; d += kDecThreads) qf[d] = bf2f(q[hoff + d]);
    __syncthreads();
    const float scale = rsqrtf((float)head_dim);
    auto key_of = [&](int w) -> int {   // cache row of score slot w, or -1 when masked
        if (w < n_persistent) return w < g.n_p ? w : -1;
        const int l = w - n_persistent;
        return l < g.ll ? g.ls + l : -1;
    };
    float mx = -FLT_MAX;
    for (int w = tid; w < aw; w += kDecThreads) {
        const int kp = key_of(w);
        float sv = -FLT_MAX;
        if (kp >= 0) {
            const unsigned short *kr = k_cache + (size_t)kp * total + hoff;
            float acc = 0.f;
            for (int d = 0; d < head_dim; d++) acc = fmaf(qf[d], bf2f(kr[d]), acc);
            sv = acc * scale;
        }
        sc[w] = sv;
        mx = fmaxf(mx, sv);
    }
    // block max
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    if ((tid & 63) == 0) wred[tid >> 6] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(wred[0], wred[1]), fmaxf(wred[2], wred[3]));
    __syncthreads();
    float sum = 0.f;
    for (int w = tid; w < aw; w += kDecThreads) {
        const float e = expf(sc[w] - mx);
        sc[w] = e;
        sum += e;
    }
    sum = wave_allreduce(sum);
    if ((tid & 63) == 0) wred[tid >> 6] = sum;
    __syncthreads();
    const float inv = 1.f / (wred[0] + wred[1] + wred[2] + wred[3]);
    // weighted sum of V: thread (grp, d) walks the slots congruent to grp
    const int ngrp = kDecThreads / head_dim;   // head_dim <= 256 and divides 256 (checked on the host)
    const int d = tid % head_dim, grp = tid / head_dim;
    float acc = 0.f;
    for (int w = grp; w < aw; w += ngrp) {
        const int kp = key_of(w);
        if (kp >= 0) acc = fmaf(sc[w] * inv, bf2f(v_cache[(size_t)kp * total + hoff + d]), acc);
    }
    red[tid] = acc;
    __syncthreads();
    if (grp == 0) {
        for (int gg = 1; gg < ngrp; gg++) acc += red[gg * head_dim + d];
        out[hoff + d] = f2bf(acc);
    }
}

static bool swa_check(const char *fn, int seq_len, int num_heads, int head_dim, int window, int batch,
                      int n_persistent) {
    if (seq_len <= 0 || num_heads <= 0 || head_dim <= 0 || window <= 0 || batch <= 0 || n_persistent < 0) {
        fail("%s: bad shape (seq_len=%d heads=%d head_dim=%d window=%d batch=%d n_persistent=%d).", fn,
             seq_len, num_heads, head_dim, window, batch, n_persistent);
        return false;
    }
    const size_t lds = (size_t)kSwaWaves * (((head_dim + 3) & ~3) + n_persistent + window) * sizeof(float);
    if (lds > 64 * 1024) {
        fail("%s: window + n_persistent = %d needs %zu bytes of LDS (limit 65536).", fn,
             window + n_persistent, lds);
        return false;
    }
    return true;
}

}  // namespace nlh

using namespace nlh;

extern "C" {

void swa_forward_f32_cuda(const uint16_t *q, const uint16_t *k, const uint16_t *v, uint16_t *out,
                          uint16_t *attn_weights, int seq_len, int num_heads, int head_dim,
                          int window_size, int batch_size, int n_persistent) {
    if (!swa_check("swa_forward_f32_cuda", seq_len, num_heads, head_dim, window_size, batch_size, n_persistent))
        return;
    if (swa_forward_mfma(q, k, v, out, attn_weights, seq_len, num_heads, head_dim, window_size, batch_size,
                         n_persistent))
        return;
    const long long nq = (long long)batch_size * num_heads * seq_len;
    const size_t lds = (size_t)kSwaWaves * (((head_dim + 3) & ~3) + n_persistent + window_size) * sizeof(float);
    hipLaunchKernelGGL(swa_forward_kernel, dim3((unsigned)((nq + kSwaWaves - 1) / kSwaWaves)),
                       dim3(kSwaWaves * 64), lds, stream(), q, k, v, out, attn_weights, seq_len, num_heads,
                       head_dim, window_size, n_persistent, nq);
    check_launch("swa_forward_kernel");
}

void swa_backward_f32_cuda(const uint16_t *q, const uint16_t *k, const uint16_t *v,
                           const uint16_t *attn_weights, const float *d_attn_out,
                           float *d_q, float *d_k, float *d_v, int seq_len, int num_heads, int head_dim,
                           int window_size, int batch_size, int n_persistent) {
    const ErrorScope es;
    if (!swa_check("swa_backward_f32_cuda", seq_len, num_heads, head_dim, window_size, batch_size, n_persistent))
        return;
    if (swa_backward_mfma(q, k, v, attn_weights, d_attn_out, d_q, d_k, d_v, seq_len, num_heads, head_dim,
                          window_size, batch_size, n_persistent))
        return;
    const long long nq = (long long)batch_size * num_heads * seq_len;
    const int aw = n_persistent + window_size;
    float *ds = scratch(0, (size_t)nq * aw * sizeof(float));
    if (es.failed()) return;
    const size_t lds = (size_t)kSwaWaves * (((head_dim + 3) & ~3) + aw) * sizeof(float);
    const dim3 grid((unsigned)((nq + kSwaWaves - 1) / kSwaWaves)), blk(kSwaWaves * 64);
    hipLaunchKernelGGL(swa_backward_query_kernel, grid, blk, lds, stream(), k, v, attn_weights, d_attn_out,
                       d_q, ds, seq_len, num_heads, head_dim, window_size, n_persistent, nq);
    check_launch("swa_backward_query_kernel");
    hipLaunchKernelGGL(swa_backward_key_kernel, grid, blk, 0, stream(), q, attn_weights, d_attn_out, ds, d_k,
                       d_v, seq_len, num_heads, head_dim, window_size, n_persistent, nq);
    check_launch("swa_backward_key_kernel");
}

void swa_forward_lse_bf16_rocm(const uint16_t *q, const uint16_t *k, const uint16_t *v, uint16_t *out, float *stats,
                               int seq_len, int num_heads, int head_dim, int window_size, int batch_size) {
    if (!swa_check("swa_forward_lse_bf16_rocm", seq_len, num_heads, head_dim, window_size, batch_size, 0)) return;
    if (!stats) return fail("swa_forward_lse_bf16_rocm: stats is null");
    if (!swa_forward_mfma(q, k, v, out, nullptr, seq_len, num_heads, head_dim, window_size, batch_size, 0, stats))
        fail("swa_forward_lse_bf16_rocm: needs head_dim 64 or 32 and window_size <= 512");
}

void swa_backward_lse_bf16_rocm(const uint16_t *q, const uint16_t *k, const uint16_t *v, const float *stats,
                                const float *d_attn_out, float *d_q, float *d_k, float *d_v, int seq_len,
                                int num_heads, int head_dim, int window_size, int batch_size) {
    const ErrorScope es;
    if (!swa_check("swa_backward_lse_bf16_rocm", seq_len, num_heads, head_dim, window_size, batch_size, 0)) return;
    if (!stats) return fail("swa_backward_lse_bf16_rocm: stats is null");
    if (!swa_backward_mfma(q, k, v, nullptr, d_attn_out, d_q, d_k, d_v, seq_len, num_heads, head_dim, window_size,
                           batch_size, 0, stats))
        fail("swa_backward_lse_bf16_rocm: needs head_dim 64 or 32 and window_size <= 512");
}

void swa_backward_lse_bf16_cols_rocm(const uint16_t *q, const uint16_t *k, const uint16_t *v, const float *stats,
                                     const float *d_attn_out, uint16_t *g_q, uint16_t *g_k, uint16_t *g_v, long long ld,
                                     int seq_len, int num_heads, int head_dim, int window_size, int batch_size) {
    const ErrorScope es;
    const char *fn = "swa_backward_lse_bf16_cols_rocm";
    if (!swa_check(fn, seq_len, num_heads, head_dim, window_size, batch_size, 0)) return;
    if (!stats || !g_q || !g_k || !g_v) return fail("%s: a pointer is null", fn);
    if (ld < (long long)num_heads * head_dim || ld % 4 || (((uintptr_t)g_q | (uintptr_t)g_k | (uintptr_t)g_v) & 7))
        return fail("%s: ld=%lld must be a multiple of 4 and at least heads * head_dim, the columns 8-byte aligned", fn, ld);
    const SwaGradCols cols{g_q, g_k, g_v, ld};
    if (!swa_backward_mfma(q, k, v, nullptr, d_attn_out, nullptr, nullptr, nullptr, seq_len, num_heads, head_dim, window_size,
                           batch_size, 0, stats, &cols))
        fail("%s: needs head_dim 64 or 32 and window_size <= 512", fn);
}

void swa_single_token_cuda(const uint16_t *q, const uint16_t *k_cache, const uint16_t *v_cache, uint16_t *out,
                           int cache_len, int num_heads, int head_dim, int window_size, int n_persistent) {
    const char *fn = "swa_single_token_cuda";
    if (cache_len <= 0 || num_heads <= 0 || head_dim <= 0 || window_size <= 0 || n_persistent < 0) {
        fail("%s: bad shape (cache_len=%d heads=%d head_dim=%d window=%d n_persistent=%d).", fn, cache_len,
             num_heads, head_dim, window_size, n_persistent);
        return;
    }
    if (head_dim > kDecThreads || kDecThreads % head_dim != 0) {
        fail("%s: head_dim=%d unsupported (must divide %d).", fn, head_dim, kDecThreads);
        return;
    }
    const size_t lds = ((size_t)head_dim + n_persistent + window_size + kDecThreads) * sizeof(float);
    if (lds > 64 * 1024) {
        fail("%s: window + n_persistent = %d needs %zu bytes of LDS (limit 65536).", fn,
             window_size + n_persistent, lds);
        return;
    }
    hipLaunchKernelGGL(swa_single_token_kernel, dim3(num_heads), dim3(kDecThreads), lds, stream(), q, k_cache,
                       v_cache, out, cache_len, num_heads, head_dim, window_size, n_persistent);
    check_launch("swa_single_token_kernel");
}

}  // extern "C"
