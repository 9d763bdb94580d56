// Kernels around the memory path that a whole-model step also needs: LayerNorm, embedding gather /
// scatter-add, transpose copy (weight tying), cross-entropy, the TNT shard helpers and the 1-D pooling
// pair.  Contracts of core/kernels/{layer_norm,embedding,cross_entropy,tnt_forward,tnt_backward,
// pool_ops}.cu (core/src/cuda_ffi.rs:484-500, 520-547, 613-668, 766-777, 1061-1084).
//
// All are HBM-bound row kernels: one wave per row with DPP sums where a row is reduced, 16-byte
// accesses where alignment allows.  Where the reference accumulates with atomicAdd (LayerNorm d_gamma /
// d_beta, embedding scatter-add, the cross-entropy loss, the TNT backward) the sums here are formed in a
// fixed order, so results are reproducible; the accumulate (+=) contracts are kept.
#include <hip/hip_runtime.h>
#include <float.h>
#include <math.h>
#include <stdint.h>

#include "../../include/nl_hecate_ffi.h"
#include "lane_ops.h"
#include "runtime.h"

namespace nlh {
namespace {

constexpr int kThreads = 256;
constexpr int kMaxBlocks = 256 * 8;

inline int blocks_for(long long items, int per_block) {
    long long b = (items + per_block - 1) / per_block;
    return (int)(b < 1 ? 1 : (b > kMaxBlocks ? kMaxBlocks : b));
}

// ── LayerNorm ────────────────────────────────────────────────────────────────
// layer_norm.cu:27-77: mean, biased variance as E[x^2] - mean^2, rstd = rsqrt(var + eps).
__global__ void layer_norm_fwd_kernel(const float *__restrict__ x, const float *__restrict__ gamma,
                                      const float *__restrict__ beta, float *__restrict__ out,
                                      float *__restrict__ mean_cache, float *__restrict__ rstd_cache, int n, int d,
                                      float eps) {
    const int lane = threadIdx.x & 63;
    const int wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6, nwaves = (gridDim.x * blockDim.x) >> 6;
    for (int r = wave; r < n; r += nwaves) {
        const float *row = x + (size_t)r * d;
        float s1 = 0.f, s2 = 0.f;
        for (int j = lane; j < d; j += 64) { const float v = row[j]; s1 += v; s2 += v * v; }
        s1 = wave_allreduce(s1);
        s2 = wave_allreduce(s2);
        const float mean = s1 / (float)d, var = s2 / (float)d - mean * mean;
        const float rstd = rsqrtf(var + eps);
        if (lane == 0) { mean_cache[r] = mean; rstd_cache[r] = rstd; }
        float *o = out + (size_t)r * d;
        for (int j = lane; j < d; j += 64) o[j] = gamma[j] * ((row[j] - mean) * rstd) + beta[j];
    }
}

// layer_norm.cu:81-136.  d_x per row, one wave per row.  A wave adds d_out * x_hat and d_out of its rows
// into its own LDS slab (a lane owns the columns lane, lane + 64, ...: no two lanes share one); the
// workgroup's slabs are added in wave order and leave as one partial row: part[2][gridDim.x][d].
__global__ void layer_norm_bwd_kernel(const float *__restrict__ d_out, const float *__restrict__ x,
                                      const float *__restrict__ gamma, const float *__restrict__ mean_cache,
                                      const float *__restrict__ rstd_cache, float *__restrict__ d_x,
                                      float *__restrict__ part, int n, int d) {
    extern __shared__ float acc[];   // [waves][2][d]
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, nwv = blockDim.x >> 6;
    float *mine = acc + (size_t)wv * 2 * d;
    for (int j = lane; j < 2 * d; j += 64) mine[j] = 0.f;
    const int rows_per_block = (n + gridDim.x - 1) / gridDim.x;
    const int r0 = blockIdx.x * rows_per_block, r1 = min(n, r0 + rows_per_block);
    for (int r = r0 + wv; r < r1; r += nwv) {
        const float *g = d_out + (size_t)r * d, *row = x + (size_t)r * d;
        const float mean = mean_cache[r], rstd = rstd_cache[r];
        float s1 = 0.f, s2 = 0.f;
        for (int j = lane; j < d; j += 64) {
            const float dg = g[j] * gamma[j];
            s1 += dg;
            s2 += dg * ((row[j] - mean) * rstd);
        }
        s1 = wave_allreduce(s1);
        s2 = wave_allreduce(s2);
        const float inv_d = 1.0f / (float)d;
        float *o = d_x + (size_t)r * d;
        for (int j = lane; j < d; j += 64) {
            const float xh = (row[j] - mean) * rstd, gj = g[j];
            o[j] = rstd * inv_d * ((float)d * (gj * gamma[j]) - s1 - xh * s2);
            mine[j] += gj * xh;
            mine[d + j] += gj;
        }
    }
    __syncthreads();
    for (int j = threadIdx.x; j < 2 * d; j += blockDim.x) {
        float sum = 0.f;
        for (int w = 0; w < nwv; w++) sum += acc[(size_t)w * 2 * d + j];
        part[((size_t)(j / d) * gridDim.x + blockIdx.x) * d + (j % d)] = sum;
    }
}

// dst_a[j] += sum_p part[0][p][j], dst_b[j] += sum_p part[1][p][j]
__global__ void add_partial_rows_kernel(const float *__restrict__ part, float *__restrict__ dst_a,
                                        float *__restrict__ dst_b, int nparts, int d) {
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= d) return;
    float a = 0.f, b = 0.f;
    for (int p = 0; p < nparts; p++) {
        a += part[(size_t)p * d + j];
        b += part[((size_t)nparts + p) * d + j];
    }
    dst_a[j] += a;
    dst_b[j] += b;
}

// ── embedding ────────────────────────────────────────────────────────────────
// embedding.cu:23-38
__global__ void embedding_gather_kernel(const float *__restrict__ w, const int *__restrict__ ids,
                                        float *__restrict__ out, int seq_len, int d) {
    const long long total = (long long)seq_len * d;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long long)gridDim.x * blockDim.x) {
        const int t = (int)(i / d), j = (int)(i % d);
        out[i] = w[(size_t)ids[t] * d + j];
    }
}

// embedding.cu:44-60 without atomics: the workgroup of position t does nothing unless t is the first
// position of its token id; then it adds the rows of every position with that id, in order.
__global__ void embedding_scatter_add_kernel(const float *__restrict__ d_embedded, const int *__restrict__ ids,
                                             float *__restrict__ d_embed, int seq_len, int d) {
    __shared__ int seen;
    for (int t = blockIdx.x; t < seq_len; t += gridDim.x) {
        const int tok = ids[t];
        if (threadIdx.x == 0) seen = 0;
        __syncthreads();
        int hit = 0;
        for (int u = threadIdx.x; u < t; u += blockDim.x) hit |= (ids[u] == tok);
        if (hit) seen = 1;   // benign: every writer stores the same value
        __syncthreads();
        const bool first = seen == 0;
        __syncthreads();
        if (!first) continue;
        for (int j = threadIdx.x; j < d; j += blockDim.x) {
            float sum = d_embed[(size_t)tok * d + j];
            for (int u = t; u < seq_len; u++)
                if (ids[u] == tok) sum += d_embedded[(size_t)u * d + j];
            d_embed[(size_t)tok * d + j] = sum;
        }
    }
}

// embedding.cu:68-80: dst[c * rows + r] = src[r * cols + c], through a padded 32 x 32 LDS tile
__global__ void transpose_copy_kernel(const float *__restrict__ src, float *__restrict__ dst, int rows, int cols) {
    __shared__ float tile[32][33];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;   // 32 x 8 threads
    const int tiles_c = (cols + 31) / 32, tiles_r = (rows + 31) / 32;
    for (int tl = blockIdx.x; tl < tiles_c * tiles_r; tl += gridDim.x) {
        const int r0 = (tl / tiles_c) * 32, c0 = (tl % tiles_c) * 32;
        for (int i = ty; i < 32; i += 8)
            if (r0 + i < rows && c0 + tx < cols) tile[i][tx] = src[(size_t)(r0 + i) * cols + c0 + tx];
        __syncthreads();
        for (int i = ty; i < 32; i += 8)
            if (c0 + i < cols && r0 + tx < rows) dst[(size_t)(c0 + i) * rows + r0 + tx] = tile[tx][i];
        __syncthreads();
    }
}

// ── cross-entropy ────────────────────────────────────────────────────────────
// Row maximum and sum of exp(x - max) in one sweep (running maximum, rescaled sum), per workgroup.
__device__ __forceinline__ void row_max_sumexp(const float *row, int vocab, float &mx, float &sum, float *red) {
    float m = -FLT_MAX, s = 0.f;
    for (int j = threadIdx.x; j < vocab; j += blockDim.x) {
        const float v = row[j];
        if (v > m) { s *= expf(m - v); m = v; }
        s += expf(v - m);
    }
    // combine (m, s) pairs: wave, then workgroup
    for (int off = 32; off > 0; off >>= 1) {
        const float m2 = __shfl_xor(m, off, 64), s2 = __shfl_xor(s, off, 64);
        const float mm = fmaxf(m, m2);
        s = s * expf(m - mm) + s2 * expf(m2 - mm);
        m = mm;
    }
    const int wv = threadIdx.x >> 6, nwv = blockDim.x >> 6;
    if ((threadIdx.x & 63) == 0) { red[2 * wv] = m; red[2 * wv + 1] = s; }
    __syncthreads();
    mx = red[0];
    for (int w = 1; w < nwv; w++) mx = fmaxf(mx, red[2 * w]);
    sum = 0.f;
    for (int w = 0; w < nwv; w++) sum += red[2 * w + 1] * expf(red[2 * w] - mx);
    __syncthreads();
}

// cross_entropy.cu:29-84: per-row NLL (0 for targets outside [0, vocab)) into nll[t]
__global__ void cross_entropy_fwd_kernel(const float *__restrict__ logits, const int *__restrict__ targets,
                                         float *__restrict__ nll, int seq_len, int vocab) {
    __shared__ float red[2 * (kThreads / 64)];
    for (int t = blockIdx.x; t < seq_len; t += gridDim.x) {
        const int target = targets[t];
        if (target < 0 || target >= vocab) {
            if (threadIdx.x == 0) nll[t] = 0.f;
            continue;
        }
        const float *row = logits + (size_t)t * vocab;
        float mx, sum;
        row_max_sumexp(row, vocab, mx, sum, red);
        if (threadIdx.x == 0) nll[t] = -(row[target] - mx - logf(sum));
    }
}

// loss_out[0] = sum_t nll[t], one workgroup, fixed order
__global__ void sum_to_scalar_kernel(const float *__restrict__ v, float *__restrict__ out, int n) {
    __shared__ float red[kThreads / 64];
    float s = 0.f;
    for (int i = threadIdx.x; i < n; i += blockDim.x) s += v[i];
    s = wave_allreduce(s);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        float tot = 0.f;
        for (int w = 0; w < (int)(blockDim.x >> 6); w++) tot += red[w];
        out[0] = tot;
    }
}

// cross_entropy.cu:101-160
__global__ void cross_entropy_bwd_kernel(const float *__restrict__ logits, const int *__restrict__ targets,
                                         float *__restrict__ d_logits, int seq_len, int vocab, float inv_count) {
    __shared__ float red[2 * (kThreads / 64)];
    for (int t = blockIdx.x; t < seq_len; t += gridDim.x) {
        const int target = targets[t];
        float *o = d_logits + (size_t)t * vocab;
        if (target < 0 || target >= vocab) {
            for (int j = threadIdx.x; j < vocab; j += blockDim.x) o[j] = 0.f;
            continue;
        }
        const float *row = logits + (size_t)t * vocab;
        float mx, sum;
        row_max_sumexp(row, vocab, mx, sum, red);
        for (int j = threadIdx.x; j < vocab; j += blockDim.x) {
            float g = expf(row[j] - mx) / sum;
            if (j == target) g -= 1.0f;
            o[j] = g * inv_count;
        }
    }
}

// ── TNT helpers ──────────────────────────────────────────────────────────────
// tnt_forward.cu:26-40
__global__ void tnt_broadcast_kernel(const float *__restrict__ src, float *__restrict__ dst, int n_local, int dd) {
    const long long total = (long long)n_local * dd;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long long)gridDim.x * blockDim.x)
        dst[i] = src[i % dd];
}
// tnt_forward.cu:62-79: column means, one thread per column, serial over the shard (the reference's order)
__global__ void tnt_summary_mean_kernel(const float *__restrict__ y, float *__restrict__ k_sum,
                                        float *__restrict__ v_sum, int shard_len, int d) {
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= d) return;
    float sum = 0.f;
    for (int t = 0; t < shard_len; t++) sum += y[(size_t)t * d + j];
    const float mean = sum / (float)shard_len;
    k_sum[j] = mean;
    v_sum[j] = mean;
}
// tnt_forward.cu:101-114
__global__ void tnt_global_update_kernel(float *__restrict__ m, const float *__restrict__ k_sum,
                                         const float *__restrict__ v_sum, int d, float alpha) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= d * d) return;
    m[idx] = alpha * m[idx] + v_sum[idx / d] * k_sum[idx % d];
}
// tnt_backward.cu:27-48: thread i < d owns row i (d_v_sum[i]) and column i (d_k_sum[i]), serial sums
__global__ void tnt_global_update_bwd_kernel(const float *__restrict__ d_m_new, const float *__restrict__ k_sum,
                                             const float *__restrict__ v_sum, float *__restrict__ d_m_old,
                                             float *__restrict__ d_k_sum, float *__restrict__ d_v_sum, int d,
                                             float alpha) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= d) return;
    float dv = 0.f, dk = 0.f;
    for (int j = 0; j < d; j++) {
        const float dm = d_m_new[(size_t)i * d + j];
        d_m_old[(size_t)i * d + j] = alpha * dm;
        dv += dm * k_sum[j];
        dk += d_m_new[(size_t)j * d + i] * v_sum[j];
    }
    d_v_sum[i] += dv;
    d_k_sum[i] += dk;
}
// tnt_backward.cu:69-82
__global__ void tnt_summary_mean_bwd_kernel(const float *__restrict__ d_k_sum, const float *__restrict__ d_v_sum,
                                            float *__restrict__ d_y, int shard_len, int d) {
    const long long total = (long long)shard_len * d;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long long)gridDim.x * blockDim.x) {
        const int j = (int)(i % d);
        d_y[i] += (d_k_sum[j] + d_v_sum[j]) / (float)shard_len;
    }
}
__global__ void add_kernel(const float *__restrict__ a, const float *__restrict__ b, float *__restrict__ out, int n) {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) out[i] = a[i] + b[i];
}

// ── 1-D pooling over groups of C tokens (pool_ops.cu) ────────────────────────
// MODE 0: out[b, g, :] = mean_i x[b, g C + i, :]        (mean_pool forward; serial over i)
// MODE 1: out[b, g, :] = sum_i  x[b, g C + i, :]        (repeat_upsample backward)
template <int MODE>
__global__ void group_reduce_kernel(const float *__restrict__ x, float *__restrict__ out, int bs, int s, int d, int C) {
    const int s_f = s / C;
    const long long total = (long long)bs * s_f * d;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long long)gridDim.x * blockDim.x) {
        const int col = (int)(i % d);
        const long long grp = i / d;
        const int b = (int)(grp / s_f), g = (int)(grp % s_f);
        const float *p = x + ((size_t)b * s + (size_t)g * C) * d + col;
        float sum = 0.f;
        for (int k = 0; k < C; k++) sum += p[(size_t)k * d];
        out[i] = MODE == 0 ? sum / (float)C : sum;
    }
}
// MODE 0: out[b, t, :]  = x[b, t / C, :]                (repeat_upsample forward)
// MODE 1: out[b, t, :] += x[b, t / C, :] * (1 / C)      (mean_pool backward)
// Tokens past the last full group have no group: they are left untouched.
template <int MODE>
__global__ void group_expand_kernel(const float *__restrict__ x, float *__restrict__ out, int bs, int s, int d, int C) {
    const int s_f = s / C;
    const float scale = 1.0f / (float)C;
    const long long total = (long long)bs * s * d;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long long)gridDim.x * blockDim.x) {
        const int col = (int)(i % d);
        const long long tok = i / d;
        const int b = (int)(tok / s), g = (int)(tok % s) / C;
        if (g >= s_f) continue;
        const float v = x[((size_t)b * s_f + g) * d + col];
        if (MODE == 0) out[i] = v;
        else out[i] += v * scale;
    }
}

}  // namespace
}  // namespace nlh

using namespace nlh;

extern "C" {

void layer_norm_forward_cuda(const float *x, const float *gamma, const float *beta, float *out, float *mean_cache,
                             float *rstd_cache, int n, int d, float eps) {
    if (n <= 0 || d <= 0) return;
    hipLaunchKernelGGL(layer_norm_fwd_kernel, dim3(blocks_for(n, kThreads / 64)), dim3(kThreads), 0, stream(), x, gamma,
                       beta, out, mean_cache, rstd_cache, n, d, eps);
    check_launch("layer_norm_fwd_kernel");
}

void layer_norm_backward_cuda(const float *d_out, const float *x, const float *gamma, const float *mean_cache,
                              const float *rstd_cache, float *d_x, float *d_gamma, float *d_beta, int n, int d) {
    const ErrorScope es;
    if (n <= 0 || d <= 0) return;
    const size_t lds = (size_t)(kThreads / 64) * 2 * d * sizeof(float);
    if (lds > 64 * 1024) {
        fail("layer_norm_backward_cuda: d=%d needs more than 64 KB of LDS for the column sums (d <= 2048).", d);
        return;
    }
    const int nblk = blocks_for(n, 64);   // some 64 rows per workgroup, at most 2048 partial rows
    float *part = scratch(5, (size_t)2 * nblk * d * sizeof(float));
    if (es.failed()) return;
    hipLaunchKernelGGL(layer_norm_bwd_kernel, dim3(nblk), dim3(kThreads), lds, stream(), d_out, x,
                       gamma, mean_cache, rstd_cache, d_x, part, n, d);
    check_launch("layer_norm_bwd_kernel");
    hipLaunchKernelGGL(add_partial_rows_kernel, dim3((d + kThreads - 1) / kThreads), dim3(kThreads), 0, stream(), part,
                       d_gamma, d_beta, nblk, d);
    check_launch("add_partial_rows_kernel");
}

void embedding_gather_cuda(const float *w_embed, const int *input_ids, float *output, int seq_len, int d) {
    if (seq_len <= 0 || d <= 0) return;
    hipLaunchKernelGGL(embedding_gather_kernel, dim3(blocks_for((long long)seq_len * d, kThreads)), dim3(kThreads), 0,
                       stream(), w_embed, input_ids, output, seq_len, d);
    check_launch("embedding_gather_kernel");
}

void embedding_scatter_add_cuda(const float *d_embedded, const int *input_ids, float *d_embed, int seq_len, int d) {
    if (seq_len <= 0 || d <= 0) return;
    hipLaunchKernelGGL(embedding_scatter_add_kernel, dim3(blocks_for(seq_len, 1)), dim3(kThreads), 0, stream(),
                       d_embedded, input_ids, d_embed, seq_len, d);
    check_launch("embedding_scatter_add_kernel");
}

void transpose_copy_cuda(const float *src, float *dst, int rows, int cols) {
    if (rows <= 0 || cols <= 0) return;
    const long long tiles = (long long)((rows + 31) / 32) * ((cols + 31) / 32);
    hipLaunchKernelGGL(transpose_copy_kernel, dim3(blocks_for(tiles, 1)), dim3(kThreads), 0, stream(), src, dst, rows,
                       cols);
    check_launch("transpose_copy_kernel");
}

void cross_entropy_forward_cuda(const float *logits, const int *target_ids, float *loss_out, int seq_len, int vocab) {
    const ErrorScope es;
    if (seq_len <= 0 || vocab <= 0) {   // the reference zeroes the loss before anything else
        float *z = scratch(5, sizeof(float));
        if (es.failed()) return;
        hipLaunchKernelGGL(sum_to_scalar_kernel, dim3(1), dim3(kThreads), 0, stream(), z, loss_out, 0);
        check_launch("sum_to_scalar_kernel");
        return;
    }
    float *nll = scratch(5, (size_t)seq_len * sizeof(float));
    if (es.failed()) return;
    hipLaunchKernelGGL(cross_entropy_fwd_kernel, dim3(blocks_for(seq_len, 1)), dim3(kThreads), 0, stream(), logits,
                       target_ids, nll, seq_len, vocab);
    check_launch("cross_entropy_fwd_kernel");
    hipLaunchKernelGGL(sum_to_scalar_kernel, dim3(1), dim3(kThreads), 0, stream(), nll, loss_out, seq_len);
    check_launch("sum_to_scalar_kernel");
}

void cross_entropy_backward_cuda(const float *logits, const int *target_ids, float *d_logits, int seq_len, int vocab,
                                 float inv_count) {
    if (seq_len <= 0 || vocab <= 0) return;
    hipLaunchKernelGGL(cross_entropy_bwd_kernel, dim3(blocks_for(seq_len, 1)), dim3(kThreads), 0, stream(), logits,
                       target_ids, d_logits, seq_len, vocab, inv_count);
    check_launch("cross_entropy_bwd_kernel");
}

void tnt_broadcast_m_f32_cuda(const float *m_src, float *m_dst, int n_local, int d) {
    if (d <= 0 || n_local <= 0) { fail("tnt_broadcast_m_f32_cuda: d=%d and N=%d must be > 0", d, n_local); return; }
    hipLaunchKernelGGL(tnt_broadcast_kernel, dim3(blocks_for((long long)n_local * d * d, kThreads)), dim3(kThreads), 0,
                       stream(), m_src, m_dst, n_local, d * d);
    check_launch("tnt_broadcast_kernel");
}

void tnt_shard_summary_mean_f32_cuda(const float *local_y, float *k_sum, float *v_sum, int shard_len, int d) {
    if (d <= 0 || shard_len <= 0) {
        fail("tnt_shard_summary_mean_f32_cuda: d=%d and shard_len=%d must be > 0", d, shard_len);
        return;
    }
    hipLaunchKernelGGL(tnt_summary_mean_kernel, dim3((d + 63) / 64), dim3(64), 0, stream(), local_y, k_sum, v_sum,
                       shard_len, d);
    check_launch("tnt_summary_mean_kernel");
}

void tnt_global_update_f32_cuda(float *global_m, const float *k_sum, const float *v_sum, int d, float alpha) {
    if (d <= 0) { fail("tnt_global_update_f32_cuda: d=%d must be > 0", d); return; }
    hipLaunchKernelGGL(tnt_global_update_kernel, dim3((d * d + kThreads - 1) / kThreads), dim3(kThreads), 0, stream(),
                       global_m, k_sum, v_sum, d, alpha);
    check_launch("tnt_global_update_kernel");
}

void tnt_global_update_backward_f32_cuda(const float *d_m_new, const float *k_sum, const float *v_sum, float *d_m_old,
                                         float *d_k_sum, float *d_v_sum, int d, float alpha) {
    if (d <= 0) { fail("tnt_global_update_backward_f32_cuda: d=%d must be > 0", d); return; }
    hipLaunchKernelGGL(tnt_global_update_bwd_kernel, dim3((d + 63) / 64), dim3(64), 0, stream(), d_m_new, k_sum, v_sum,
                       d_m_old, d_k_sum, d_v_sum, d, alpha);
    check_launch("tnt_global_update_bwd_kernel");
}

void tnt_shard_summary_mean_backward_f32_cuda(const float *d_k_sum, const float *d_v_sum, float *d_local_y,
                                              int shard_len, int d) {
    if (d <= 0 || shard_len <= 0) {
        fail("tnt_shard_summary_mean_backward_f32_cuda: d=%d and shard_len=%d must be > 0", d, shard_len);
        return;
    }
    hipLaunchKernelGGL(tnt_summary_mean_bwd_kernel, dim3(blocks_for((long long)shard_len * d, kThreads)), dim3(kThreads),
                       0, stream(), d_k_sum, d_v_sum, d_local_y, shard_len, d);
    check_launch("tnt_summary_mean_bwd_kernel");
}

void tnt_combine_gradients_f32_cuda(const float *d_y_upstream, const float *d_y_global, float *d_y_combined, int n) {
    if (n <= 0) return;
    hipLaunchKernelGGL(add_kernel, dim3(blocks_for(n, kThreads)), dim3(kThreads), 0, stream(), d_y_upstream, d_y_global,
                       d_y_combined, n);
    check_launch("add_kernel");
}

static bool pool_args_ok(const char *fn, int bs, int s, int d, int C) {
    if (C <= 0 || d <= 0 || bs < 0 || s < 0) { fail("%s: bs=%d s=%d d=%d C=%d out of range.", fn, bs, s, d, C); return false; }
    return true;
}

void mean_pool_1d_f32_cuda(const float *x, float *out, int bs, int s, int d, int C) {
    if (!pool_args_ok("mean_pool_1d_f32_cuda", bs, s, d, C) || (long long)bs * (s / C) == 0) return;
    hipLaunchKernelGGL(group_reduce_kernel<0>, dim3(blocks_for((long long)bs * (s / C) * d, kThreads)), dim3(kThreads), 0,
                       stream(), x, out, bs, s, d, C);
    check_launch("group_reduce_kernel");
}

void repeat_upsample_1d_f32_cuda(const float *x, float *out, int bs, int s, int d, int C) {
    if (!pool_args_ok("repeat_upsample_1d_f32_cuda", bs, s, d, C) || (long long)bs * s == 0) return;
    hipLaunchKernelGGL(group_expand_kernel<0>, dim3(blocks_for((long long)bs * s * d, kThreads)), dim3(kThreads), 0,
                       stream(), x, out, bs, s, d, C);
    check_launch("group_expand_kernel");
}

void mean_pool_1d_backward_f32_cuda(const float *d_out, float *d_x, int bs, int s, int d, int C) {
    if (!pool_args_ok("mean_pool_1d_backward_f32_cuda", bs, s, d, C) || (long long)bs * s == 0) return;
    hipLaunchKernelGGL(group_expand_kernel<1>, dim3(blocks_for((long long)bs * s * d, kThreads)), dim3(kThreads), 0,
                       stream(), d_out, d_x, bs, s, d, C);
    check_launch("group_expand_kernel");
}

void repeat_upsample_1d_backward_f32_cuda(const float *d_out, float *d_x, int bs, int s, int d, int C) {
    if (!pool_args_ok("repeat_upsample_1d_backward_f32_cuda", bs, s, d, C) || (long long)bs * (s / C) == 0) return;
    hipLaunchKernelGGL(group_reduce_kernel<1>, dim3(blocks_for((long long)bs * (s / C) * d, kThreads)), dim3(kThreads), 0,
                       stream(), d_out, d_x, bs, s, d, C);
    check_launch("group_reduce_kernel");
}

}  // extern "C"
