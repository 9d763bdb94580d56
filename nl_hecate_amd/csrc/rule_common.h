// Device helpers shared by the memory-rule kernels, and the host helpers the
// kernel files share with each other.
#pragma once
#include <hip/hip_runtime.h>

#include "lane_ops.h"
#include "rule_tiles.h"
#include "runtime.h"

namespace nlh {

constexpr int TB = 16;  // tokens per LDS tile

// blockIdx -> (chain, part).  Workgroups are dealt round-robin to the 8 XCDs, so
// consecutive block ids land on different L2s; remap so that the parts of one
// chain (which read the same k/q rows) share an XCD.
__device__ __forceinline__ void map_block(int parts, int &chain, int &part) {
    int n = blockIdx.x, nb = gridDim.x, L = n;
    if (nb % 8 == 0) L = (n % 8) * (nb / 8) + n / 8;
    chain = L / parts;
    part = L % parts;
}

__device__ __forceinline__ bool mnorm_active(float m_norm_max) {
    return m_norm_max > 0.f && m_norm_max < 1e30f;  // core/kernels/m_norm_project.cuh:27
}

__device__ __forceinline__ float4 f4_zero() { return make_float4(0.f, 0.f, 0.f, 0.f); }
__device__ __forceinline__ float4 f4_scale(float a, const float4 &x) {
    return make_float4(a * x.x, a * x.y, a * x.z, a * x.w);
}
// a*x + b*y
__device__ __forceinline__ float4 f4_axpby(float a, const float4 &x, float b, const float4 &y) {
    return make_float4(a * x.x + b * y.x, a * x.y + b * y.y, a * x.z + b * y.z, a * x.w + b * y.w);
}
__device__ __forceinline__ void f4_fma(float4 &acc, float a, const float4 &x) {
    acc.x += a * x.x; acc.y += a * x.y; acc.z += a * x.z; acc.w += a * x.w;
}
__device__ __forceinline__ void f4_add(float4 &acc, const float4 &x) {
    acc.x += x.x; acc.y += x.y; acc.z += x.z; acc.w += x.w;
}

// Workgroup-wide sum of one float per lane (COUPLED kernels only: every wave of
// the workgroup must call it).  `slot` points at kWaves floats of LDS that no
// other reduction uses until the next barrier after this one.
__device__ __forceinline__ float block_allreduce(float x, float *slot, int tid) {
    x = wave_allreduce(x);
    if ((tid & 63) == 0) slot[tid >> 6] = x;
    __syncthreads();
    return slot[0] + slot[1] + slot[2] + slot[3];
}


// ── host helpers (defined in memory_rules.hip) ──────────────────────────────
int n_ckpt_count(int seq_len, int c);  // core/src/gpu_forward.rs:2885-2897
bool check_dims(const char *fn, int seq_len, int d, int batch);
void unsupported(const char *fn, int d, bool coupled);
bool coupled_needed(float error_clip, float m_norm_max);
// dst[i] += sum_b src[b, i]
void accumulate_over_batch(const float *src, float *dst, int batch, int n);
// the same for two pairs in one launch (src_b may be null)
void accumulate_over_batch2(const float *src_a, float *dst_a, const float *src_b, float *dst_b, int batch, int n);
// d_q/d_k/gates = sum over parts of the partial buffers, tokens [t_start, t_end)
void finalize_parts(const float *ws_dq, const float *ws_dk, const float *ws_gate,
                    float *d_q, float *d_k, float *d_alpha, float *d_theta, float *d_eta,
                    int parts, int batch, int seq_len, int d, int t_start, int t_end);

// Checkpointed / chunkwise backward over all segments in one call.
// has_s: Titans (momentum) vs Delta; frozen: frozen-M0 chunkwise rule.
// The fused form returns false when it does not cover (d, C), and, given a bound (m_norm_guard > 0), when the
// replayed states may have reached it (nothing has been added to d_m_initial / d_s_initial then).
bool backward_ckpt_fused(bool has_s, bool frozen, const float *k, const float *v, const float *q,
                         const float *alpha, const float *theta, const float *eta,
                         const float *m_ckpt, const float *s_ckpt, const float *d_y,
                         float *d_k, float *d_v, float *d_q,
                         float *d_alpha, float *d_theta, float *d_eta,
                         float *d_m_initial, float *d_s_initial,
                         int seq_len, int d, int batch, int C, float m_norm_guard = 0.f);

}  // namespace nlh
