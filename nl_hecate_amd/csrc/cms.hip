// CMS (continuum memory system) dispatch: the Conductor / Pulse timing rule, the
// frequency-aware AdamW driver built on it, the level combine + MAG sigmoid gate
// and the read-only path of a frozen level.
//
// Host logic mirrors core/src/conductor.rs and core/src/gpu_optimizer.rs:403-515;
// device work is a handful of fused launches instead of one launch per tensor
// and per elementwise step.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdio.h>

#include <vector>

#include "../../include/nl_hecate_ffi.h"
#include "lane_ops.h"
#include "runtime.h"

// ── Conductor (core/src/conductor.rs:36-155) ────────────────────────────────
struct nlh_conductor {
    int k;
    std::vector<long long> chunk_sizes;
    long long step;
    long long seq_len;
};

// ── frequency-aware AdamW state (core/src/adamw.rs:1-13, gpu_optimizer.rs) ──
struct nlh_adamw_tensor {
    int group;  // -1: always active (attention / aggregation weights); l >= 0: CMS level l
    float *w, *g, *m, *v;
    int n;
    bool clamp;
    float lo, hi;
};
struct nlh_adamw {
    int k;
    float beta1, beta2, eps, weight_decay;
    unsigned step;                     // always-active group's counter
    std::vector<unsigned> level_step;  // per-level counters: advance only when the level fires
    std::vector<nlh_adamw_tensor> tensors;
};

namespace nlh {

constexpr int kCmsThreads = 256;
constexpr int kMaxLevels = 8;

struct LevelPtrs { const float *y[kMaxLevels]; };

// gate = sigmoid(scale * sum_l y_l); gated = attn * gate   (core/src/gpu_forward.rs:1027-1070)
__global__ void cms_combine_gate_kernel(LevelPtrs lv, int k, float scale, const float *__restrict__ attn,
                                        float *__restrict__ y_comb, float *__restrict__ gate,
                                        float *__restrict__ gated, long long n) {
    const long long stride = (long long)gridDim.x * blockDim.x;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        float s = 0.f;
        for (int l = 0; l < k; l++) s += lv.y[l][i];
        s *= scale;
        const float g = 1.0f / (1.0f + expf(-s));
        if (y_comb) y_comb[i] = s;
        gate[i] = g;
        gated[i] = attn[i] * g;
    }
}

// d_attn = d_gated*gate; d_y_comb = d_gated*attn*gate*(1-gate)*scale
// (core/src/gpu_backward.rs:263-283: gating_backward, sigmoid_backward, 1/sqrt(k))
__global__ void cms_gate_backward_kernel(const float *__restrict__ d_gated, const float *__restrict__ attn,
                                         const float *__restrict__ gate, float scale,
                                         float *__restrict__ d_attn, float *__restrict__ d_y, long long n) {
    const long long stride = (long long)gridDim.x * blockDim.x;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const float dg = d_gated[i], g = gate[i];
        d_attn[i] = dg * g;
        d_y[i] = dg * attn[i] * g * (1.0f - g) * scale;
    }
}

// Frozen level: y[t, h*hd + i] = sum_j M[h][i][j] q[t, h*hd + j]
// (core/src/gpu_forward.rs:2906-2950), token-major in and out, no transposes.
// One workgroup per (head, 64-token tile); M_h and the q tile sit in LDS.
__global__ __launch_bounds__(kCmsThreads) void memory_read_only_kernel(
    const float *__restrict__ q, const float *__restrict__ m, float *__restrict__ y, long long n_tok,
    int nh, int hd) {
    extern __shared__ float smem[];
    float *sm = smem;                       // [hd][hd+1]
    float *sq = smem + hd * (hd + 1);       // [64][hd+1]
    const int h = blockIdx.y;
    const long long t0 = (long long)blockIdx.x * 64;
    const int d = nh * hd;
    for (int i = threadIdx.x; i < hd * hd; i += blockDim.x)
        sm[(i / hd) * (hd + 1) + i % hd] = m[(size_t)h * hd * hd + i];
    for (int i = threadIdx.x; i < 64 * hd; i += blockDim.x) {
        const long long t = t0 + i / hd;
        sq[(i / hd) * (hd + 1) + i % hd] = t < n_tok ? q[t * d + h * hd + i % hd] : 0.f;
    }
    __syncthreads();
    for (int o = threadIdx.x; o < 64 * hd; o += blockDim.x) {
        const int tt = o / hd, i = o % hd;
        const long long t = t0 + tt;
        if (t >= n_tok) continue;
        float acc = 0.f;
        for (int j = 0; j < hd; j++) acc += sm[i * (hd + 1) + j] * sq[tt * (hd + 1) + j];
        y[t * d + h * hd + i] = acc;
    }
}

static int blocks_for(long long n) {
    long long b = (n + kCmsThreads - 1) / kCmsThreads;
    return (int)(b < 1 ? 1 : (b > 4096 ? 4096 : b));
}

}  // namespace nlh

using namespace nlh;

extern "C" {

// ── Conductor ────────────────────────────────────────────────────────────────
nlh_conductor *nlh_conductor_new(int k, const long long *chunk_sizes) {
    if (k < 1 || k > kMaxLevels) { fail("nlh_conductor_new: k=%d must be in [1, %d].", k, kMaxLevels); return nullptr; }
    for (int i = 0; i < k; i++)
        if (chunk_sizes[i] < 1) { fail("nlh_conductor_new: chunk_sizes[%d] must be >= 1.", i); return nullptr; }
    nlh_conductor *c = new nlh_conductor();
    c->k = k;
    c->chunk_sizes.assign(chunk_sizes, chunk_sizes + k);
    c->step = 0;
    c->seq_len = 0;
    return c;
}
void nlh_conductor_free(nlh_conductor *c) { delete c; }
void nlh_conductor_set_seq_len(nlh_conductor *c, long long seq_len) { c->seq_len = seq_len; }
long long nlh_conductor_step(const nlh_conductor *c) { return c->step; }
void nlh_conductor_advance(nlh_conductor *c) { c->step += 1; }

// Pulse for the current step (core/src/conductor.rs:136-144); active[k] receives 0/1;
// returns the bitmask (bit l = level l active, core/src/gpu_forward.rs:2449-2457).
unsigned nlh_conductor_pulse(const nlh_conductor *c, int *active) {
    unsigned mask = 0;
    for (int l = 0; l < c->k; l++) {
        const long long cs = c->chunk_sizes[l];
        const int a = (c->step % cs == 0) || (c->seq_len > 0 && c->seq_len >= cs);
        if (active) active[l] = a;
        if (a && l < 8) mask |= 1u << l;
    }
    return mask;
}

unsigned nlh_pulse_to_bitmask(const int *active, int k) {
    unsigned mask = 0;
    for (int i = 0; i < (k < 8 ? k : 8); i++)
        if (active[i]) mask |= 1u << i;
    return mask;
}

// Restore (core/src/conductor.rs:105-128): 0 ok; 1 config mismatch (k or chunk
// sizes differ); 2 pulse mismatch (stream cursor's pulse id != saved step).
int nlh_conductor_restore(nlh_conductor *c, int k, const long long *chunk_sizes, long long step,
                          long long stream_pulse_id) {
    if (k != c->k) return 1;
    for (int i = 0; i < k; i++)
        if (chunk_sizes[i] != c->chunk_sizes[i]) return 1;
    if (stream_pulse_id != step) return 2;
    c->step = step;
    return 0;
}

// ── frequency-aware AdamW ───────────────────────────────────────────────────
nlh_adamw *nlh_adamw_new(int k, float beta1, float beta2, float eps, float weight_decay) {
    if (k < 0 || k > kMaxLevels) { fail("nlh_adamw_new: k=%d out of range.", k); return nullptr; }
    nlh_adamw *o = new nlh_adamw();
    o->k = k;
    o->beta1 = beta1; o->beta2 = beta2; o->eps = eps; o->weight_decay = weight_decay;
    o->step = 0;
    o->level_step.assign(k, 0);
    return o;
}
void nlh_adamw_free(nlh_adamw *o) { delete o; }

// group -1: always-active tensors; group l in [0,k): tensors of CMS level l.
// m and v are caller-owned device buffers of n floats (zero-initialised).
int nlh_adamw_add_tensor(nlh_adamw *o, int group, float *w, float *g, float *m, float *v, int n) {
    if (group < -1 || group >= o->k) { fail("nlh_adamw_add_tensor: group %d out of range.", group); return -1; }
    o->tensors.push_back(nlh_adamw_tensor{group, w, g, m, v, n, false, 0.f, 0.f});
    return (int)o->tensors.size() - 1;
}
// Post-update clamp of a tensor (b_theta in [-10, 2], core/src/gpu_optimizer.rs:491-493).
void nlh_adamw_set_clamp(nlh_adamw *o, int tensor, float lo, float hi) {
    if (tensor < 0 || tensor >= (int)o->tensors.size()) { fail("nlh_adamw_set_clamp: bad tensor id %d.", tensor); return; }
    o->tensors[tensor].clamp = true;
    o->tensors[tensor].lo = lo;
    o->tensors[tensor].hi = hi;
}
unsigned nlh_adamw_swa_step(const nlh_adamw *o) { return o->step; }
unsigned nlh_adamw_level_step(const nlh_adamw *o, int level) {
    return (level >= 0 && level < o->k) ? o->level_step[level] : 0;
}

// One optimizer step (core/src/gpu_optimizer.rs:403-515).  The global L2 norm
// runs over every registered gradient; norm_scale (device, 2 floats) receives
// {norm, scale} and the clip is applied on device without a host read-back.
// Levels whose pulse is off are skipped entirely: no update, no counter advance.
unsigned nlh_adamw_step(nlh_adamw *o, const int *active_levels, float lr, float max_grad_norm,
                        float *norm_scale) {
    const size_t nt = o->tensors.size();
    std::vector<float *> w, g, m, v;
    std::vector<int> n;
    std::vector<float> bc1, bc2;
    if (max_grad_norm > 0.0f) {
        if (!norm_scale) { fail("nlh_adamw_step: norm_scale must be a device buffer of 2 floats when clipping."); return 1; }
        for (auto &t : o->tensors) { g.push_back(t.g); n.push_back(t.n); }
        unsigned rc = grad_norm_clip_multi_rocm(g.data(), n.data(), (int)nt, max_grad_norm, norm_scale,
                                                norm_scale + 1);
        if (rc) return rc;
        g.clear(); n.clear();
    }
    o->step += 1;
    const float t0 = (float)o->step;
    const float sbc1 = 1.0f / (1.0f - powf(o->beta1, t0)), sbc2 = 1.0f / (1.0f - powf(o->beta2, t0));
    std::vector<float> lbc1(o->k, 0.f), lbc2(o->k, 0.f);
    for (int l = 0; l < o->k; l++) {
        if (!active_levels || !active_levels[l]) continue;
        o->level_step[l] += 1;
        const float lt = (float)o->level_step[l];
        lbc1[l] = 1.0f / (1.0f - powf(o->beta1, lt));
        lbc2[l] = 1.0f / (1.0f - powf(o->beta2, lt));
    }
    for (auto &t : o->tensors) {
        if (t.group >= 0 && (!active_levels || !active_levels[t.group])) continue;
        w.push_back(t.w); g.push_back(t.g); m.push_back(t.m); v.push_back(t.v); n.push_back(t.n);
        bc1.push_back(t.group < 0 ? sbc1 : lbc1[t.group]);
        bc2.push_back(t.group < 0 ? sbc2 : lbc2[t.group]);
    }
    unsigned rc = adamw_update_multi_rocm(w.data(), (const float *const *)g.data(), m.data(), v.data(),
                                          n.data(), bc1.data(), bc2.data(), (int)w.size(), lr, o->beta1,
                                          o->beta2, o->eps, o->weight_decay);
    if (rc) return rc;
    for (auto &t : o->tensors)
        if (t.clamp && (t.group < 0 || (active_levels && active_levels[t.group])))
            clamp_f32_cuda(t.w, t.n, t.lo, t.hi);
    return 0;
}

// ── level combine + MAG gate ────────────────────────────────────────────────
// gate = sigmoid(c * sum_l y_l), gated = attn_out * gate, c = 1/sqrt(k) for k > 2
// else 1 (core/src/gpu_forward.rs:1027-1070; mag.rs:709-718).  y_levels is a
// HOST array of k device pointers; y_combined may be NULL.
void cms_combine_gate_rocm(const float *const *y_levels, int k, const float *attn_out,
                           float *y_combined, float *gate, float *gated, long long n) {
    if (k < 1 || k > kMaxLevels) { fail("cms_combine_gate_rocm: k=%d must be in [1, %d].", k, kMaxLevels); return; }
    if (n <= 0) return;
    LevelPtrs lv;
    for (int l = 0; l < k; l++) lv.y[l] = y_levels[l];
    const float scale = k > 2 ? 1.0f / sqrtf((float)k) : 1.0f;
    hipLaunchKernelGGL(cms_combine_gate_kernel, dim3(blocks_for(n)), dim3(kCmsThreads), 0, stream(), lv, k,
                       scale, attn_out, y_combined, gate, gated, n);
    check_launch("cms_combine_gate_kernel");
}

// d_attn = d_gated*gate; d_y_combined = d_gated*attn_out*gate*(1-gate)*c — the
// same d_y_combined is handed to every level (core/src/gpu_backward.rs:263-331).
void cms_gate_backward_rocm(const float *d_gated, const float *attn_out, const float *gate, int k,
                            float *d_attn, float *d_y_combined, long long n) {
    if (n <= 0) return;
    const float scale = k > 2 ? 1.0f / sqrtf((float)k) : 1.0f;
    hipLaunchKernelGGL(cms_gate_backward_kernel, dim3(blocks_for(n)), dim3(kCmsThreads), 0, stream(),
                       d_gated, attn_out, gate, scale, d_attn, d_y_combined, n);
    check_launch("cms_gate_backward_kernel");
}

// Frozen level read: y[t, h*hd+i] = sum_j M[h,i,j] q[t, h*hd+j]; m is [nh, hd, hd].
void memory_read_only_f32_rocm(const float *q_mem, const float *m, float *y, long long n_tokens, int nh,
                               int hd) {
    if (n_tokens <= 0 || nh <= 0 || hd <= 0) return;
    const size_t lds = (size_t)(hd + 64) * (hd + 1) * sizeof(float);
    if (lds > 64 * 1024) { fail("memory_read_only_f32_rocm: head_dim=%d too large for the LDS tile.", hd); return; }
    hipLaunchKernelGGL(memory_read_only_kernel, dim3((unsigned)((n_tokens + 63) / 64), nh),
                       dim3(kCmsThreads), lds, stream(), q_mem, m, y, n_tokens, nh, hd);
    check_launch("memory_read_only_kernel");
}

}  // extern "C"
