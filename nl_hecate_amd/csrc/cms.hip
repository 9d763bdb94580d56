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
#include "optim_steps.h"
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

// ── ErrorBuffer of one frozen level (core/src/conductor.rs:224-261) ─────────
struct nlh_error_buffer {
    std::vector<float *> acc;   // caller-owned device accumulators, one per parameter tensor
    std::vector<int> n;
    long long steps_accumulated;
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
// transposed != 0 reads M_h^T instead: the backward of the read, d_q = M_h^T d_y.
__global__ __launch_bounds__(kCmsThreads) void memory_read_only_kernel(
    const float *__restrict__ q, const float *__restrict__ m, float *__restrict__ y, long long n_tok,
    int nh, int hd, int transposed) {
    extern __shared__ float smem[];
    float *sm = smem;                       // [hd][hd+1]
    float *sq = smem + hd * (hd + 1);       // [64][hd+1]
    const int h = blockIdx.y;
    const long long t0 = (long long)blockIdx.x * 64;
    const int d = nh * hd;
    for (int i = threadIdx.x; i < hd * hd; i += blockDim.x) {
        const int r = i / hd, c = i % hd;
        sm[(transposed ? c * (hd + 1) + r : r * (hd + 1) + c)] = m[(size_t)h * hd * hd + i];
    }
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

// Multi-tensor maps of the ErrorBuffer / ContextState: the pointer table travels in the kernel argument.
constexpr int kEbMax = 24;
struct EbBatch {
    float *dst[kEbMax];
    float *src[kEbMax];
    int n[kEbMax];
    int blk_begin[kEbMax + 1];
    int count;
};
// mode 0: dst += src (accumulate); 1: dst -= lr * src, then src <- 0 (apply_and_reset);
// 2: dst <- 0 (reset); 3: dst <- src (seed)
__global__ void eb_map_kernel(EbBatch b, int mode, float lr) {
    int t = 0;
    while (t + 1 < b.count && (int)blockIdx.x >= b.blk_begin[t + 1]) t++;
    const int nblk = b.blk_begin[t + 1] - b.blk_begin[t], local = blockIdx.x - b.blk_begin[t];
    float *d = b.dst[t];
    float *sp = b.src[t];
    for (int i = local * blockDim.x + threadIdx.x; i < b.n[t]; i += nblk * blockDim.x) {
        if (mode == 0) d[i] += sp[i];
        else if (mode == 1) { d[i] -= lr * sp[i]; sp[i] = 0.f; }
        else if (mode == 2) d[i] = 0.f;
        else d[i] = sp[i];
    }
}
// sum of squares over a tensor list -> out[which] (one workgroup; the lists are a level's parameters)
__global__ void eb_norm_sq_kernel(EbBatch b, int use_src, float *out) {
    __shared__ float part[kCmsThreads / 64];
    float acc = 0.f;
    for (int t = 0; t < b.count; t++) {
        const float *p = use_src ? b.src[t] : b.dst[t];
        for (int i = threadIdx.x; i < b.n[t]; i += blockDim.x) acc = fmaf(p[i], p[i], acc);
    }
    acc = group_allreduce<64>(acc);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        float sum = 0.f;
        for (int w = 0; w < kCmsThreads / 64; w++) sum += part[w];
        out[use_src] = sum;
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
    const bool clip = max_grad_norm > 0.0f;
    if (clip) {
        // the clip factor stays on the device; the update below applies it to the gradients it reads (and writes
        // them back scaled), so only the tensors that take no update this step need a scaling pass of their own
        if (!norm_scale) { fail("nlh_adamw_step: norm_scale must be a device buffer of 2 floats when clipping."); return 1; }
        for (auto &t : o->tensors) { g.push_back(t.g); n.push_back(t.n); }
        unsigned rc = nlh::grad_norm_scale_multi(g.data(), n.data(), (int)nt, max_grad_norm, norm_scale, norm_scale + 1);
        if (rc) return rc;
        g.clear(); n.clear();
        for (auto &t : o->tensors)
            if (t.group >= 0 && (!active_levels || !active_levels[t.group])) { g.push_back(t.g); n.push_back(t.n); }
        if (!g.empty()) {
            rc = nlh::grad_scale_multi(g.data(), n.data(), (int)g.size(), norm_scale + 1);
            if (rc) return rc;
        }
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
    unsigned rc = nlh::adamw_update_multi_scaled(w.data(), (const float *const *)g.data(), m.data(), v.data(),
                                                 n.data(), bc1.data(), bc2.data(), (int)w.size(), lr, o->beta1,
                                                 o->beta2, o->eps, o->weight_decay, clip ? norm_scale + 1 : nullptr);
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
// ── ErrorBuffer (core/src/conductor.rs:224-261) ─────────────────────────────
static bool eb_launch(const std::vector<float *> &dst, const float *const *src, const std::vector<int> &n, int mode,
                      float lr, const char *what) {
    for (size_t first = 0; first < dst.size(); first += nlh::kEbMax) {
        nlh::EbBatch b;
        b.count = 0;
        int blocks = 0;
        for (size_t i = first; i < dst.size() && i < first + nlh::kEbMax; i++) {
            if (n[i] <= 0) continue;
            const int c = b.count++;
            b.dst[c] = dst[i];
            b.src[c] = src ? const_cast<float *>(src[i]) : nullptr;
            b.n[c] = n[i];
            b.blk_begin[c] = blocks;
            const int nb = (n[i] + nlh::kCmsThreads * 4 - 1) / (nlh::kCmsThreads * 4);
            blocks += nb < 1 ? 1 : (nb > 128 ? 128 : nb);
        }
        if (b.count == 0) continue;
        b.blk_begin[b.count] = blocks;
        hipLaunchKernelGGL(nlh::eb_map_kernel, dim3(blocks), dim3(nlh::kCmsThreads), 0, nlh::stream(), b, mode, lr);
        nlh::check_launch(what);
    }
    return true;
}

nlh_error_buffer *nlh_error_buffer_new(void) {
    nlh_error_buffer *b = new nlh_error_buffer();
    b->steps_accumulated = 0;
    return b;
}
void nlh_error_buffer_free(nlh_error_buffer *b) { delete b; }
int nlh_error_buffer_add_tensor(nlh_error_buffer *b, float *accumulator, int n) {
    if (!b || (n > 0 && !accumulator) || n < 0) { nlh::fail("nlh_error_buffer_add_tensor: bad argument"); return -1; }
    b->acc.push_back(accumulator);
    b->n.push_back(n);
    return (int)b->acc.size() - 1;
}
long long nlh_error_buffer_steps(const nlh_error_buffer *b) { return b->steps_accumulated; }
void nlh_error_buffer_accumulate(nlh_error_buffer *b, const float *const *level_grads) {
    eb_launch(b->acc, level_grads, b->n, 0, 0.f, "nlh_error_buffer_accumulate");
    b->steps_accumulated += 1;
}
void nlh_error_buffer_apply_and_reset(nlh_error_buffer *b, float *const *params, float lr) {
    if (b->steps_accumulated <= 0) return;
    std::vector<float *> dst(params, params + b->acc.size());
    eb_launch(dst, b->acc.data(), b->n, 1, lr, "nlh_error_buffer_apply_and_reset");
    b->steps_accumulated = 0;
}
int nlh_error_buffer_health_check(const nlh_error_buffer *b, const float *const *single_step_grads, float *ratio) {
    if (b->acc.size() > (size_t)nlh::kEbMax) { nlh::fail("nlh_error_buffer_health_check: more than %d tensors", nlh::kEbMax); return -1; }
    const nlh::ErrorScope es;
    float *out = nlh::scratch(15, 2 * sizeof(float));
    if (es.failed()) return -1;
    nlh::EbBatch e;
    e.count = 0;
    for (size_t i = 0; i < b->acc.size(); i++) {
        if (b->n[i] <= 0) continue;
        const int c = e.count++;
        e.dst[c] = b->acc[i];
        e.src[c] = const_cast<float *>(single_step_grads[i]);
        e.n[c] = b->n[i];
    }
    hipLaunchKernelGGL(nlh::eb_norm_sq_kernel, dim3(1), dim3(nlh::kCmsThreads), 0, nlh::stream(), e, 0, out);
    hipLaunchKernelGGL(nlh::eb_norm_sq_kernel, dim3(1), dim3(nlh::kCmsThreads), 0, nlh::stream(), e, 1, out);
    nlh::check_launch("nlh_error_buffer_health_check");
    float h[2] = {0.f, 0.f};
    nlh::check_hip(hipMemcpyAsync(h, out, sizeof(h), hipMemcpyDeviceToHost, nlh::stream()), "health_check: copy out");
    nlh::check_hip(hipStreamSynchronize(nlh::stream()), "health_check: synchronize");
    if (es.failed()) return -1;
    const float single = sqrtf(h[1]);
    if (single < 1e-12f) return 0;   // None
    *ratio = sqrtf(h[0]) / single;
    return 1;
}

// ── ContextState (core/src/conductor.rs:156-221) ─────────────────────────────
void nlh_context_state_reset(float *const *buffers, const int *n, int count) {
    std::vector<float *> dst(buffers, buffers + count);
    std::vector<int> nn(n, n + count);
    eb_launch(dst, nullptr, nn, 2, 0.f, "nlh_context_state_reset");
}
void nlh_context_state_seed_self_ref(float *mems, const float *m_k_init, const float *m_v_init, const float *m_q_init,
                                     const float *m_eta_init, const float *m_alpha_init, const float *m_mem_init,
                                     int batch, int d) {
    if (batch <= 0 || d <= 0 || !mems) { nlh::fail("nlh_context_state_seed_self_ref: bad argument"); return; }
    const int dd = d * d;
    // the five projection memories are seeded together or not at all (SelfRefState::from_init)
    const float *proj[5] = {m_k_init, m_v_init, m_q_init, m_eta_init, m_alpha_init};
    const bool have_proj = m_k_init != nullptr;
    if (have_proj && !(m_v_init && m_q_init && m_eta_init && m_alpha_init)) {
        nlh::fail("nlh_context_state_seed_self_ref: m_k_init is given, so m_v/m_q/m_eta/m_alpha_init must be too");
        return;
    }
    std::vector<float *> dst;
    std::vector<const float *> src;
    for (int b = 0; b < batch; b++) {
        float *chain = mems + (size_t)b * 6 * dd;
        if (have_proj)
            for (int c = 0; c < 5; c++) { dst.push_back(chain + (size_t)c * dd); src.push_back(proj[c]); }
        if (m_mem_init) { dst.push_back(chain + (size_t)5 * dd); src.push_back(m_mem_init); }
    }
    std::vector<int> nn(dst.size(), dd);
    eb_launch(dst, src.data(), nn, 3, 0.f, "nlh_context_state_seed_self_ref");
}

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
                       dim3(kCmsThreads), lds, stream(), q_mem, m, y, n_tokens, nh, hd, 0);
    check_launch("memory_read_only_kernel");
}

// Its backward (the frozen-read adapter, core/src/opaque_adapters.rs:1030-1047, per head):
// d_q[t, h*hd+j] = sum_i M[h,i,j] d_y[t, h*hd+i].  No gradient reaches M: the level did not fire.
void memory_read_only_backward_f32_rocm(const float *d_y, const float *m, float *d_q, long long n_tokens, int nh,
                                        int hd) {
    if (n_tokens <= 0 || nh <= 0 || hd <= 0) return;
    const size_t lds = (size_t)(hd + 64) * (hd + 1) * sizeof(float);
    if (lds > 64 * 1024) { fail("memory_read_only_backward_f32_rocm: head_dim=%d too large for the LDS tile.", hd); return; }
    hipLaunchKernelGGL(memory_read_only_kernel, dim3((unsigned)((n_tokens + 63) / 64), nh),
                       dim3(kCmsThreads), lds, stream(), d_y, m, d_q, n_tokens, nh, hd, 1);
    check_launch("memory_read_only_kernel");
}

}  // extern "C"
