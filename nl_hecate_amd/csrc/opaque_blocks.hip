// Opaque VJP blocks of the Wengert tape on the GPU: the backward adapters that the tape's registry
// maps an OpaqueKey to (core/src/tape.rs:100-150, core/src/opaque_adapters.rs:1731-1760), with the
// reference's saved-buffer layouts, for host slices (the tape is a CPU structure).
//
//   nlh_opaque_backward(key, d_outputs, saved, d_inputs): stages the saved buffers of one block on the
//   device, runs the block's backward there and ADDS the result into the caller's d_inputs (the tape
//   accumulates what an adapter returns into its gradient buffers, tape.rs:839-866; here that sum is
//   part of the call, so d_inputs may hold gradients from other consumers of the same buffers).
//
// Blocks: DeltaRule and TitansLMM (inputs [embedded, level_params_flat]; opaque_adapters.rs:290-380,
// :386-592: token recurrence backward, gate backward with the gates' feedback into k and v and the
// straight-through clamp masks of delta_rule.rs:560-569 / titans_lmm.rs:1707-1724, row L2 norm
// backward, projection backward against the bf16 copy of the matrices), DGD (:1680-1725), SWA
// (:952-997) and the frozen read-only variants (:1004-1072).  Default configuration only: L2
// attentional bias, identity feature map, no Conv1D, linear memory, EMA momentum; anything else in the
// metadata is refused with a message (the reference falls back to its CPU adapter there).
#include <hip/hip_runtime.h>
#include <rocblas/rocblas.h>
#include <stdint.h>
#include <string.h>

#include <vector>

#include "../../include/nl_hecate_ffi.h"
#include "runtime.h"

namespace nlh {
namespace {

constexpr int kThr = 256;
inline int blocks_for(size_t n) {
    const size_t b = (n + kThr - 1) / kThr;
    return (int)(b < 1 ? 1 : (b > 4096 ? 4096 : b));
}

template <typename T>
struct Dev {
    T *ptr = nullptr;
    size_t n;
    explicit Dev(size_t count) : n(count) {
        check_hip(hipMalloc(reinterpret_cast<void **>(&ptr), (n ? n : 1) * sizeof(T)), "opaque block: hipMalloc");
    }
    ~Dev() { if (ptr) (void)hipFree(ptr); }
    Dev(const Dev &) = delete;
    Dev &operator=(const Dev &) = delete;
    void from_host(const T *src) {
        if (ptr && n) check_hip(hipMemcpyAsync(ptr, src, n * sizeof(T), hipMemcpyHostToDevice, stream()), "opaque block: copy in");
    }
    void zero() {
        if (ptr && n) check_hip(hipMemsetAsync(ptr, 0, n * sizeof(T), stream()), "opaque block: zero");
    }
    std::vector<T> to_host() {
        std::vector<T> h(n);
        if (ptr && n) check_hip(hipMemcpy(h.data(), ptr, n * sizeof(T), hipMemcpyDeviceToHost), "opaque block: copy out");
        return h;
    }
};

rocblas_handle blas() {
    static rocblas_handle h = nullptr;
    if (!h && rocblas_create_handle(&h) != rocblas_status_success) {
        h = nullptr;
        fail("opaque block: rocblas_create_handle failed.");
        return nullptr;
    }
    if (rocblas_set_stream(h, stream()) != rocblas_status_success) {
        fail("opaque block: rocblas_set_stream failed.");
        return nullptr;
    }
    return h;
}
// Row-major C [m, n] = beta C + A B with A [m, k] (or its transpose, stored [k, m]) and B [k, n].
bool gemm_rm(bool trans_a, int m, int n, int k, const float *A, const float *B, float beta, float *C) {
    rocblas_handle h = blas();
    if (!h) return false;
    const float one = 1.0f;
    // column-major view: C^T [n, m] = B^T [n, k] A^T [k, m]; a row-major matrix is its transpose column-major
    const rocblas_status st =
        rocblas_sgemm(h, rocblas_operation_none, trans_a ? rocblas_operation_transpose : rocblas_operation_none, n, m,
                      k, &one, B, n, A, trans_a ? m : k, &beta, C, n);
    if (st != rocblas_status_success) { fail("opaque block: rocblas_sgemm failed with status %d.", (int)st); return false; }
    return true;
}

__device__ __forceinline__ float sigmoid_ref(float x) {   // tensor.rs:202-207
    return x >= 15.f ? 1.f : (x <= -15.f ? 0.f : 1.f / (1.f + expf(-x)));
}
__device__ __forceinline__ float softplus_ref(float x) {   // tensor.rs:222-227
    return x >= 15.f ? x : (x <= -15.f ? 0.f : logf(1.f + expf(x)));
}

// Gate pre-activation gradients with the rule's straight-through clamp masks.
// titans: masks on the unclamped alpha and theta (titans_lmm.rs:1707-1719); delta: theta mask on the
// clamped value, none for alpha (delta_rule.rs:560-569).
__global__ void gate_pre_kernel(const float *d_alpha, const float *alpha, const float *alpha_pre, const float *d_theta,
                                const float *theta, const float *theta_pre, const float *d_eta, const float *eta,
                                float *pre, int s, int titans, float a_lo, float a_hi, float t_lo, float t_hi) {
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= s) return;
    float da = d_alpha[t] * alpha[t] * (1.f - alpha[t]);
    float t_raw = theta[t];
    if (titans) {
        const float a_raw = sigmoid_ref(alpha_pre[t]);
        if (a_raw <= a_lo || a_raw >= a_hi) da = 0.f;
        t_raw = softplus_ref(theta_pre[t]);
    }
    float dt = d_theta[t] * sigmoid_ref(theta_pre[t]);
    if (t_raw <= t_lo || t_raw >= t_hi) dt = 0.f;
    pre[t] = da;
    pre[s + t] = dt;
    pre[2 * s + t] = titans ? d_eta[t] * eta[t] * (1.f - eta[t]) : 0.f;
}

// grads of the gate vectors and biases: out[g][c] = sum_t pre[g][t] concat[t][c] (c < 2d), out[g][2d] = sum_t pre[g][t];
// one thread per (gate, column), tokens in order (reproducible)
__global__ void gate_weight_grads_kernel(const float *pre, const float *k, const float *v, float *out, int s, int d) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x, g = blockIdx.y;
    if (c > 2 * d) return;
    const float *p = pre + (size_t)g * s;
    float acc = 0.f;
    if (c == 2 * d) {
        for (int t = 0; t < s; t++) acc += p[t];
    } else {
        const float *src = c < d ? k + c : v + (c - d);
        for (int t = 0; t < s; t++) acc = fmaf(p[t], src[(size_t)t * d], acc);
    }
    out[(size_t)g * (2 * d + 1) + c] = acc;
}

// concat backward: the gates read k and v (w [3][2d + 1] = gate vectors as stored in the flat buffer, with bias)
__global__ void gate_feedback_kernel(const float *pre, const float *w_alpha, const float *w_theta, const float *w_eta,
                                     float *d_k, float *d_v, int s, int d, int titans) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)s * d) return;
    const int t = (int)(i / d), c = (int)(i % d);
    const float pa = pre[t], pt = pre[s + t], pe = titans ? pre[2 * s + t] : 0.f;
    d_k[i] += pa * w_alpha[c] + pt * w_theta[c] + (titans ? pe * w_eta[c] : 0.f);
    d_v[i] += pa * w_alpha[d + c] + pt * w_theta[d + c] + (titans ? pe * w_eta[d + c] : 0.f);
}

// d_q[t] = M^T d_y[t]  (frozen read, opaque_adapters.rs:1030-1047)
__global__ void frozen_read_backward_kernel(const float *m, const float *d_y, float *d_q, int s, int d) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)s * d) return;
    const int t = (int)(i / d), c = (int)(i % d);
    float acc = 0.f;
    for (int j = 0; j < d; j++) acc = fmaf(m[(size_t)j * d + c], d_y[(size_t)t * d + j], acc);
    d_q[i] = acc;
}

struct Slices {
    const float *const *ptr;
    const long long *len;
    int n;
    const float *operator[](int i) const { return ptr[i]; }
};

bool want(const char *what, const Slices &sl, int i, long long n) {
    if (i >= sl.n) { fail("nlh_opaque_backward: %s (buffer %d) is missing: %d buffers given", what, i, sl.n); return false; }
    if (sl.len[i] != n) { fail("nlh_opaque_backward: %s has %lld elements, expected %lld", what, sl.len[i], n); return false; }
    return true;
}

void add_into(float *dst, const std::vector<float> &src, size_t n) {
    for (size_t i = 0; i < n; i++) dst[i] += src[i];
}

int rule_block_backward(bool titans, const Slices &dout, const Slices &saved, float *const *d_inputs,
                        const long long *d_input_lens, int n_inputs) {
    const ErrorScope es;
    const char *name = titans ? "TitansLMM" : "DeltaRule";
    const float *meta = saved[0];
    const long long ml = saved.len[0];
    if (ml < (titans ? 16 : 12)) {
        fail("nlh_opaque_backward(%s): metadata of %lld values is an older recording format (needs %d)", name, ml,
             titans ? 16 : 12);
        return 2;
    }
    const int s = (int)meta[0], d = (int)meta[1];
    const float bias = meta[2];
    const int o = titans ? 1 : 0;   // the Titans metadata carries momentum_kind at [4]
    const float t_lo = meta[4 + o], t_hi = meta[5 + o], fm_kind = meta[6 + o], a_lo = meta[9 + o], a_hi = meta[10 + o];
    const float kernel_size = meta[ml - 1];
    if (bias != 2.0f || fm_kind != 0.0f || kernel_size != 0.0f || (titans && (meta[4] != 1.0f || meta[12] != 1.0f))) {
        fail("nlh_opaque_backward(%s): only the default block is built (L2 bias, identity feature map, no Conv1D%s); "
             "metadata says bias=%g fm_kind=%g kernel_size=%g%s", name, titans ? ", EMA momentum, linear memory" : "",
             (double)bias, (double)fm_kind, (double)kernel_size, titans ? " (see momentum_kind, memory_layers)" : "");
        return 2;
    }
    if (s <= 0 || d <= 0) { fail("nlh_opaque_backward(%s): seq_len=%d d=%d", name, s, d); return 2; }
    const long long sd = (long long)s * d, dd = (long long)d * d, traj = (long long)(s + 1) * dd;
    const long long flat_min = 3 * dd + 6 * d + 3;
    // saved order: meta, level_params_flat, embedded, then the cache fields (see the file header)
    const int iM = 3, iS = titans ? 4 : -1, iK = titans ? 5 : 4, iV = iK + 1, iQ = iK + 2, iAP = iK + 4, iA = iK + 5,
              iTP = iK + 6, iT = iK + 7, iEP = titans ? iK + 8 : -1, iE = titans ? iK + 9 : -1,
              iKN = titans ? 18 : 15, iQN = iKN + 1;
    if (saved.n <= iQN) { fail("nlh_opaque_backward(%s): %d saved buffers, expected at least %d", name, saved.n, iQN + 1); return 2; }
    if (saved.len[1] < flat_min) { fail("nlh_opaque_backward(%s): level_params_flat has %lld values, expected >= %lld", name, saved.len[1], flat_min); return 2; }
    if (!want("embedded", saved, 2, sd) || !want("m_states", saved, iM, traj) || !want("k_mem", saved, iK, sd) ||
        !want("v_mem", saved, iV, sd) || !want("q_mem", saved, iQ, sd) || !want("alpha_pre", saved, iAP, s) ||
        !want("alpha", saved, iA, s) || !want("theta_pre", saved, iTP, s) || !want("theta", saved, iT, s) ||
        !want("k_mem_norms", saved, iKN, s) || !want("q_mem_norms", saved, iQN, s))
        return 2;
    if (titans && (!want("s_states", saved, iS, traj) || !want("eta_pre", saved, iEP, s) || !want("eta", saved, iE, s))) return 2;
    if (dout.n < 1 || dout.len[0] != sd) { fail("nlh_opaque_backward(%s): d_outputs[0] must hold %lld values", name, sd); return 2; }
    if (n_inputs < 2 || d_input_lens[0] != sd || d_input_lens[1] < flat_min) {
        fail("nlh_opaque_backward(%s): d_inputs must be [d_embedded (%lld), d_level_params (>= %lld)]", name, sd, flat_min);
        return 2;
    }

    Dev<float> emb(sd), lp(flat_min), ms(traj), ss(titans ? traj : 1), k(sd), v(sd), q(sd), gates(8 * (size_t)s), kn(s),
        qn(s), dy(sd);
    Dev<float> dk(sd), dv(sd), dq(sd), dg(3 * (size_t)s), dm(2 * dd), pre(3 * (size_t)s), gw(3 * (size_t)(2 * d + 1)),
        dkr(sd), dqr(sd), wr(3 * dd), dw(3 * dd), demb(sd);
    Dev<uint16_t> wb(3 * dd);
    if (es.failed()) return 3;
    emb.from_host(saved[2]); lp.from_host(saved[1]); ms.from_host(saved[iM]);
    k.from_host(saved[iK]); v.from_host(saved[iV]); q.from_host(saved[iQ]);
    kn.from_host(saved[iKN]); qn.from_host(saved[iQN]); dy.from_host(dout[0]);
    float *g_ap = gates.ptr, *g_a = g_ap + s, *g_tp = g_a + s, *g_t = g_tp + s, *g_ep = g_t + s, *g_e = g_ep + s;
    const size_t sb = (size_t)s * sizeof(float);
    check_hip(hipMemcpyAsync(g_ap, saved[iAP], sb, hipMemcpyHostToDevice, stream()), "opaque block: copy in");
    check_hip(hipMemcpyAsync(g_a, saved[iA], sb, hipMemcpyHostToDevice, stream()), "opaque block: copy in");
    check_hip(hipMemcpyAsync(g_tp, saved[iTP], sb, hipMemcpyHostToDevice, stream()), "opaque block: copy in");
    check_hip(hipMemcpyAsync(g_t, saved[iT], sb, hipMemcpyHostToDevice, stream()), "opaque block: copy in");
    if (titans) {
        ss.from_host(saved[iS]);
        check_hip(hipMemcpyAsync(g_ep, saved[iEP], sb, hipMemcpyHostToDevice, stream()), "opaque block: copy in");
        check_hip(hipMemcpyAsync(g_e, saved[iE], sb, hipMemcpyHostToDevice, stream()), "opaque block: copy in");
    }
    dk.zero(); dv.zero(); dq.zero(); dg.zero(); dm.zero();
    if (es.failed()) return 3;
    // 1. the token recurrence in reverse (one chain, memory d x d)
    float *d_al = dg.ptr, *d_th = d_al + s, *d_et = d_th + s;
    if (titans)
        titans_backward_f32_cuda(k.ptr, v.ptr, q.ptr, g_a, g_t, g_e, ms.ptr, ss.ptr, dy.ptr, dk.ptr, dv.ptr, dq.ptr, d_al,
                                 d_th, d_et, dm.ptr, dm.ptr + dd, s, d, 1, 0.0f);
    else
        delta_backward_f32_cuda(k.ptr, v.ptr, q.ptr, g_a, g_t, ms.ptr, dy.ptr, dk.ptr, dv.ptr, dq.ptr, d_al, d_th, dm.ptr,
                                s, d, 1, 0.0f);
    if (es.failed()) return 3;
    // 2. gates: pre-activation gradients, gate vector / bias gradients, feedback into k and v
    const float *w_alpha = lp.ptr + 3 * dd, *w_theta = w_alpha + 2 * d + 1, *w_eta = w_theta + 2 * d + 1;
    hipLaunchKernelGGL(gate_pre_kernel, dim3(blocks_for(s)), dim3(kThr), 0, stream(), d_al, g_a, g_ap, d_th, g_t, g_tp,
                       d_et, g_e, pre.ptr, s, titans ? 1 : 0, a_lo, a_hi, t_lo, t_hi);
    hipLaunchKernelGGL(gate_weight_grads_kernel, dim3(blocks_for(2 * d + 1), 3), dim3(kThr), 0, stream(), pre.ptr, k.ptr,
                       v.ptr, gw.ptr, s, d);
    hipLaunchKernelGGL(gate_feedback_kernel, dim3(blocks_for(sd)), dim3(kThr), 0, stream(), pre.ptr, w_alpha, w_theta,
                       w_eta, dk.ptr, dv.ptr, s, d, titans ? 1 : 0);
    check_launch("opaque block gate kernels");
    // 3. row L2 norm of k and q
    l2_normalize_backward_f32_cuda(dk.ptr, k.ptr, kn.ptr, dkr.ptr, s, d, 1e-8f);
    l2_normalize_backward_f32_cuda(dq.ptr, q.ptr, qn.ptr, dqr.ptr, s, d, 1e-8f);
    // 4. projections: weight gradients against embedded, input gradient against the bf16 copy of the matrices
    f32_to_bf16_cuda(lp.ptr, wb.ptr, (int)(3 * dd));
    bf16_to_f32_cuda(wb.ptr, wr.ptr, (int)(3 * dd));
    const float *grads_in[3] = {dkr.ptr, dv.ptr, dqr.ptr};
    for (int i = 0; i < 3; i++) {
        if (!gemm_rm(true, d, d, s, grads_in[i], emb.ptr, 0.0f, dw.ptr + (size_t)i * dd)) return 3;   // dW = d_x^T embedded
        if (!gemm_rm(false, s, d, d, grads_in[i], wr.ptr + (size_t)i * dd, i ? 1.0f : 0.0f, demb.ptr)) return 3;
    }
    if (es.failed()) return 3;
    check_hip(hipStreamSynchronize(stream()), "opaque block: synchronize");
    if (es.failed()) return 3;
    // 5. add into the caller's buffers: d_embedded, then the flat parameter gradient (fields the rule
    //    does not produce stay as they are: level_params_grads_to_flat_padded adds zeros there)
    add_into(d_inputs[0], demb.to_host(), (size_t)sd);
    float *flat = d_inputs[1];
    add_into(flat, dw.to_host(), (size_t)(3 * dd));
    const std::vector<float> gwh = gw.to_host();
    for (int g = 0; g < (titans ? 3 : 2); g++)
        for (int c = 0; c <= 2 * d; c++) flat[3 * dd + (size_t)g * (2 * d + 1) + c] += gwh[(size_t)g * (2 * d + 1) + c];
    return es.failed() ? 3 : 0;
}

int dgd_block_backward(const Slices &dout, const Slices &saved, float *const *d_inputs, const long long *d_input_lens,
                       int n_inputs) {
    // saved: [meta = [seq_len, d, (error_clip)], k_mem, v_mem, q_mem, alpha, theta, m_states]
    if (saved.n < 7 || saved.len[0] < 2) { fail("nlh_opaque_backward(DGD): 7 saved buffers expected, got %d", saved.n); return 2; }
    const int s = (int)saved[0][0], d = (int)saved[0][1];
    const float clip = saved.len[0] > 2 ? saved[0][2] : 0.0f;
    const long long sd = (long long)s * d, dd = (long long)d * d;
    if (s <= 0 || d <= 0) { fail("nlh_opaque_backward(DGD): seq_len=%d d=%d", s, d); return 2; }
    if (!want("k_mem", saved, 1, sd) || !want("v_mem", saved, 2, sd) || !want("q_mem", saved, 3, sd) ||
        !want("alpha", saved, 4, s) || !want("theta", saved, 5, s) || !want("m_states", saved, 6, (long long)(s + 1) * dd))
        return 2;
    const long long need[6] = {sd, sd, sd, s, s, dd};
    if (n_inputs < 6 || dout.n < 1 || dout.len[0] != sd) { fail("nlh_opaque_backward(DGD): 6 d_inputs and d_y [seq_len*d] expected"); return 2; }
    for (int i = 0; i < 6; i++)
        if (d_input_lens[i] != need[i]) { fail("nlh_opaque_backward(DGD): d_inputs[%d] has %lld values, expected %lld", i, d_input_lens[i], need[i]); return 2; }
    std::vector<std::vector<float>> g(6);
    for (int i = 0; i < 6; i++) g[i].assign((size_t)need[i], 0.f);
    const ErrorScope es;
    nlh_dgd_backward_dispatch(saved[1], saved[2], saved[3], saved[4], saved[5], saved[6], dout[0], g[0].data(), g[1].data(),
                              g[2].data(), g[3].data(), g[4].data(), g[5].data(), s, d, clip);
    if (es.failed()) return 3;
    for (int i = 0; i < 6; i++) add_into(d_inputs[i], g[i], (size_t)need[i]);
    return 0;
}

int swa_block_backward(const Slices &dout, const Slices &saved, float *const *d_inputs, const long long *d_input_lens,
                       int n_inputs) {
    // saved: [meta = [seq_len, num_heads, head_dim, window_size], q, k, v, attn_weights]
    if (saved.n < 5 || saved.len[0] < 4) { fail("nlh_opaque_backward(SWA): 5 saved buffers expected, got %d", saved.n); return 2; }
    const int s = (int)saved[0][0], nh = (int)saved[0][1], hd = (int)saved[0][2], ws = (int)saved[0][3];
    const long long full = (long long)s * nh * hd;
    if (s <= 0 || nh <= 0 || hd <= 0 || ws <= 0) { fail("nlh_opaque_backward(SWA): bad metadata"); return 2; }
    if (!want("q", saved, 1, full) || !want("k", saved, 2, full) || !want("v", saved, 3, full) ||
        !want("attn_weights", saved, 4, (long long)nh * s * ws))
        return 2;
    if (n_inputs < 3 || dout.n < 1 || dout.len[0] != full || d_input_lens[0] != full || d_input_lens[1] != full ||
        d_input_lens[2] != full) {
        fail("nlh_opaque_backward(SWA): d_outputs[0] and d_inputs[0..2] must hold %lld values each", full);
        return 2;
    }
    std::vector<float> dq((size_t)full, 0.f), dk((size_t)full, 0.f), dv((size_t)full, 0.f);
    const ErrorScope es;
    nlh_swa_backward_dispatch(saved[1], saved[2], saved[3], saved[4], dout[0], dq.data(), dk.data(), dv.data(), s, nh, hd, ws);
    if (es.failed()) return 3;
    add_into(d_inputs[0], dq, (size_t)full);
    add_into(d_inputs[1], dk, (size_t)full);
    add_into(d_inputs[2], dv, (size_t)full);
    return 0;
}

int frozen_block_backward(const Slices &dout, const Slices &saved, float *const *d_inputs, const long long *d_input_lens,
                          int n_inputs) {
    // saved: [meta = [seq_len, d] (identity feature map), m_frozen [d*d]]; d_inputs[0] = d_q
    if (saved.n < 2 || saved.len[0] < 2) { fail("nlh_opaque_backward(frozen read): 2 saved buffers expected, got %d", saved.n); return 2; }
    if (saved.len[0] != 2 && !(saved.len[0] >= 4 && saved[0][2] == 0.0f)) {
        fail("nlh_opaque_backward(frozen read): only the identity feature map and a linear memory are built");
        return 2;
    }
    const int s = (int)saved[0][0], d = (int)saved[0][1];
    const long long sd = (long long)s * d;
    if (s <= 0 || d <= 0) { fail("nlh_opaque_backward(frozen read): seq_len=%d d=%d", s, d); return 2; }
    if (!want("m_frozen", saved, 1, (long long)d * d)) return 2;
    if (n_inputs < 1 || dout.n < 1 || dout.len[0] != sd || d_input_lens[0] != sd) {
        fail("nlh_opaque_backward(frozen read): d_outputs[0] and d_inputs[0] must hold %lld values", sd);
        return 2;
    }
    const ErrorScope es;
    Dev<float> m((size_t)d * d), dy(sd), dq(sd);
    if (es.failed()) return 3;
    m.from_host(saved[1]);
    dy.from_host(dout[0]);
    hipLaunchKernelGGL(frozen_read_backward_kernel, dim3(blocks_for(sd)), dim3(kThr), 0, stream(), m.ptr, dy.ptr, dq.ptr, s, d);
    check_launch("frozen_read_backward_kernel");
    check_hip(hipStreamSynchronize(stream()), "opaque block: synchronize");
    if (es.failed()) return 3;
    add_into(d_inputs[0], dq.to_host(), (size_t)sd);
    return es.failed() ? 3 : 0;
}

}  // namespace
}  // namespace nlh

using namespace nlh;

extern "C" int nlh_opaque_backward(int key, const float *const *d_outputs, const long long *d_output_lens,
                                   int n_outputs, const float *const *saved, const long long *saved_lens, int n_saved,
                                   float *const *d_inputs, const long long *d_input_lens, int n_inputs) {
    if (!d_outputs || !d_output_lens || !saved || !saved_lens || !d_inputs || !d_input_lens || n_outputs < 1 ||
        n_saved < 1 || n_inputs < 1) {
        fail("nlh_opaque_backward: null argument or empty buffer list");
        return 1;
    }
    const Slices dout{d_outputs, d_output_lens, n_outputs}, sv{saved, saved_lens, n_saved};
    switch (key) {
        case NLH_OPAQUE_DELTA_RULE: return rule_block_backward(false, dout, sv, d_inputs, d_input_lens, n_inputs);
        case NLH_OPAQUE_TITANS_LMM: return rule_block_backward(true, dout, sv, d_inputs, d_input_lens, n_inputs);
        case NLH_OPAQUE_DGD: return dgd_block_backward(dout, sv, d_inputs, d_input_lens, n_inputs);
        case NLH_OPAQUE_SWA: return swa_block_backward(dout, sv, d_inputs, d_input_lens, n_inputs);
        case NLH_OPAQUE_FROZEN_DELTA_RULE:
        case NLH_OPAQUE_FROZEN_TITANS_LMM: return frozen_block_backward(dout, sv, d_inputs, d_input_lens, n_inputs);
        default:
            fail("nlh_opaque_backward: OpaqueKey %d has no GPU adapter (built: DeltaRule 0, TitansLMM 1, DGD 9, SWA 10, "
                 "FrozenDeltaRule 11, FrozenTitansLMM 12)", key);
            return 1;
    }
}
