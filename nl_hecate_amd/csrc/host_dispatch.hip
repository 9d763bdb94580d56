// Host-slice dispatch: the entry points a CPU caller (the rule structs and the
// opaque VJP blocks of the Wengert tape) reaches through `*_dispatch`
// (core/src/dispatch.rs:378-460 SWA, 746-895 Delta / Titans, 1083-1224 Hebbian /
// DGD).  Arguments are host pointers in the order of those functions; each call
// stages one chain on the device the way the reference's helpers do
// (core/src/dispatch.rs:637-744, 1665-2085: allocate, copy in, zero the outputs,
// launch with batch_size = 1, synchronise, copy out) and frees its buffers.
// Nothing here computes on the host except the bf16 conversion of the SWA
// operands (core/src/dispatch.rs:463-490).
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string.h>

#include <vector>

#include "../../include/nl_hecate_ffi.h"
#include "runtime.h"

namespace nlh {
namespace {

// One device array of n elements of T, released when the call returns.
template <typename T>
struct Staged {
    T *ptr = nullptr;
    size_t n;
    explicit Staged(size_t count) : n(count) {
        check_hip(hipMalloc(reinterpret_cast<void **>(&ptr), (n ? n : 1) * sizeof(T)), "host dispatch: hipMalloc");
    }
    ~Staged() { if (ptr) (void)hipFree(ptr); }
    Staged(const Staged &) = delete;
    Staged &operator=(const Staged &) = delete;
    void from_host(const T *src) {
        if (ptr && n) check_hip(hipMemcpyAsync(ptr, src, n * sizeof(T), hipMemcpyHostToDevice, stream()), "host dispatch: copy in");
    }
    void zero() {
        if (ptr && n) check_hip(hipMemsetAsync(ptr, 0, n * sizeof(T), stream()), "host dispatch: zero");
    }
    void to_host(T *dst) {
        if (ptr && n) check_hip(hipMemcpyAsync(dst, ptr, n * sizeof(T), hipMemcpyDeviceToHost, stream()), "host dispatch: copy out");
    }
};

void finish(const char *what) { check_hip(hipStreamSynchronize(stream()), what); }

bool positive(const char *fn, int seq_len, int d) {
    if (seq_len <= 0 || d <= 0) { fail("%s: seq_len and d must be positive", fn); return false; }
    return true;
}

// core/src/dispatch.rs:463-475: round to nearest even on the upper 16 bits.
uint16_t f32_to_bf16_bits(float x) {
    uint32_t bits;
    memcpy(&bits, &x, 4);
    const uint32_t round = ((bits >> 16) & 1u) + 0x7FFFu;
    return (uint16_t)((bits + round) >> 16);
}
float bf16_bits_to_f32(uint16_t h) {
    const uint32_t bits = (uint32_t)h << 16;
    float x;
    memcpy(&x, &bits, 4);
    return x;
}

struct StagedBf16 {
    Staged<uint16_t> dev;
    std::vector<uint16_t> host;
    explicit StagedBf16(size_t n) : dev(n), host(n) {}
    void from_host_f32(const float *src) {
        for (size_t i = 0; i < host.size(); i++) host[i] = f32_to_bf16_bits(src[i]);
        dev.from_host(host.data());
        // the staging vector is reused by to_host_f32 only after the stream has drained
    }
    void to_host_f32(float *dst) {
        dev.to_host(host.data());
        finish("host dispatch: bf16 copy out");
        for (size_t i = 0; i < host.size(); i++) dst[i] = bf16_bits_to_f32(host[i]);
    }
};

bool swa_head_dim_ok(const char *fn, int head_dim) {
    if (head_dim <= 0 || head_dim > 1024 || (head_dim & (head_dim - 1))) {
        fail("%s: head_dim must be a power of two of at most 1024, got %d", fn, head_dim);
        return false;
    }
    return true;
}

}  // namespace
}  // namespace nlh

using namespace nlh;

// ── Delta rule ───────────────────────────────────────────────────────────────
extern "C" void nlh_delta_forward_dispatch(const float *k_mem, const float *v_mem, const float *q_mem,
                                           const float *alpha, const float *theta, const float *m_initial,
                                           float *m_states, float *y, int seq_len, int d, float error_clip,
                                           float m_norm_max) {
    const ErrorScope es;
    if (!positive("nlh_delta_forward_dispatch", seq_len, d)) return;
    const size_t sd = (size_t)seq_len * d, dd = (size_t)d * d;
    Staged<float> km(sd), vm(sd), qm(sd), al(seq_len), th(seq_len), m0(dd), ms((seq_len + 1) * dd), yy(sd);
    if (es.failed()) return;
    km.from_host(k_mem); vm.from_host(v_mem); qm.from_host(q_mem);
    al.from_host(alpha); th.from_host(theta); m0.from_host(m_initial);
    ms.zero(); yy.zero();
    delta_forward_f32_cuda(km.ptr, vm.ptr, qm.ptr, al.ptr, th.ptr, m0.ptr, ms.ptr, yy.ptr, seq_len, d, 1, seq_len,
                           (int)dd, error_clip, m_norm_max);
    ms.to_host(m_states); yy.to_host(y);
    finish("nlh_delta_forward_dispatch");
}

extern "C" void nlh_delta_backward_dispatch(const float *k_mem, const float *v_mem, const float *q_mem,
                                            const float *alpha, const float *theta, const float *m_states,
                                            const float *d_y, float *d_k_mem, float *d_v_mem, float *d_q_mem,
                                            float *d_alpha, float *d_theta, float *d_m_initial, int seq_len, int d,
                                            float error_clip) {
    const ErrorScope es;
    if (!positive("nlh_delta_backward_dispatch", seq_len, d)) return;
    const size_t sd = (size_t)seq_len * d, dd = (size_t)d * d;
    Staged<float> km(sd), vm(sd), qm(sd), al(seq_len), th(seq_len), ms((seq_len + 1) * dd), dy(sd);
    Staged<float> dk(sd), dv(sd), dq(sd), da(seq_len), dt(seq_len), dm(dd);
    if (es.failed()) return;
    km.from_host(k_mem); vm.from_host(v_mem); qm.from_host(q_mem);
    al.from_host(alpha); th.from_host(theta); ms.from_host(m_states); dy.from_host(d_y);
    dk.zero(); dv.zero(); dq.zero(); da.zero(); dt.zero(); dm.zero();
    delta_backward_f32_cuda(km.ptr, vm.ptr, qm.ptr, al.ptr, th.ptr, ms.ptr, dy.ptr, dk.ptr, dv.ptr, dq.ptr, da.ptr,
                            dt.ptr, dm.ptr, seq_len, d, 1, error_clip);
    dk.to_host(d_k_mem); dv.to_host(d_v_mem); dq.to_host(d_q_mem);
    da.to_host(d_alpha); dt.to_host(d_theta); dm.to_host(d_m_initial);
    finish("nlh_delta_backward_dispatch");
}

// ── Titans LMM ───────────────────────────────────────────────────────────────
extern "C" void nlh_titans_forward_dispatch(const float *k_mem, const float *v_mem, const float *q_mem,
                                            const float *alpha, const float *theta, const float *eta,
                                            const float *m_initial, const float *s_initial, float *m_states,
                                            float *s_states, float *y, int seq_len, int d, float error_clip,
                                            float m_norm_max) {
    const ErrorScope es;
    if (!positive("nlh_titans_forward_dispatch", seq_len, d)) return;
    const size_t sd = (size_t)seq_len * d, dd = (size_t)d * d;
    Staged<float> km(sd), vm(sd), qm(sd), al(seq_len), th(seq_len), et(seq_len), m0(dd), s0(dd);
    Staged<float> ms((seq_len + 1) * dd), ss((seq_len + 1) * dd), yy(sd);
    if (es.failed()) return;
    km.from_host(k_mem); vm.from_host(v_mem); qm.from_host(q_mem);
    al.from_host(alpha); th.from_host(theta); et.from_host(eta);
    m0.from_host(m_initial); s0.from_host(s_initial);
    ms.zero(); ss.zero(); yy.zero();
    titans_forward_f32_cuda(km.ptr, vm.ptr, qm.ptr, al.ptr, th.ptr, et.ptr, m0.ptr, s0.ptr, ms.ptr, ss.ptr, yy.ptr,
                            seq_len, d, 1, seq_len, (int)dd, error_clip, m_norm_max);
    ms.to_host(m_states); ss.to_host(s_states); yy.to_host(y);
    finish("nlh_titans_forward_dispatch");
}

extern "C" void nlh_titans_backward_dispatch(const float *k_mem, const float *v_mem, const float *q_mem,
                                             const float *alpha, const float *theta, const float *eta,
                                             const float *m_states, const float *s_states, const float *d_y,
                                             float *d_k_mem, float *d_v_mem, float *d_q_mem, float *d_alpha,
                                             float *d_theta, float *d_eta, float *d_m_initial, float *d_s_initial,
                                             int seq_len, int d, float error_clip) {
    const ErrorScope es;
    if (!positive("nlh_titans_backward_dispatch", seq_len, d)) return;
    const size_t sd = (size_t)seq_len * d, dd = (size_t)d * d;
    Staged<float> km(sd), vm(sd), qm(sd), al(seq_len), th(seq_len), et(seq_len);
    Staged<float> ms((seq_len + 1) * dd), ss((seq_len + 1) * dd), dy(sd);
    Staged<float> dk(sd), dv(sd), dq(sd), da(seq_len), dt(seq_len), de(seq_len), dm(dd), ds(dd);
    if (es.failed()) return;
    km.from_host(k_mem); vm.from_host(v_mem); qm.from_host(q_mem);
    al.from_host(alpha); th.from_host(theta); et.from_host(eta);
    ms.from_host(m_states); ss.from_host(s_states); dy.from_host(d_y);
    dk.zero(); dv.zero(); dq.zero(); da.zero(); dt.zero(); de.zero(); dm.zero(); ds.zero();
    titans_backward_f32_cuda(km.ptr, vm.ptr, qm.ptr, al.ptr, th.ptr, et.ptr, ms.ptr, ss.ptr, dy.ptr, dk.ptr, dv.ptr,
                             dq.ptr, da.ptr, dt.ptr, de.ptr, dm.ptr, ds.ptr, seq_len, d, 1, error_clip);
    dk.to_host(d_k_mem); dv.to_host(d_v_mem); dq.to_host(d_q_mem);
    da.to_host(d_alpha); dt.to_host(d_theta); de.to_host(d_eta);
    dm.to_host(d_m_initial); ds.to_host(d_s_initial);
    finish("nlh_titans_backward_dispatch");
}

// ── Hebbian rule ─────────────────────────────────────────────────────────────
// The reference runs the clamped case (0 < m_norm_max < f32::MAX) on the CPU
// (core/src/dispatch.rs:1096-1105): the device kernel has no clamp, and this
// library has no CPU path, so that case is refused.
extern "C" void nlh_hebbian_forward_dispatch(const float *k_mem, const float *v_mem, const float *q_mem,
                                             const float *alpha, const float *m_initial, float *m_states, float *y,
                                             int seq_len, int d, float m_norm_max) {
    const ErrorScope es;
    if (!positive("nlh_hebbian_forward_dispatch", seq_len, d)) return;
    if (m_norm_max > 0.f && m_norm_max < 3.4028234e38f) {
        fail("nlh_hebbian_forward_dispatch: the Hebbian kernel has no norm clamp (m_norm_max=%g)", (double)m_norm_max);
        return;
    }
    const size_t sd = (size_t)seq_len * d, dd = (size_t)d * d;
    Staged<float> km(sd), vm(sd), qm(sd), al(seq_len), m0(dd), ms((seq_len + 1) * dd), yy(sd);
    if (es.failed()) return;
    km.from_host(k_mem); vm.from_host(v_mem); qm.from_host(q_mem); al.from_host(alpha); m0.from_host(m_initial);
    ms.zero(); yy.zero();
    hebbian_forward_f32_cuda(km.ptr, vm.ptr, qm.ptr, al.ptr, m0.ptr, ms.ptr, yy.ptr, seq_len, d, 1, seq_len, (int)dd);
    ms.to_host(m_states); yy.to_host(y);
    finish("nlh_hebbian_forward_dispatch");
}

extern "C" void nlh_hebbian_backward_dispatch(const float *k_mem, const float *v_mem, const float *q_mem,
                                              const float *alpha, const float *m_states, const float *d_y,
                                              float *d_k_mem, float *d_v_mem, float *d_q_mem, float *d_alpha,
                                              float *d_m_initial, int seq_len, int d) {
    const ErrorScope es;
    if (!positive("nlh_hebbian_backward_dispatch", seq_len, d)) return;
    const size_t sd = (size_t)seq_len * d, dd = (size_t)d * d;
    Staged<float> km(sd), vm(sd), qm(sd), al(seq_len), ms((seq_len + 1) * dd), dy(sd);
    Staged<float> dk(sd), dv(sd), dq(sd), da(seq_len), dm(dd);
    if (es.failed()) return;
    km.from_host(k_mem); vm.from_host(v_mem); qm.from_host(q_mem); al.from_host(alpha);
    ms.from_host(m_states); dy.from_host(d_y);
    dk.zero(); dv.zero(); dq.zero(); da.zero(); dm.zero();
    hebbian_backward_f32_cuda(km.ptr, vm.ptr, qm.ptr, al.ptr, ms.ptr, dy.ptr, dk.ptr, dv.ptr, dq.ptr, da.ptr, dm.ptr,
                              seq_len, d);
    dk.to_host(d_k_mem); dv.to_host(d_v_mem); dq.to_host(d_q_mem); da.to_host(d_alpha); dm.to_host(d_m_initial);
    finish("nlh_hebbian_backward_dispatch");
}

// ── DGD ──────────────────────────────────────────────────────────────────────
extern "C" void nlh_dgd_forward_dispatch(const float *k_mem, const float *v_mem, const float *q_mem,
                                         const float *alpha, const float *theta, const float *m_initial,
                                         float *m_states, float *y, int seq_len, int d, float error_clip) {
    const ErrorScope es;
    if (!positive("nlh_dgd_forward_dispatch", seq_len, d)) return;
    const size_t sd = (size_t)seq_len * d, dd = (size_t)d * d;
    Staged<float> km(sd), vm(sd), qm(sd), al(seq_len), th(seq_len), m0(dd), ms((seq_len + 1) * dd), yy(sd);
    if (es.failed()) return;
    km.from_host(k_mem); vm.from_host(v_mem); qm.from_host(q_mem);
    al.from_host(alpha); th.from_host(theta); m0.from_host(m_initial);
    ms.zero(); yy.zero();
    dgd_forward_f32_cuda(km.ptr, vm.ptr, qm.ptr, al.ptr, th.ptr, m0.ptr, ms.ptr, yy.ptr, seq_len, d, 1, seq_len,
                         (int)dd, error_clip);
    ms.to_host(m_states); yy.to_host(y);
    finish("nlh_dgd_forward_dispatch");
}

extern "C" void nlh_dgd_backward_dispatch(const float *k_mem, const float *v_mem, const float *q_mem,
                                          const float *alpha, const float *theta, const float *m_states,
                                          const float *d_y, float *d_k_mem, float *d_v_mem, float *d_q_mem,
                                          float *d_alpha, float *d_theta, float *d_m_initial, int seq_len, int d,
                                          float error_clip) {
    const ErrorScope es;
    if (!positive("nlh_dgd_backward_dispatch", seq_len, d)) return;
    const size_t sd = (size_t)seq_len * d, dd = (size_t)d * d;
    Staged<float> km(sd), vm(sd), qm(sd), al(seq_len), th(seq_len), ms((seq_len + 1) * dd), dy(sd);
    Staged<float> dk(sd), dv(sd), dq(sd), da(seq_len), dt(seq_len), dm(dd);
    if (es.failed()) return;
    km.from_host(k_mem); vm.from_host(v_mem); qm.from_host(q_mem);
    al.from_host(alpha); th.from_host(theta); ms.from_host(m_states); dy.from_host(d_y);
    dk.zero(); dv.zero(); dq.zero(); da.zero(); dt.zero(); dm.zero();
    dgd_backward_f32_cuda(km.ptr, vm.ptr, qm.ptr, al.ptr, th.ptr, ms.ptr, dy.ptr, dk.ptr, dv.ptr, dq.ptr, da.ptr,
                          dt.ptr, dm.ptr, seq_len, d, error_clip);
    dk.to_host(d_k_mem); dv.to_host(d_v_mem); dq.to_host(d_q_mem);
    da.to_host(d_alpha); dt.to_host(d_theta); dm.to_host(d_m_initial);
    finish("nlh_dgd_backward_dispatch");
}

// ── Sliding-window attention ─────────────────────────────────────────────────
// q, k, v, out and the attention weights travel as float on the host and as bf16
// on the device (n_persistent = 0, one sequence), as in the reference's helper.
extern "C" void nlh_swa_forward_dispatch(const float *q, const float *k, const float *v, float *out,
                                         float *attn_weights, int seq_len, int num_heads, int head_dim,
                                         int window_size) {
    const ErrorScope es;
    if (!positive("nlh_swa_forward_dispatch", seq_len, head_dim) || !swa_head_dim_ok("nlh_swa_forward_dispatch", head_dim))
        return;
    const size_t total = (size_t)seq_len * num_heads * head_dim, aw_total = (size_t)num_heads * seq_len * window_size;
    StagedBf16 dq(total), dk(total), dv(total), dout(total), daw(aw_total);
    if (es.failed()) return;
    dq.from_host_f32(q); dk.from_host_f32(k); dv.from_host_f32(v);
    dout.dev.zero(); daw.dev.zero();
    swa_forward_f32_cuda(dq.dev.ptr, dk.dev.ptr, dv.dev.ptr, dout.dev.ptr, daw.dev.ptr, seq_len, num_heads, head_dim,
                         window_size, 1, 0);
    dout.to_host_f32(out);
    daw.to_host_f32(attn_weights);
}

// The caller zeroes d_q, d_k, d_v (core/src/dispatch.rs:407): d_k, d_v are accumulated into, d_q is overwritten.
extern "C" void nlh_swa_backward_dispatch(const float *q, const float *k, const float *v, const float *attn_weights,
                                          const float *d_attn_out, float *d_q, float *d_k, float *d_v, int seq_len,
                                          int num_heads, int head_dim, int window_size) {
    const ErrorScope es;
    if (!positive("nlh_swa_backward_dispatch", seq_len, head_dim) || !swa_head_dim_ok("nlh_swa_backward_dispatch", head_dim))
        return;
    const size_t total = (size_t)seq_len * num_heads * head_dim, aw_total = (size_t)num_heads * seq_len * window_size;
    StagedBf16 bq(total), bk(total), bv(total), baw(aw_total);
    Staged<float> dao(total), gq(total), gk(total), gv(total);
    if (es.failed()) return;
    bq.from_host_f32(q); bk.from_host_f32(k); bv.from_host_f32(v); baw.from_host_f32(attn_weights);
    dao.from_host(d_attn_out); gq.from_host(d_q); gk.from_host(d_k); gv.from_host(d_v);
    swa_backward_f32_cuda(bq.dev.ptr, bk.dev.ptr, bv.dev.ptr, baw.dev.ptr, dao.ptr, gq.ptr, gk.ptr, gv.ptr, seq_len,
                          num_heads, head_dim, window_size, 1, 0);
    gq.to_host(d_q); gk.to_host(d_k); gv.to_host(d_v);
    finish("nlh_swa_backward_dispatch");
}
