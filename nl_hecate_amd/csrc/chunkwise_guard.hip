// Guard of the matrix-form chunkwise kernels under the reference's production arguments.
//
// The reference applies two per-token couplings inside its chunkwise kernels: the error clip
// (core/kernels/error_clip.cuh: e <- e * clip / |e| when |e| > clip) and the Frobenius projection of the memory
// (core/kernels/m_norm_project.cuh, titans_chunkwise_forward.cu:158: M <- M * max / |M|_F when |M|_F > max).  Both
// break the linearity that the matrix form rests on, but only when they fire.  This file decides, on the device
// and from quantities the matrix form has already produced, whether they can fire at all:
//   * the frozen-M0 errors e_t = M0 k_t - v_t of a chunk are known exactly from the chunk-start state, so the clip
//     is idle iff max_t |e_t| <= clip;
//   * inside a chunk |S_t| <= eta_t |S_{t-1}| + theta_t |e_t| |k_t| and |M_t| <= (1 - alpha_t) |M_{t-1}| + |S_t|
//     (triangle inequality through the update, every coefficient non-negative), started from the exact norms of
//     the chunk-start states; if this scalar recurrence stays below the bound, no projection fires in the chunk.
// A chunk for which either test fails raises one flag; the caller then runs the sequential kernels, which apply
// the couplings token by token.  When the flag stays down the matrix form's results are the reference's.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/nl_hecate_ffi.h"
#include "chunkwise_chain.h"
#include "chunkwise_guard.h"
#include "lane_ops.h"
#include "mm_tiles.h"
#include "runtime.h"

namespace nlh {
namespace {

using namespace mmt;

constexpr float kSlack = 1.0f + 1e-4f;   // covers the rounding of the fp32 sums below

// four consecutive elements of a token row as floats
__device__ __forceinline__ float4 tok4(const float *p, size_t i) { return *reinterpret_cast<const float4 *>(p + i); }
__device__ __forceinline__ float4 tok4(const uint16_t *p, size_t i) {
    const uint2 u = *reinterpret_cast<const uint2 *>(p + i);
    return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u), __uint_as_float(u.y << 16),
                       __uint_as_float(u.y & 0xffff0000u));
}

__device__ __forceinline__ float lane_value(float x, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), lane));
}

// One workgroup (8 waves) per chunk; four workgroups share a compute unit, so one's loads overlap another's
// product (a persistent variant with the next chunk's tiles requested a chunk ahead needs twice the registers,
// halves the workgroups per compute unit and is slower).  E = K M0^T - V on the fp32 matrix cores, a 16 x 32
// strip per wave; the sums of squares of the states come from the registers the tiles were loaded into; wave 0
// then runs the scalar recurrence with lane t holding token t's numbers.
template <typename TOK, bool HAS_S>
__global__ __launch_bounds__(kThr) void cw_guard_kernel(const TOK *__restrict__ k, const TOK *__restrict__ v,
                                                        const float *__restrict__ alpha, const float *__restrict__ theta,
                                                        const float *__restrict__ eta, const float *__restrict__ m_states,
                                                        const float *__restrict__ s_states, int seq_len, int C, int nc,
                                                        float clip, float mmax, int *__restrict__ flag) {
    __shared__ float Ks[MAT], Ms[MAT];
    __shared__ float en2[2][CW], kn2[CW], red[2][8];
    const int tid = threadIdx.x, chunk = blockIdx.x % nc, chain = blockIdx.x / nc;
    const int t0 = chunk * C, L = min(C, seq_len - t0);
    const size_t st0 = ((size_t)chain * (nc + 1) + chunk) * HD * HD;
    const size_t tok = (size_t)chain * seq_len + t0;
    const int w = tid >> 6, m0 = 16 * (w >> 1), n0 = 32 * (w & 1), nh = w & 1;
    Tile<TOK> tk;
    Tile<float> tm, ts;
    fetch(tk, k + tok * HD, L);
    fetch(tm, m_states + st0, 64);
    if (HAS_S) fetch(ts, s_states + st0, 64);
    // -V at this wave's accumulator positions
    Strip e = zero_strip();
    for_c(e, [&](int r, int c, float &x) { x = m0 + r < L ? -to_f32(v[(tok + m0 + r) * HD + n0 + c]) : 0.f; });
    float al = 0.f, th = 0.f, et = 0.f;
    if (w == 0 && tid < L) {
        al = alpha[tok + tid];
        th = theta[tok + tid];
        if (HAS_S) et = eta[tok + tid];
    }
    commit(Ks, tk);
    commit(Ms, tm);
    {
        float msq = 0.f, ssq = 0.f;
#pragma unroll
        for (int it = 0; it < 2; it++) {
            msq += tm.x[it].x * tm.x[it].x + tm.x[it].y * tm.x[it].y + tm.x[it].z * tm.x[it].z + tm.x[it].w * tm.x[it].w;
            if (HAS_S) ssq += ts.x[it].x * ts.x[it].x + ts.x[it].y * ts.x[it].y + ts.x[it].z * ts.x[it].z + ts.x[it].w * ts.x[it].w;
        }
        msq = wave_allreduce(msq);
        ssq = wave_allreduce(ssq);
        if ((tid & 63) == 0) { red[0][w] = msq; red[1][w] = ssq; }
    }
    __syncthreads();
    if (w == 1) {   // |k_t|^2 of row (lane) (rows beyond L were staged as zeros)
        const int t = tid & 63;
        float x = 0.f;
#pragma unroll 16
        for (int c = 0; c < HD; c++) x = fmaf(Ks[t * LDM + c], Ks[t * LDM + c], x);
        kn2[t] = x;
    }
    mma(e, [&](int m, int kk) { return Ks[(m0 + m) * LDM + kk]; }, [&](int kk, int n) { return Ms[(n0 + n) * LDM + kk]; });
    for_c(e, [&](int, int, float &x) { x *= x; });
    strip_row_sums(e);
    if (row_writer()) {
#pragma unroll
        for (int i = 0; i < 4; i++) en2[nh][m0 + row_of(i)] = e.t[0][i];
    }
    __syncthreads();
    if (w == 0) {
        const float en = sqrtf(en2[0][tid] + en2[1][tid]) * kSlack, kn = sqrtf(kn2[tid]) * kSlack;
        const float drive = th * en * kn, keep = 1.0f - al;
        float nM = 0.f, nS = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) { nM += red[0][i]; nS += red[1][i]; }
        nM = sqrtf(nM) * kSlack;
        nS = HAS_S ? sqrtf(nS) * kSlack : 0.f;
        const bool clip_on = clip > 0.f, proj_on = mmax > 0.f && mmax < 1e30f;
        bool bad = clip_on && tid < L && en > clip;
        float worst = 0.f;
#pragma unroll 8
        for (int t = 0; t < CW; t++) {   // tokens beyond L carry keep = 1, eta = 0, no drive: they only repeat nM
            nS = (HAS_S ? lane_value(et, t) * nS : 0.f) + lane_value(drive, t);
            nM = lane_value(keep, t) * nM + nS;
            worst = t < L ? fmaxf(worst, nM) : worst;
        }
        if (proj_on && worst * kSlack > mmax) bad = true;
        if (bad) *flag = 1;
    }
}

// The same test from what the bf16 forward chain kernel leaves behind (ChainTracks): per token the squared error
// norm of each half of the memory rows, per chunk eight partial sums of squares of the chunk-start states.  One wave
// per chunk, lane = token; reads k once for |k_t|.  The errors there were formed against a hi + lo bf16 copy of M0
// (16 mantissa bits): |e_t| is raised by 2^-15 |M0|_F |k_t| to cover it.
template <typename TOK, bool HAS_S>
__global__ __launch_bounds__(256) void cw_guard_tracks_kernel(const TOK *__restrict__ k, const float *__restrict__ alpha,
                                                              const float *__restrict__ theta, const float *__restrict__ eta,
                                                              const float *__restrict__ e2, const float *__restrict__ nrm,
                                                              int seq_len, int C, int nc, int nchunks, float clip, float mmax,
                                                              float split_slack, int *__restrict__ flag) {
    const int lane = threadIdx.x & 63, task = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (task >= nchunks) return;   // waves are independent: no barrier below
    const int chain = task / nc, c = task % nc, t0 = c * C, L = min(C, seq_len - t0);
    const bool in = lane < L;
    const size_t tok = (size_t)chain * seq_len + t0 + lane;
    float ksq = 0.f, esq = 0.f, al = 0.f, th = 0.f, et = 0.f;
    if (in) {
#pragma unroll
        for (int i = 0; i < HD / 4; i++) {
            const float4 x = tok4(k, tok * HD + 4 * i);
            ksq += x.x * x.x + x.y * x.y + x.z * x.z + x.w * x.w;
        }
        esq = e2[(((size_t)chain * 2 + 0) * nc + c) * CW + lane] + e2[(((size_t)chain * 2 + 1) * nc + c) * CW + lane];
        al = alpha[tok];
        th = theta[tok];
        if (HAS_S) et = eta[tok];
    }
    float2 part = make_float2(0.f, 0.f);
    if (lane < 8) part = reinterpret_cast<const float2 *>(nrm)[((size_t)chain * nc + c) * 8 + lane];
    float nM = sqrtf(wave_allreduce(part.x)) * kSlack;
    float nS = HAS_S ? sqrtf(wave_allreduce(part.y)) * kSlack : 0.f;
    const float kn = sqrtf(ksq) * kSlack;
    const float en = sqrtf(esq) * kSlack + split_slack * nM * kn;
    const float drive = th * en * kn, keep = 1.0f - al;
    const bool clip_on = clip > 0.f, proj_on = mmax > 0.f && mmax < 1e30f;
    bool bad = clip_on && in && en > clip;
    float worst = 0.f;
#pragma unroll 8
    for (int t = 0; t < CW; t++) {   // tokens beyond L carry keep = 1, eta = 0, no drive
        nS = (HAS_S ? lane_value(et, t) * nS : 0.f) + lane_value(drive, t);
        nM = lane_value(keep, t) * nM + nS;
        worst = t < L ? fmaxf(worst, nM) : worst;
    }
    if (proj_on && worst * kSlack > mmax) bad = true;
    if (bad) *flag = 1;
}

__global__ void guard_clear_kernel(int *flag) { *flag = 0; }

int *g_host_flag = nullptr;

}  // namespace

bool force_sequential = false;
bool last_test_fired = false;

bool guard_possible() {
    if (force_sequential) return false;
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    return !(hipStreamIsCapturing(stream(), &cap) == hipSuccess && cap != hipStreamCaptureStatusNone);
}

template <typename TOK>
static bool couplings_may_fire_t(const TOK *k, const TOK *v, const float *alpha, const float *theta, const float *eta,
                                 const float *m_states, const float *s_states, int seq_len, int batch, int chunk_size,
                                 float error_clip, float m_norm_max) {
    const ErrorScope es;
    int *flag = reinterpret_cast<int *>(scratch(31, 256));
    if (!g_host_flag) check_hip(hipHostMalloc(reinterpret_cast<void **>(&g_host_flag), 256, hipHostMallocDefault), "hipHostMalloc");
    if (es.failed() || !g_host_flag) return true;
    const int nc = (seq_len + chunk_size - 1) / chunk_size;
    {
        KernelTimer kt("cw_guard_kernel");
        hipLaunchKernelGGL(guard_clear_kernel, dim3(1), dim3(1), 0, stream(), flag);
        const dim3 grid((unsigned)batch * nc);
        if (s_states)
            hipLaunchKernelGGL((cw_guard_kernel<TOK, true>), grid, dim3(kThr), 0, stream(), k, v, alpha, theta, eta, m_states,
                               s_states, seq_len, chunk_size, nc, error_clip, m_norm_max, flag);
        else
            hipLaunchKernelGGL((cw_guard_kernel<TOK, false>), grid, dim3(kThr), 0, stream(), k, v, alpha, theta, eta, m_states,
                               s_states, seq_len, chunk_size, nc, error_clip, m_norm_max, flag);
        check_launch("cw_guard_kernel");
    }
    *g_host_flag = 1;
    check_hip(hipMemcpyAsync(g_host_flag, flag, sizeof(int), hipMemcpyDeviceToHost, stream()), "guard flag copy");
    check_hip(hipStreamSynchronize(stream()), "guard flag sync");
    last_test_fired = es.failed() || *g_host_flag != 0;
    return last_test_fired;
}

namespace {
__global__ void norm_bound_kernel(const float *__restrict__ msq_part, int batch, int parts, float limit_sq, int *flag) {
    const int b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= batch) return;
    float tot = 0.f;
    for (int p = 0; p < parts; p++) tot += msq_part[b * parts + p];
    if (!(tot * (1.0f + 1e-3f) <= limit_sq)) *flag = 1;   // also raised by a NaN
}
}  // namespace

bool norm_bound_exceeded(const float *msq_part, int batch, int parts, float m_norm_max) {
    const ErrorScope es;
    int *flag = reinterpret_cast<int *>(scratch(31, 256));
    if (!g_host_flag) check_hip(hipHostMalloc(reinterpret_cast<void **>(&g_host_flag), 256, hipHostMallocDefault), "hipHostMalloc");
    if (es.failed() || !g_host_flag) return true;
    {
        KernelTimer kt("norm_bound_kernel");
        hipLaunchKernelGGL(guard_clear_kernel, dim3(1), dim3(1), 0, stream(), flag);
        hipLaunchKernelGGL(norm_bound_kernel, dim3((batch + 255) / 256), dim3(256), 0, stream(), msq_part, batch, parts,
                           m_norm_max * m_norm_max, flag);
        check_launch("norm_bound_kernel");
    }
    *g_host_flag = 1;
    check_hip(hipMemcpyAsync(g_host_flag, flag, sizeof(int), hipMemcpyDeviceToHost, stream()), "guard flag copy");
    check_hip(hipStreamSynchronize(stream()), "guard flag sync");
    last_test_fired = es.failed() || *g_host_flag != 0;
    return last_test_fired;
}

template <typename TOK>
static bool tracked_test(const TOK *k, const float *alpha, const float *theta, const float *eta, const ChainTracks &tr,
                         bool has_s, int seq_len, int batch, int chunk_size, float error_clip, float m_norm_max,
                         float split_slack) {
    const ErrorScope es;
    int *flag = reinterpret_cast<int *>(scratch(31, 256));
    if (!g_host_flag) check_hip(hipHostMalloc(reinterpret_cast<void **>(&g_host_flag), 256, hipHostMallocDefault), "hipHostMalloc");
    if (es.failed() || !g_host_flag) return true;
    const int nc = (seq_len + chunk_size - 1) / chunk_size, nchunks = batch * nc;
    {
        KernelTimer kt("cw_guard_tracks_kernel");
        hipLaunchKernelGGL(guard_clear_kernel, dim3(1), dim3(1), 0, stream(), flag);
        const dim3 grid((unsigned)((nchunks + 3) / 4));
        if (has_s)
            hipLaunchKernelGGL((cw_guard_tracks_kernel<TOK, true>), grid, dim3(256), 0, stream(), k, alpha, theta, eta, tr.e2,
                               tr.nrm, seq_len, chunk_size, nc, nchunks, error_clip, m_norm_max, split_slack, flag);
        else
            hipLaunchKernelGGL((cw_guard_tracks_kernel<TOK, false>), grid, dim3(256), 0, stream(), k, alpha, theta, eta, tr.e2,
                               tr.nrm, seq_len, chunk_size, nc, nchunks, error_clip, m_norm_max, split_slack, flag);
        check_launch("cw_guard_tracks_kernel");
    }
    *g_host_flag = 1;
    check_hip(hipMemcpyAsync(g_host_flag, flag, sizeof(int), hipMemcpyDeviceToHost, stream()), "guard flag copy");
    check_hip(hipStreamSynchronize(stream()), "guard flag sync");
    last_test_fired = es.failed() || *g_host_flag != 0;
    return last_test_fired;
}

ChainTracks chain_tracks(int seq_len, int batch, int chunk_size) {
    const int nc = (seq_len + chunk_size - 1) / chunk_size;
    const size_t e2_floats = (size_t)batch * 2 * nc * 64, nrm_floats = (size_t)batch * nc * 16;
    float *buf = scratch(12, (e2_floats + nrm_floats) * sizeof(float));
    return ChainTracks{buf, buf ? buf + e2_floats : nullptr};
}

// bf16 tokens: the errors were formed against a hi + lo bf16 copy of M0, hence the 2^-15 |M0|_F |k_t| on top
bool couplings_may_fire_tracked(const uint16_t *k, const float *alpha, const float *theta, const float *eta,
                                const ChainTracks &tr, bool has_s, int seq_len, int batch, int chunk_size, float error_clip,
                                float m_norm_max) {
    return tracked_test(k, alpha, theta, eta, tr, has_s, seq_len, batch, chunk_size, error_clip, m_norm_max, 3.0517578125e-5f);
}
bool couplings_may_fire_tracked(const float *k, const float *alpha, const float *theta, const float *eta,
                                const ChainTracks &tr, bool has_s, int seq_len, int batch, int chunk_size, float error_clip,
                                float m_norm_max) {
    return tracked_test(k, alpha, theta, eta, tr, has_s, seq_len, batch, chunk_size, error_clip, m_norm_max, 0.f);
}

bool couplings_may_fire(const float *k, const float *v, const float *alpha, const float *theta, const float *eta,
                        const float *m_states, const float *s_states, int seq_len, int batch, int chunk_size,
                        float error_clip, float m_norm_max) {
    return couplings_may_fire_t<float>(k, v, alpha, theta, eta, m_states, s_states, seq_len, batch, chunk_size, error_clip,
                                       m_norm_max);
}
bool couplings_may_fire_bf16(const uint16_t *k, const uint16_t *v, const float *alpha, const float *theta, const float *eta,
                             const float *m_states, const float *s_states, int seq_len, int batch, int chunk_size,
                             float error_clip, float m_norm_max) {
    return couplings_may_fire_t<uint16_t>(k, v, alpha, theta, eta, m_states, s_states, seq_len, batch, chunk_size, error_clip,
                                          m_norm_max);
}

}  // namespace nlh

using namespace nlh;

namespace {
bool coupled(float error_clip, float m_norm_max) { return error_clip > 0.f || (m_norm_max > 0.f && m_norm_max < 1e30f); }
struct ForceSequential {
    ForceSequential() { force_sequential = true; }
    ~ForceSequential() { force_sequential = false; }
};
// bf16 tokens as fp32 in scratch, for the sequential kernels
const float *widen(int slot, const uint16_t *x, size_t count) {
    float *out = scratch(slot, count * sizeof(float));
    if (out) bf16_to_f32_cuda(x, out, (int)count);
    return out;
}
}  // namespace

extern "C" {

void titans_chunkwise_forward_bf16_guarded_rocm(const uint16_t *k_mem, const uint16_t *v_mem, const uint16_t *q_mem,
                                                const float *alpha, const float *theta, const float *eta,
                                                const float *m_initial, const float *s_initial, float *m_chunk_states,
                                                float *s_chunk_states, float *y, int seq_len, int d, int batch_size,
                                                int chunk_size, float error_clip, float m_norm_max) {
    const ErrorScope es;
    if (seq_len <= 0 || batch_size <= 0) return;
    const bool mm = d == 64 && chunk_size >= 1 && chunk_size <= 64;
    if (mm && coupled(error_clip, m_norm_max) && guard_possible()) {
        // the chain kernel leaves the error and state norms behind as it goes: the test is then a scalar recurrence
        const ChainTracks tr = chain_tracks(seq_len, batch_size, chunk_size);
        if (es.failed()) return;
        if (chunkwise_chain_forward_bf16("titans_chunkwise_forward_bf16_guarded_rocm", k_mem, v_mem, q_mem, alpha, theta, eta,
                                         m_initial, s_initial, m_chunk_states, s_chunk_states, y, seq_len, d, batch_size,
                                         chunk_size, true, nullptr, &tr)) {
            if (es.failed()) return;
            if (!couplings_may_fire_tracked(k_mem, alpha, theta, eta, tr, true, seq_len, batch_size, chunk_size, error_clip,
                                            m_norm_max))
                return;
        }
    } else if (mm && (!coupled(error_clip, m_norm_max) || guard_possible())) {
        titans_chunkwise_forward_bf16_rocm(k_mem, v_mem, q_mem, alpha, theta, eta, m_initial, s_initial, m_chunk_states,
                                           s_chunk_states, y, seq_len, d, batch_size, chunk_size);
        if (es.failed()) return;
        if (!coupled(error_clip, m_norm_max) ||
            !couplings_may_fire_bf16(k_mem, v_mem, alpha, theta, eta, m_chunk_states, s_chunk_states, seq_len, batch_size,
                                     chunk_size, error_clip, m_norm_max))
            return;
    }
    const size_t cnt = (size_t)batch_size * seq_len * d;
    if (cnt > 0x7fffffffULL) { fail("titans_chunkwise_forward_bf16_guarded_rocm: batch * seq_len * d exceeds 2^31."); return; }
    const float *kf = widen(20, k_mem, cnt), *vf = widen(21, v_mem, cnt), *qf = widen(22, q_mem, cnt);
    if (es.failed()) return;
    const ForceSequential fs;
    titans_chunkwise_forward_f32_cuda(kf, vf, qf, alpha, theta, eta, m_initial, s_initial, m_chunk_states, s_chunk_states, y,
                                      seq_len, d, batch_size, chunk_size, error_clip, m_norm_max);
}

void titans_chunkwise_backward_bf16_guarded_rocm(const uint16_t *k_mem, const uint16_t *v_mem, const uint16_t *q_mem,
                                                 const float *alpha, const float *theta, const float *eta,
                                                 const float *m_chunk_states, const float *s_chunk_states, const float *d_y,
                                                 float *d_k_mem, float *d_v_mem, float *d_q_mem, float *d_alpha, float *d_theta,
                                                 float *d_eta, float *d_m_initial, float *d_s_initial, int seq_len, int d,
                                                 int batch_size, int chunk_size, float error_clip, float m_norm_max) {
    const ErrorScope es;
    if (seq_len <= 0 || batch_size <= 0) return;
    const bool mm = d == 64 && chunk_size >= 1 && chunk_size <= 64;
    if (mm && coupled(error_clip, m_norm_max) && guard_possible() && !last_test_fired) {
        // the test inside the matrix-form pass (its gradient kernel forms the errors anyway); see memory_rules.hip for
        // why the order of work follows the last test
        if (chunkwise_backward_bf16_guarded("titans_chunkwise_backward_bf16_guarded_rocm", k_mem, v_mem, q_mem, alpha, theta, eta,
                                            m_chunk_states, s_chunk_states, d_y, d_k_mem, d_v_mem, d_q_mem, d_alpha, d_theta,
                                            d_eta, d_m_initial, d_s_initial, seq_len, d, batch_size, chunk_size, true, error_clip,
                                            m_norm_max))
            return;
    } else if (mm && (!coupled(error_clip, m_norm_max) ||
               (guard_possible() && !couplings_may_fire_bf16(k_mem, v_mem, alpha, theta, eta, m_chunk_states, s_chunk_states,
                                                             seq_len, batch_size, chunk_size, error_clip, m_norm_max)))) {
        titans_chunkwise_backward_bf16_rocm(k_mem, v_mem, q_mem, alpha, theta, eta, m_chunk_states, s_chunk_states, d_y, d_k_mem,
                                            d_v_mem, d_q_mem, d_alpha, d_theta, d_eta, d_m_initial, d_s_initial, seq_len, d,
                                            batch_size, chunk_size);
        return;
    }
    if (es.failed()) return;
    const size_t cnt = (size_t)batch_size * seq_len * d;
    if (cnt > 0x7fffffffULL) { fail("titans_chunkwise_backward_bf16_guarded_rocm: batch * seq_len * d exceeds 2^31."); return; }
    const float *kf = widen(20, k_mem, cnt), *vf = widen(21, v_mem, cnt), *qf = widen(22, q_mem, cnt);
    if (es.failed()) return;
    const ForceSequential fs;
    titans_chunkwise_backward_f32_cuda(kf, vf, qf, alpha, theta, eta, m_chunk_states, s_chunk_states, d_y, d_k_mem, d_v_mem,
                                       d_q_mem, d_alpha, d_theta, d_eta, d_m_initial, d_s_initial, seq_len, d, batch_size,
                                       chunk_size, error_clip, m_norm_max);
}

}  // extern "C"
