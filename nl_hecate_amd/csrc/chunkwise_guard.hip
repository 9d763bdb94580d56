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
#include "chunkwise_guard.h"
#include "lane_ops.h"
#include "runtime.h"

namespace nlh {
namespace {

constexpr int GD = 64;        // head size of the matrix form
constexpr int GS = 68;        // LDS row stride (16-byte rows)
constexpr float kSlack = 1.0f + 1e-4f;   // covers the rounding of the fp32 sums below

__device__ __forceinline__ float tok1(const float *p, size_t i) { return p[i]; }
__device__ __forceinline__ float tok1(const uint16_t *p, size_t i) { return __uint_as_float(((unsigned)p[i]) << 16); }
// four consecutive tokens' elements as floats
__device__ __forceinline__ float4 tok4(const float *p, size_t i) { return *reinterpret_cast<const float4 *>(p + i); }
__device__ __forceinline__ float4 tok4(const uint16_t *p, size_t i) {
    const uint2 u = *reinterpret_cast<const uint2 *>(p + i);
    return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u), __uint_as_float(u.y << 16),
                       __uint_as_float(u.y & 0xffff0000u));
}

template <typename TOK, bool HAS_S>
__global__ __launch_bounds__(256) void cw_guard_kernel(const TOK *__restrict__ k, const TOK *__restrict__ v,
                                                       const float *__restrict__ alpha, const float *__restrict__ theta,
                                                       const float *__restrict__ eta, const float *__restrict__ m_states,
                                                       const float *__restrict__ s_states, int seq_len, int C, int nc,
                                                       float clip, float mmax, int *__restrict__ flag) {
    __shared__ __align__(16) float M0[GD * GS], Ks[GD * GS];
    __shared__ float en[GD], kn[GD], gate[3][GD], red[2][4];
    const int tid = threadIdx.x, chunk = blockIdx.x % nc, chain = blockIdx.x / nc;
    const int t0 = chunk * C, L = min(C, seq_len - t0);
    const float *m0 = m_states + ((size_t)chain * (nc + 1) + chunk) * GD * GD;
    const float *s0 = HAS_S ? s_states + ((size_t)chain * (nc + 1) + chunk) * GD * GD : nullptr;
    float msq = 0.f, ssq = 0.f;
    for (int e = tid; e < GD * GD / 4; e += 256) {
        const float4 x = reinterpret_cast<const float4 *>(m0)[e];
        *reinterpret_cast<float4 *>(M0 + (e / 16) * GS + (e % 16) * 4) = x;
        msq += x.x * x.x + x.y * x.y + x.z * x.z + x.w * x.w;
        if (HAS_S) {
            const float4 y = reinterpret_cast<const float4 *>(s0)[e];
            ssq += y.x * y.x + y.y * y.y + y.z * y.z + y.w * y.w;
        }
    }
    const size_t tok0 = ((size_t)chain * seq_len + t0) * GD;
    for (int e = tid; e < GD * GD / 4; e += 256) {
        const int t = e / 16, j = (e % 16) * 4;
        float4 kx = make_float4(0.f, 0.f, 0.f, 0.f);
        if (t < L) kx = tok4(k, tok0 + 4 * (size_t)e);
        *reinterpret_cast<float4 *>(Ks + t * GS + j) = kx;
    }
    if (tid < GD) {
        const size_t g = (size_t)chain * seq_len + t0 + tid;
        gate[0][tid] = tid < L ? alpha[g] : 0.f;
        gate[1][tid] = tid < L ? theta[g] : 0.f;
        gate[2][tid] = (HAS_S && tid < L) ? eta[g] : 0.f;
    }
    // -V: every thread its own 16 elements (consecutive lanes on consecutive columns), requested before the barrier
    float e[4][4];
    {
        const int ti = tid >> 4, ii = tid & 15;
#pragma unroll
        for (int a = 0; a < 4; a++)
#pragma unroll
            for (int b = 0; b < 4; b++)
                e[a][b] = 4 * ti + a < L ? -tok1(v, tok0 + (size_t)(4 * ti + a) * GD + ii + 16 * b) : 0.f;
    }
    msq = wave_allreduce(msq);
    ssq = wave_allreduce(ssq);
    if ((tid & 63) == 0) { red[0][tid >> 6] = msq; red[1][tid >> 6] = ssq; }
    __syncthreads();
    {   // E = K M0^T - V in 4 x 4 register blocks: thread (ti, ii) owns tokens 4 ti .. + 3 and rows ii, ii + 16, ii + 32,
        // ii + 48 of M0 (consecutive lanes on consecutive rows: conflict-free 16-byte reads at row stride 68)
        const int ti = tid >> 4, ii = tid & 15;
        float ksq[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
        for (int j4 = 0; j4 < GD / 4; j4++) {
            float4 kx[4], mx[4];
#pragma unroll
            for (int a = 0; a < 4; a++) kx[a] = *reinterpret_cast<const float4 *>(Ks + (4 * ti + a) * GS + 4 * j4);
#pragma unroll
            for (int b = 0; b < 4; b++) mx[b] = *reinterpret_cast<const float4 *>(M0 + (ii + 16 * b) * GS + 4 * j4);
#pragma unroll
            for (int a = 0; a < 4; a++) {
                if ((j4 & 15) == ii) ksq[a] += kx[a].x * kx[a].x + kx[a].y * kx[a].y + kx[a].z * kx[a].z + kx[a].w * kx[a].w;
#pragma unroll
                for (int b = 0; b < 4; b++)
                    e[a][b] += kx[a].x * mx[b].x + kx[a].y * mx[b].y + kx[a].z * mx[b].z + kx[a].w * mx[b].w;
            }
        }
#pragma unroll
        for (int a = 0; a < 4; a++) {
            float esq = e[a][0] * e[a][0] + e[a][1] * e[a][1] + e[a][2] * e[a][2] + e[a][3] * e[a][3];
            esq = group_allreduce<16>(esq);
            const float kq = group_allreduce<16>(ksq[a]);
            if (ii == 0) { en[4 * ti + a] = sqrtf(esq) * kSlack; kn[4 * ti + a] = sqrtf(kq) * kSlack; }
        }
    }
    __syncthreads();
    if (tid == 0) {
        float nM = sqrtf(red[0][0] + red[0][1] + red[0][2] + red[0][3]) * kSlack;
        float nS = HAS_S ? sqrtf(red[1][0] + red[1][1] + red[1][2] + red[1][3]) * kSlack : 0.f;
        const bool clip_on = clip > 0.f, proj_on = mmax > 0.f && mmax < 1e30f;
        bool bad = false;
        for (int t = 0; t < L; t++) {
            if (clip_on && en[t] > clip) bad = true;
            nS = (HAS_S ? gate[2][t] * nS : 0.f) + gate[1][t] * en[t] * kn[t];
            nM = (1.0f - gate[0][t]) * nM + nS;
            if (proj_on && nM * kSlack > mmax) bad = true;
        }
        if (bad) *flag = 1;
    }
}

__global__ void guard_clear_kernel(int *flag) { *flag = 0; }

int *g_host_flag = nullptr;

}  // namespace

bool force_sequential = false;

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
            hipLaunchKernelGGL((cw_guard_kernel<TOK, true>), grid, dim3(256), 0, stream(), k, v, alpha, theta, eta, m_states,
                               s_states, seq_len, chunk_size, nc, error_clip, m_norm_max, flag);
        else
            hipLaunchKernelGGL((cw_guard_kernel<TOK, false>), grid, dim3(256), 0, stream(), k, v, alpha, theta, eta, m_states,
                               s_states, seq_len, chunk_size, nc, error_clip, m_norm_max, flag);
        check_launch("cw_guard_kernel");
    }
    *g_host_flag = 1;
    check_hip(hipMemcpyAsync(g_host_flag, flag, sizeof(int), hipMemcpyDeviceToHost, stream()), "guard flag copy");
    check_hip(hipStreamSynchronize(stream()), "guard flag sync");
    return es.failed() || *g_host_flag != 0;
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
    if (mm && (!coupled(error_clip, m_norm_max) || guard_possible())) {
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
    if (mm && (!coupled(error_clip, m_norm_max) ||
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
