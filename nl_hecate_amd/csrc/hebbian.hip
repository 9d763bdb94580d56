// Hebbian rule: M_{t+1} = (1 - alpha_t) M_t + v_t k_t^T, y_t = M_{t+1} q_t (no error term, no theta).
// Contracts of core/kernels/hebbian_forward.cu / hebbian_backward.cu (core/src/cuda_ffi.rs:186-214,
// 240-245, 275-281); arithmetic of core/src/dispatch.rs:1566-1660.
//
// Lane (r, cq) keeps columns [cq*D/4, (cq+1)*D/4) of row r of M (forward) or of dM (backward) in
// registers for the whole sequence, four lanes per row.  Rows never mix in this rule, so a chain's rows
// are split over up to 8 workgroups (blockIdx.y) when the batch alone does not fill the chip: one
// compute unit moves only some 16 GB/s, and the trajectory is d*d floats per token.  The forward needs no exchange between lanes beyond a quad sum for y, so it runs without
// LDS and without barriers: its cost is the trajectory the contract asks for (d*d floats per token).
// The backward reads each trajectory matrix once (M_t of one token is M_{t+1} of the next one down),
// and has two column sums (d_q = M_{t+1}^T dy, d_k = dM^T v) and one full sum (d_alpha) per token:
// reduced inside the wave with DPP, across waves through a double-buffered LDS tile: one barrier per
// token.  With the rows split, each part writes partial sums and one more launch adds the parts.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "quad_rows.h"
#include "rule_common.h"
#include "runtime.h"

namespace nlh {
namespace {

// staging registers: arrays of HIP's float4 class are not promoted to registers here, the native vector is
typedef float f32x4 __attribute__((ext_vector_type(4)));
enum { HEB_TRAJ = 0, HEB_CKPT = 1 };

// threads per workgroup: 4 per row, at least one full wave (d = 8 leaves the upper half idle)
constexpr int heb_threads(int d) { return 4 * d < 64 ? 64 : 4 * d; }

// CP consecutive floats (CP = 2 for d = 8, else a multiple of 4)
template <int CP>
__device__ __forceinline__ void gload(float (&dst)[CP], const float *src) {
    if constexpr (CP % 4 == 0) {
#pragma unroll
        for (int i = 0; i < CP; i += 4) {
            const float4 t = *reinterpret_cast<const float4 *>(src + i);
            dst[i] = t.x; dst[i + 1] = t.y; dst[i + 2] = t.z; dst[i + 3] = t.w;
        }
    } else {
#pragma unroll
        for (int i = 0; i < CP; i += 2) {
            const float2 t = *reinterpret_cast<const float2 *>(src + i);
            dst[i] = t.x; dst[i + 1] = t.y;
        }
    }
}
template <int CP>
__device__ __forceinline__ void gstore(float *dst, const float (&src)[CP]) {
    if constexpr (CP % 4 == 0) {
        vec_store<CP>(dst, src);
    } else {
#pragma unroll
        for (int i = 0; i < CP; i += 2) *reinterpret_cast<float2 *>(dst + i) = make_float2(src[i], src[i + 1]);
    }
}
template <int CP>
__device__ __forceinline__ void clear(float (&x)[CP]) {
#pragma unroll
    for (int i = 0; i < CP; i++) x[i] = 0.f;
}

// Sums over the 16 rows of a wave of the CP columns a lane holds -> dst[column] (one writer per column).
template <int CP>
__device__ __forceinline__ void wave_column_sums(const float (&zv)[CP], float *dst, int lane, int c0) {
    if constexpr (CP >= 4) {
        float zo[CP / 4];
        rows_reduce_scatter<CP>(zv, zo);
        const int rho = lane >> 4, zoff = c0 + (CP / 2) * (rho >> 1) + (CP / 4) * (rho & 1);
        if (((lane & 15) >> 2) == 0) {
#pragma unroll
            for (int i = 0; i < CP / 4; i++) dst[zoff + i] = zo[i];
        }
    } else {
#pragma unroll
        for (int i = 0; i < CP; i++) {
            const float sum = rows_allreduce(zv[i]);
            if ((lane >> 2) == 0) dst[c0 + i] = sum;
        }
    }
}

// A tile of T tokens x NV vectors of D floats, fetched by the whole workgroup into registers (a plain
// local array) one tile ahead of its use and then written to LDS: a lane's per-token operands then cost
// LDS reads, and the HBM latency is paid once per tile instead of once per token.  vec[which] + token * D
// is the source of vector `which` (v0 .. v3); tok(j) maps the tile's j-th slot to a token (clamped by the
// caller to valid ones).
constexpr int tile_chunks(int d, int t, int nv) { return t * nv * d / 4; }                    // float4 chunks of a tile
constexpr int tile_per_lane(int d, int t, int nv) { return (tile_chunks(d, t, nv) + 63) / 64; }  // at the smallest workgroup (one wave)
template <int D, int T, int NV, typename Tok>
__device__ __forceinline__ void tile_fetch(f32x4 (&r)[tile_per_lane(D, T, NV)], float &al, const float *v0,
                                           const float *v1, const float *v2, const float *v3, const float *alpha,
                                           Tok tok) {
    constexpr int kChunks = tile_chunks(D, T, NV);
    const int tid = threadIdx.x;
#pragma unroll
    for (int i = 0; i < tile_per_lane(D, T, NV); i++) {
        const int c = min(tid + i * (int)blockDim.x, kChunks - 1);   // surplus lanes repeat the last chunk
        const int j = c / (NV * D / 4), rem = c % (NV * D / 4), which = rem / (D / 4);
        // the vector's base by selects on scalars: an array of pointers indexed by a lane value lands in scratch
        const float *src = which == 0 ? v0 : (which == 1 ? v1 : (which == 2 ? v2 : v3));
        r[i] = *reinterpret_cast<const f32x4 *>(src + (size_t)tok(j) * D + 4 * (rem % (D / 4)));
    }
    al = alpha[tok(min(tid, T - 1))];
}
template <int D, int T, int NV>
__device__ __forceinline__ void tile_commit(float (*tile)[NV][D], float *tal,
                                            const f32x4 (&r)[tile_per_lane(D, T, NV)], float al) {
    constexpr int kChunks = tile_chunks(D, T, NV);
    const int tid = threadIdx.x;
#pragma unroll
    for (int i = 0; i < tile_per_lane(D, T, NV); i++) {
        const int c = tid + i * blockDim.x;
        if (c < kChunks) {
            const int j = c / (NV * D / 4), rem = c % (NV * D / 4);
            *reinterpret_cast<f32x4 *>(&tile[j][rem / (D / 4)][4 * (rem % (D / 4))]) = r[i];
        }
    }
    if (tid < T) tal[tid] = al;
}

template <int CP>
__device__ __forceinline__ void lds_vec(float (&dst)[CP], const float *src) {
    if constexpr (CP % 4 == 0) {
        lds_read<CP>(dst, src);
    } else {
#pragma unroll
        for (int i = 0; i < CP; i++) dst[i] = src[i];
    }
}

struct HebFwdArgs {
    const float *k, *v, *q, *alpha, *m_initial;
    float *m_states, *y;
    int seq_len, input_stride, m_stride, ckpt, rows;
    long long states_per_chain;   // matrices of m_states per chain
};

template <int D, int STORE>
__global__ __launch_bounds__(heb_threads(D)) void hebbian_fwd_kernel(HebFwdArgs a) {
    constexpr int CP = D / 4, T = 8;
    __shared__ __align__(16) float tile[2][T][3][D];   // k, q, v of a tile's tokens
    __shared__ float tal[2][T];
    const int b = blockIdx.x, tid = threadIdx.x, cq = tid & 3, c0 = cq * CP;
    const int rl = min(tid >> 2, a.rows - 1);          // lanes beyond the rows (d = 8) shadow the last row
    const bool valid = (tid >> 2) < a.rows;
    const int r = blockIdx.y * a.rows + rl;            // a.rows rows of the chain per workgroup
    const size_t tok0 = (size_t)b * a.input_stride;
    const float *kb = a.k + tok0 * D, *qb = a.q + tok0 * D, *vb = a.v + tok0 * D;
    const float *ab = a.alpha + tok0;
    float *ms = a.m_states + (size_t)b * a.states_per_chain * D * D + r * D + c0;
    float *yb = a.y + (size_t)b * a.seq_len * D;
    float M[CP];
    gload<CP>(M, a.m_initial + (size_t)b * a.m_stride + r * D + c0);
    if (valid) gstore<CP>(ms, M);
    if (a.seq_len == 0) return;
    int ck = 1;
    const int last = a.seq_len - 1, ntile = (a.seq_len + T - 1) / T;
    f32x4 stage[tile_per_lane(D, T, 3)];
    float stage_al;
    tile_fetch<D, T, 3>(stage, stage_al, kb, qb, vb, vb, ab, [&](int j) { return min(j, last); });
    tile_commit<D, T, 3>(tile[0], tal[0], stage, stage_al);
    lds_barrier();
    for (int g = 0; g < ntile; g++) {
        const int buf = g & 1;
        tile_fetch<D, T, 3>(stage, stage_al, kb, qb, vb, vb, ab, [&](int j) { return min((g + 1) * T + j, last); });   // clamped: unconditional
        for (int j = 0; j < T; j++) {
            const int t = g * T + j;
            if (t > last) break;
            float kc[CP], qc[CP];
            lds_vec<CP>(kc, &tile[buf][j][0][c0]);
            lds_vec<CP>(qc, &tile[buf][j][1][c0]);
            const float v_r = tile[buf][j][2][r], ret = 1.0f - tal[buf][j];
#pragma unroll
            for (int i = 0; i < CP; i++) M[i] = ret * M[i] + v_r * kc[i];
            if (STORE == HEB_TRAJ) {
                if (valid) gstore<CP>(ms + (size_t)(t + 1) * D * D, M);
            } else if (((t + 1) % a.ckpt == 0) || (t + 1 == a.seq_len)) {
                if (valid) gstore<CP>(ms + (size_t)ck * D * D, M);
                ck++;
            }
            const float y_r = quad_allreduce(dotn<CP>(M, qc));
            if (valid && cq == 0) yb[(size_t)t * D + r] = y_r;
        }
        tile_commit<D, T, 3>(tile[buf ^ 1], tal[buf ^ 1], stage, stage_al);   // last read two barriers ago
        lds_barrier();
    }
}

struct HebBwdArgs {
    const float *k, *v, *q, *alpha, *m_states, *d_y, *d_m_seed;
    float *d_k, *d_v, *d_q, *d_alpha, *d_m_out;
    float *ws_dq, *ws_dk, *ws_gate;   // per-part partial sums when the rows are split (gridDim.y > 1)
    int seq_len, t_start, t_end, rows;
};

// Reverse sweep in groups of G tokens, RW rows of the chain per workgroup.  The trajectory matrices
// travel in a ring of G register sets (each element is used by exactly one lane, so LDS would add
// nothing): as soon as a token is done with its set, the matrix of the token G places further down is
// requested into it, so every load has G tokens of work to hide behind.  The small per-token vectors
// come through a token tile.  Inside a group a token costs no barrier: its per-wave column sums and its
// d_alpha partial are parked in LDS, and after the group's one barrier the workgroup adds the waves
// and writes the group's d_q, d_k, d_alpha rows in one go while the next group is already running.
// Lanes beyond the rows (d = 8) keep zeros: they take part in the wave reductions, and add nothing.
template <int D, int RW>
__global__ __launch_bounds__(heb_threads(RW)) void hebbian_bwd_kernel(HebBwdArgs a) {
    constexpr int CP = D / 4, NT = heb_threads(RW), NW = NT / 64, G = D == 128 ? 2 : (D == 64 ? 6 : 8);
    __shared__ __align__(16) float zp[2][G][2][NW][D];  // [group parity][token][d_q | d_k][wave][column]
    __shared__ float sp[2][G][NW];
    __shared__ __align__(16) float tile[2][G][4][D];    // k, q, dy, v of a group's tokens
    __shared__ float tal[2][G];
    const int b = blockIdx.x, tid = threadIdx.x, cq = tid & 3, c0 = cq * CP;
    const int part = blockIdx.y, parts = gridDim.y;
    const bool valid = (tid >> 2) < RW;
    const int r = part * RW + min(tid >> 2, RW - 1);
    const int wave = tid >> 6, lane = tid & 63;
    const int seg = a.t_end - a.t_start;
    const size_t tok0 = (size_t)b * a.seq_len;
    const float *kb = a.k + tok0 * D, *qb = a.q + tok0 * D, *dyb = a.d_y + tok0 * D, *vb = a.v + tok0 * D;
    const float *ab = a.alpha + tok0;
    const float *ms = a.m_states + (size_t)b * (seg + 1) * D * D + r * D + c0;
    float *dvb = a.d_v + tok0 * D;
    float *oq = parts == 1 ? a.d_q : a.ws_dq + (size_t)part * gridDim.x * a.seq_len * D;
    float *ok = parts == 1 ? a.d_k : a.ws_dk + (size_t)part * gridDim.x * a.seq_len * D;
    float *oa = parts == 1 ? a.d_alpha : a.ws_gate + (size_t)part * gridDim.x * a.seq_len * 4;
    const int oa_stride = parts == 1 ? 1 : 4;
    float dM[CP], Mn[CP];
    clear<CP>(dM); clear<CP>(Mn);
    if (valid && a.d_m_seed) gload<CP>(dM, a.d_m_seed + (size_t)b * D * D + r * D + c0);
    if (seg <= 0) {
        if (valid) gstore<CP>(a.d_m_out + (size_t)b * D * D + r * D + c0, dM);
        return;
    }
    if (valid) gload<CP>(Mn, ms + (size_t)seg * D * D);
    // slot j of group gi is token t_end - 1 - gi * G - j (clamped to the segment for the fetches)
    auto token = [&](int gi, int j) { return max(a.t_end - 1 - gi * G - j, a.t_start); };
    float Mr[G][CP];
    f32x4 stage[tile_per_lane(D, G, 4)];
    float stage_al;
    // one token: everything that stays inside the wave
    auto token_step = [&](int gi, int j, bool refill) {
        const int buf = gi & 1, t = a.t_end - 1 - gi * G - j;
        float kc[CP], qc[CP], zv[CP];
        lds_vec<CP>(kc, &tile[buf][j][0][c0]);
        lds_vec<CP>(qc, &tile[buf][j][1][c0]);
        const float dy_r = valid ? tile[buf][j][2][r] : 0.f, v_r = valid ? tile[buf][j][3][r] : 0.f;
        const float ret = 1.0f - tal[buf][j];
#pragma unroll
        for (int i = 0; i < CP; i++) { dM[i] = fmaf(dy_r, qc[i], dM[i]); zv[i] = Mn[i] * dy_r; }
        wave_column_sums<CP>(zv, zp[buf][j][0][wave], lane, c0);
#pragma unroll
        for (int i = 0; i < CP; i++) zv[i] = dM[i] * v_r;
        wave_column_sums<CP>(zv, zp[buf][j][1][wave], lane, c0);
        const float alp = wave_allreduce(dotn<CP>(Mr[j], dM));
        if (lane == 0) sp[buf][j][wave] = alp;
        const float dv_r = quad_allreduce(dotn<CP>(dM, kc));
        if (valid && cq == 0) dvb[(size_t)t * D + r] = dv_r;
#pragma unroll
        for (int i = 0; i < CP; i++) { dM[i] *= ret; Mn[i] = Mr[j][i]; }
        if (refill && valid) gload<CP>(Mr[j], ms + (size_t)(token(gi + 1, j) - a.t_start) * D * D);   // clamped: unconditional
    };
    // after the group's barrier: sums over the waves, rows of n tokens to HBM
    auto group_out = [&](int gi, int n) {
        const int buf = gi & 1;
#pragma unroll
        for (int i = 0; i < (G * 2 * D + NT - 1) / NT; i++) {
            const int e = tid + i * NT, j = e / (2 * D), which = (e / D) & 1, c = e % D;
            if (j < n) {
                float sum = 0.f;
#pragma unroll
                for (int x = 0; x < NW; x++) sum += zp[buf][j][which][x][c];
                const size_t o = tok0 + (a.t_end - 1 - gi * G - j);
                (which ? ok : oq)[o * D + c] = sum;
            }
        }
        if (tid < n) {
            float sum = 0.f;
#pragma unroll
            for (int x = 0; x < NW; x++) sum += sp[buf][tid][x];
            oa[(tok0 + (a.t_end - 1 - gi * G - tid)) * oa_stride] = -sum;
        }
    };
    const int ng = seg / G, rem = seg - ng * G;   // full groups, then a shorter one
#pragma unroll
    for (int j = 0; j < G; j++) {
        clear<CP>(Mr[j]);
        if (valid) gload<CP>(Mr[j], ms + (size_t)(token(0, j) - a.t_start) * D * D);
    }
    tile_fetch<D, G, 4>(stage, stage_al, kb, qb, dyb, vb, ab, [&](int j) { return token(0, j); });
    tile_commit<D, G, 4>(tile[0], tal[0], stage, stage_al);
    lds_barrier();
    for (int gi = 0; gi < ng; gi++) {
        tile_fetch<D, G, 4>(stage, stage_al, kb, qb, dyb, vb, ab, [&](int j) { return token(gi + 1, j); });
#pragma unroll
        for (int j = 0; j < G; j++) token_step(gi, j, true);
        tile_commit<D, G, 4>(tile[(gi & 1) ^ 1], tal[(gi & 1) ^ 1], stage, stage_al);
        lds_barrier();
        group_out(gi, G);
    }
    if (rem > 0) {
#pragma unroll
        for (int j = 0; j < G; j++)
            if (j < rem) token_step(ng, j, false);
        lds_barrier();
        group_out(ng, rem);
    }
    if (valid) gstore<CP>(a.d_m_out + (size_t)b * D * D + r * D + c0, dM);
}

// Rows of a chain per workgroup: the whole matrix unless the batch leaves compute units idle; at least
// 16 rows (one wave), at most 8 parts.
int rows_per_workgroup(int d, int batch) {
    int rows = d;
    while (rows > 16 && d / rows < 8 && (long long)batch * (d / rows) * 2 <= 512) rows /= 2;
    return rows;
}

template <int STORE>
bool launch_fwd(HebFwdArgs a, int d, int batch) {
    a.rows = rows_per_workgroup(d, batch);
    const dim3 grid(batch, d / a.rows), block(4 * a.rows < 64 ? 64 : 4 * a.rows);
    switch (d) {
        case 8: hipLaunchKernelGGL((hebbian_fwd_kernel<8, STORE>), grid, block, 0, stream(), a); break;
        case 16: hipLaunchKernelGGL((hebbian_fwd_kernel<16, STORE>), grid, block, 0, stream(), a); break;
        case 32: hipLaunchKernelGGL((hebbian_fwd_kernel<32, STORE>), grid, block, 0, stream(), a); break;
        case 64: hipLaunchKernelGGL((hebbian_fwd_kernel<64, STORE>), grid, block, 0, stream(), a); break;
        case 128: hipLaunchKernelGGL((hebbian_fwd_kernel<128, STORE>), grid, block, 0, stream(), a); break;
        default: return false;
    }
    check_launch("hebbian_fwd_kernel");
    return true;
}

template <int D, int RW>
void launch_bwd_rows(const HebBwdArgs &a, int batch) {
    hipLaunchKernelGGL((hebbian_bwd_kernel<D, RW>), dim3(batch, D / RW), dim3(heb_threads(RW)), 0, stream(), a);
}
template <int D>
void launch_bwd_d(const HebBwdArgs &a, int batch) {
    if constexpr (D <= 16) {
        launch_bwd_rows<D, D>(a, batch);
    } else {
        if (a.rows == D) launch_bwd_rows<D, D>(a, batch);
        else if (a.rows == D / 2) launch_bwd_rows<D, D / 2>(a, batch);
        else if constexpr (D >= 64) {
            if (a.rows == D / 4) launch_bwd_rows<D, D / 4>(a, batch);
            else if constexpr (D >= 128) launch_bwd_rows<D, D / 8>(a, batch);
        }
    }
}

bool launch_bwd(HebBwdArgs a, int d, int batch) {
    if (d != 8 && d != 16 && d != 32 && d != 64 && d != 128) return false;
    a.rows = rows_per_workgroup(d, batch);
    const int parts = d / a.rows;
    if (parts > 1) {
        const size_t n = (size_t)parts * batch * a.seq_len;
        a.ws_dq = scratch(2, n * d * sizeof(float));
        a.ws_dk = scratch(3, n * d * sizeof(float));
        a.ws_gate = scratch(4, n * 4 * sizeof(float));
        if (failed()) return true;
    }
    switch (d) {
        case 8: launch_bwd_d<8>(a, batch); break;
        case 16: launch_bwd_d<16>(a, batch); break;
        case 32: launch_bwd_d<32>(a, batch); break;
        case 64: launch_bwd_d<64>(a, batch); break;
        default: launch_bwd_d<128>(a, batch); break;
    }
    check_launch("hebbian_bwd_kernel");
    if (parts > 1)
        finalize_parts(a.ws_dq, a.ws_dk, a.ws_gate, a.d_q, a.d_k, a.d_alpha, nullptr, nullptr, parts, batch,
                       a.seq_len, d, a.t_start, a.t_end);
    return true;
}

void bad_d(const char *fn, int d) {
    fail("%s: d=%d is not supported by the gfx950 kernels (d in {8, 16, 32, 64, 128}).", fn, d);
}

}  // namespace
}  // namespace nlh

using namespace nlh;

extern "C" {

void hebbian_forward_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem, const float *alpha,
                              const float *m_initial, float *m_states, float *y, int seq_len, int d,
                              int batch_size, int input_stride, int m_stride) {
    if (!check_dims("hebbian_forward_f32_cuda", seq_len, d, batch_size) || batch_size == 0) return;
    const HebFwdArgs a{k_mem, v_mem, q_mem, alpha, m_initial, m_states, y, seq_len, input_stride, m_stride, 1, 0,
                       (long long)seq_len + 1};
    if (!launch_fwd<HEB_TRAJ>(a, d, batch_size)) bad_d("hebbian_forward_f32_cuda", d);
}

void hebbian_forward_ckpt_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem, const float *alpha,
                                   const float *m_initial, float *m_states, float *y, int seq_len, int d,
                                   int checkpoint_interval) {
    if (!check_dims("hebbian_forward_ckpt_f32_cuda", seq_len, d, 1)) return;
    if (checkpoint_interval <= 0) {
        fail("hebbian_forward_ckpt_f32_cuda: checkpoint_interval=%d must be > 0.", checkpoint_interval);
        return;
    }
    const HebFwdArgs a{k_mem, v_mem, q_mem, alpha, m_initial, m_states, y, seq_len, seq_len, d * d,
                       checkpoint_interval, 0, (long long)n_ckpt_count(seq_len, checkpoint_interval)};
    if (!launch_fwd<HEB_CKPT>(a, d, 1)) bad_d("hebbian_forward_ckpt_f32_cuda", d);
}

void hebbian_backward_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem, const float *alpha,
                               const float *m_states, const float *d_y, float *d_k_mem, float *d_v_mem,
                               float *d_q_mem, float *d_alpha, float *d_m_initial, int seq_len, int d) {
    if (!check_dims("hebbian_backward_f32_cuda", seq_len, d, 1)) return;
    const HebBwdArgs a{k_mem, v_mem, q_mem, alpha, m_states, d_y, nullptr, d_k_mem, d_v_mem, d_q_mem, d_alpha,
                       d_m_initial, nullptr, nullptr, nullptr, seq_len, 0, seq_len, 0};
    if (!launch_bwd(a, d, 1)) bad_d("hebbian_backward_f32_cuda", d);
}

void hebbian_backward_segment_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem,
                                       const float *alpha, const float *m_states, const float *d_y,
                                       const float *d_m_seed, float *d_k_mem, float *d_v_mem, float *d_q_mem,
                                       float *d_alpha, float *d_m_out, int t_start, int t_end, int d,
                                       int batch_size, int seq_len) {
    if (!check_dims("hebbian_backward_segment_f32_cuda", seq_len, d, batch_size) || batch_size == 0) return;
    if (t_start < 0 || t_end < t_start || t_end > seq_len) {
        fail("hebbian_backward_segment_f32_cuda: segment [%d, %d) is not inside [0, %d).", t_start, t_end, seq_len);
        return;
    }
    const HebBwdArgs a{k_mem, v_mem, q_mem, alpha, m_states, d_y, d_m_seed, d_k_mem, d_v_mem, d_q_mem, d_alpha,
                       d_m_out, nullptr, nullptr, nullptr, seq_len, t_start, t_end, 0};
    if (!launch_bwd(a, d, batch_size)) bad_d("hebbian_backward_segment_f32_cuda", d);
}

}  // extern "C"
