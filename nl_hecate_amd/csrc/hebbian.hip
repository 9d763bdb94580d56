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
// At d = 64 both directions take a chunk-parallel form instead (64-token chunks, a scan over the chunks,
// 64 x 64 products on the matrix cores), described at those kernels; the per-token kernels
// remain the path of every other width and of short sequences.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <algorithm>

#include "hebbian_generic.h"
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
// The forward's ownership of a row's columns: lane cq of the row's four takes the 16-byte pieces at columns
// 4 cq + 16 i (CP a multiple of 4; the CP consecutive columns cq * CP .. for d = 8).  A store instruction of a
// wave then writes 64 contiguous bytes per row instead of four 16-byte pieces 64 bytes apart; the forward with
// the whole trajectory as its output is bound by its stores.
template <int CP>
__device__ __forceinline__ void row_load(float (&dst)[CP], const float *row, int cq) {
    if constexpr (CP % 4 == 0) {
#pragma unroll
        for (int i = 0; i < CP; i += 4) {
            const float4 t = *reinterpret_cast<const float4 *>(row + 4 * i + 4 * cq);
            dst[i] = t.x; dst[i + 1] = t.y; dst[i + 2] = t.z; dst[i + 3] = t.w;
        }
    } else {
        gload<CP>(dst, row + cq * CP);
    }
}
template <int CP>
__device__ __forceinline__ void row_store(float *row, int cq, const float (&src)[CP]) {
    if constexpr (CP % 4 == 0) {
#pragma unroll
        for (int i = 0; i < CP; i += 4)
            *reinterpret_cast<float4 *>(row + 4 * i + 4 * cq) = make_float4(src[i], src[i + 1], src[i + 2], src[i + 3]);
    } else {
        gstore<CP>(row + cq * CP, src);
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
    int chunks;                   // > 0: workgroup x is chunk x % chunks of chain x / chunks, m_initial holds the
                                  // chunk-start states [chain][chunk][D*D] (trajectory mode only)
};

constexpr int kHC = 64;   // tokens per chunk of the chunk-parallel kernels

template <int D, int STORE>
__global__ __launch_bounds__(heb_threads(D)) void hebbian_fwd_kernel(HebFwdArgs a) {
    constexpr int CP = D / 4, T = 8;
    __shared__ __align__(16) float tile[2][T][3][D];   // k, q, v of a tile's tokens
    __shared__ float tal[2][T];
    const int tid = threadIdx.x, cq = tid & 3;
    const int b = a.chunks ? blockIdx.x / a.chunks : blockIdx.x, chunk = a.chunks ? blockIdx.x % a.chunks : 0;
    const int t_off = chunk * kHC, len = a.chunks ? min(kHC, a.seq_len - t_off) : a.seq_len;
    const bool inner_chunk = a.chunks && chunk + 1 < a.chunks;   // its last state is the next chunk's first store
    const int rl = min(tid >> 2, a.rows - 1);          // lanes beyond the rows (d = 8) shadow the last row
    const bool valid = (tid >> 2) < a.rows;
    const int r = blockIdx.y * a.rows + rl;            // a.rows rows of the chain per workgroup
    const size_t tok0 = (size_t)b * a.input_stride + t_off;
    const float *kb = a.k + tok0 * D, *qb = a.q + tok0 * D, *vb = a.v + tok0 * D;
    const float *ab = a.alpha + tok0;
    float *ms = a.m_states + ((size_t)b * a.states_per_chain + t_off) * D * D + r * D;   // this lane's row
    float *yb = a.y + ((size_t)b * a.seq_len + t_off) * D;
    float M[CP];
    row_load<CP>(M, a.m_initial + (a.chunks ? (size_t)blockIdx.x * D * D : (size_t)b * a.m_stride) + r * D, cq);
    if (valid) row_store<CP>(ms, cq, M);
    if (len == 0) return;
    int ck = 1;
    const int last = len - 1, ntile = (len + T - 1) / T;
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
            row_load<CP>(kc, &tile[buf][j][0][0], cq);
            row_load<CP>(qc, &tile[buf][j][1][0], cq);
            const float v_r = tile[buf][j][2][r], ret = 1.0f - tal[buf][j];
#pragma unroll
            for (int i = 0; i < CP; i++) M[i] = ret * M[i] + v_r * kc[i];
            if (STORE == HEB_TRAJ) {
                if (valid && !(inner_chunk && t == last)) row_store<CP>(ms + (size_t)(t + 1) * D * D, cq, M);
            } else if (((t + 1) % a.ckpt == 0) || (t + 1 == a.seq_len)) {
                if (valid) row_store<CP>(ms + (size_t)ck * D * D, cq, M);
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

// Forward in chunks (d = 64, trajectory mode): the state at the start of chunk c+1 is
// gamma_c M_{c,0} + P_c with P_c = sum_s rho(L-1, s) v_s k_s^T and gamma_c = A(L), so after one product
// per chunk and a scan over the chunks every chunk of every chain writes its part of the trajectory in
// its own workgroup (the trajectory is what the forward has to move: 16 KB per token and chain).
__global__ __launch_bounds__(256) void heb_chunk_fwd_seed_kernel(HebFwdArgs a, float *P, float *gamma, int nch);
__global__ __launch_bounds__(256) void heb_chunk_fwd_scan_kernel(const float *P, const float *gamma,
                                                                 const float *m_initial, int m_stride, float *Mstart,
                                                                 int nch);
bool launch_fwd_chunks(HebFwdArgs a, int batch);

template <int STORE>
bool launch_fwd(HebFwdArgs a, int d, int batch) {
    if (d != 8 && d != 16 && d != 32 && d != 64 && d != 128) return false;
    if (STORE == HEB_TRAJ && d == 64 && a.seq_len > 2 * kHC && a.chunks == 0 && launch_fwd_chunks(a, batch)) return true;
    const int groups = a.chunks ? batch * a.chunks : batch;
    a.rows = rows_per_workgroup(d, groups);
    const dim3 grid(groups, d / a.rows), block(4 * a.rows < 64 ? 64 : 4 * a.rows);
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

// ── backward in chunk-parallel matrix form (d = 64) ─────────────────────────
// The rule is linear in M, so with r_t = 1 - alpha_t and, inside a chunk of up to 64 tokens that
// starts at state M_0 and receives the gradient S from the tokens after it,
//     rho(tau, t) = prod_{t < r <= tau} r_r,   A(t) = prod_{r < t} r_r,   rho_L(t) = rho(L - 1, t),
//     E_t  = sum_{tau >= t} rho(tau, t) dy_tau q_tau^T + rho_L(t) S          (gradient w.r.t. M_{t+1})
//     M_t  = A(t) M_0 + sum_{s < t} rho(t - 1, s) v_s k_s^T
// every output is a product of 64 x 64 matrices:
//     d_v = (R o K Q^T) dY + rho_L o (K S^T)        d_k = (R o V dY^T) Q + rho_L o (V S)
//     d_q = (R o V dY^T)^T K + A(t+1) o (dY M_0)    d_alpha_t = -<M_t, E_t>  (four sums, below)
// with R[t][tau] = rho(tau, t) for t <= tau < L and 0 elsewhere.  Only the states at chunk starts are
// read (1/64 of the trajectory), no division is needed, and the chunks are independent once S is known:
// S_{c-1} = P_c + gamma_c S_c with P_c = sum_tau A(tau+1) dy_tau q_tau^T, gamma_c = A(L), a scan over
// the chunks of a chain that costs d*d multiply-adds per chunk.  Three launches: P and gamma per chunk,
// the scan, the gradients per chunk; all products on v_mfma_f32_16x16x4_f32 (fp32 in and out).
constexpr int kHL = 68;   // LDS row stride (= 4 mod 64: the operand reads of a wave fall on 64 banks)

__device__ __forceinline__ void heb_clear(f32x4 (&acc)[4]) {
#pragma unroll
    for (int jt = 0; jt < 4; jt++) acc[jt] = f32x4{0.f, 0.f, 0.f, 0.f};
}

// rows [0, L) of a [tokens, 64] block into an LDS matrix, zeros behind them
__device__ __forceinline__ void heb_stage_rows(float *dst, const float *src, int L, int tid) {
    for (int e = tid; e < kHC * 16; e += 256) {
        const int row = e >> 4, j = (e & 15) * 4;
        f32x4 x = f32x4{0.f, 0.f, 0.f, 0.f};
        if (row < L) x = *reinterpret_cast<const f32x4 *>(src + (size_t)row * 64 + j);
        *reinterpret_cast<f32x4 *>(dst + row * kHL + j) = x;
    }
}

// P_c and gamma_c of every chunk: one workgroup per (chain, chunk).
__global__ __launch_bounds__(256) void heb_chunk_seed_kernel(HebBwdArgs a, float *P, float *gamma, int nch) {
    __shared__ __align__(16) float sDY[kHC * kHL];
    __shared__ __align__(16) float sQ[kHC * kHL];
    __shared__ float sa[kHC + 1];
    const int tid = threadIdx.x, lane = tid & 63, wr = 16 * (tid >> 6), ml = lane & 15, kg = lane >> 4;
    const int chunk = blockIdx.x % nch, b = blockIdx.x / nch;
    const int t0 = a.t_start + chunk * kHC, L = min(kHC, a.t_end - t0);
    const size_t tok = (size_t)b * a.seq_len + t0;
    heb_stage_rows(sDY, a.d_y + tok * 64, L, tid);
    heb_stage_rows(sQ, a.q + tok * 64, L, tid);
    if (tid < 64) {
        // A(t + 1) = prod_{r <= t} (1 - alpha_r), constant behind the chunk's last token: a scan over the first wave
        float x = tid < L ? 1.f - a.alpha[tok + tid] : 1.f;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const float y = __shfl_up(x, o);
            if (tid >= o) x *= y;
        }
        sa[tid + 1] = x;
        if (tid == 0) sa[0] = 1.f;
    }
    __syncthreads();
    f32x4 acc[4];
    heb_clear(acc);
#pragma unroll 4
    for (int k0 = 0; k0 < kHC; k0 += 4) {
        const float av = sDY[(k0 + kg) * kHL + wr + ml] * sa[k0 + kg + 1];
#pragma unroll
        for (int jt = 0; jt < 4; jt++)
            acc[jt] = __builtin_amdgcn_mfma_f32_16x16x4f32(av, sQ[(k0 + kg) * kHL + 16 * jt + ml], acc[jt], 0, 0, 0);
    }
    float *dst = P + (size_t)blockIdx.x * 4096;
#pragma unroll
    for (int jt = 0; jt < 4; jt++) {
#pragma unroll
        for (int v = 0; v < 4; v++) dst[(wr + 4 * kg + v) * 64 + 16 * jt + ml] = acc[jt][v];
    }
    if (tid == 0) gamma[blockIdx.x] = sa[L];
}

// S_c for every chunk of a chain (the gradient entering the chunk from the tokens after it) and the
// gradient leaving the segment: element-wise over d*d, sequential over the chunks.
__global__ __launch_bounds__(256) void heb_chunk_scan_kernel(const float *P, const float *gamma, const float *seed,
                                                             float *S, float *d_m_out, int nch) {
    const int b = blockIdx.y, e = blockIdx.x * 256 + threadIdx.x;
    float sv = seed ? seed[(size_t)b * 4096 + e] : 0.f;
    for (int c = nch - 1; c >= 0; c--) {
        const size_t o = ((size_t)b * nch + c) * 4096 + e;
        S[o] = sv;
        sv = fmaf(gamma[b * nch + c], sv, P[o]);
    }
    d_m_out[(size_t)b * 4096 + e] = sv;
}

constexpr int kHebGradLds = (8 * kHC * kHL + 1024) * (int)sizeof(float);
constexpr int kHebGradThr = 512;   // 8 waves, two per SIMD: one's operand reads and epilogues run under the other's products

// acc[jt] += A B for the wave's 16-row strip (rows wr ..) and two 16-column tiles from column cb on; AT / BT read
// the operand transposed (A[i][k] = bufA[k][i], B[k][n] = bufB[n][k]).
template <bool AT, bool BT>
__device__ __forceinline__ void heb_half_mma(const float *bufA, const float *bufB, f32x4 (&acc)[2], int wr, int cb,
                                             int ml, int kg) {
#pragma unroll 4
    for (int k0 = 0; k0 < kHC; k0 += 4) {
        const float av = AT ? bufA[(k0 + kg) * kHL + wr + ml] : bufA[(wr + ml) * kHL + k0 + kg];
#pragma unroll
        for (int jt = 0; jt < 2; jt++) {
            const int col = cb + 16 * jt + ml;
            const float bv = BT ? bufB[col * kHL + k0 + kg] : bufB[(k0 + kg) * kHL + col];
            acc[jt] = __builtin_amdgcn_mfma_f32_16x16x4f32(av, bv, acc[jt], 0, 0, 0);
        }
    }
}
__device__ __forceinline__ void heb_clear2(f32x4 (&acc)[2]) {
    acc[0] = f32x4{0.f, 0.f, 0.f, 0.f};
    acc[1] = f32x4{0.f, 0.f, 0.f, 0.f};
}
// Wave w owns rows 16 (w / 2) .. of every product and the 32 columns from 32 (w % 2) on; sums over a row's 64
// columns are left as two halves (one per wave of the pair) and added where they are used.
__global__ __launch_bounds__(kHebGradThr) void heb_chunk_grads_kernel(HebBwdArgs a, const float *Sc, int nch,
                                                                      int ntask) {
    extern __shared__ __align__(16) float heb_lds[];
    float *bK = heb_lds, *bV = bK + kHC * kHL, *bQ = bV + kHC * kHL, *bDY = bQ + kHC * kHL, *bM = bDY + kHC * kHL;
    float *bW1 = bM + kHC * kHL, *bW2 = bW1 + kHC * kHL, *bR = bW2 + kHC * kHL;
    float *rr = bR + kHC * kHL, *aa = rr + 64, *rhoL = aa + 80, *A1 = rhoL + 64, *gs = A1 + 128, *colp = gs + 128;
    float *red = colp + 256;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, ml = lane & 15, kg = lane >> 4;
    const int strip = wave >> 1, half = wave & 1, wr = 16 * strip, cb = 32 * half;
    const int seg = a.t_end - a.t_start;
    // A workgroup walks over chunk tasks blockIdx.x, blockIdx.x + gridDim.x, ...; the six input matrices of the next
    // task (two 16-byte pieces per thread and matrix) are requested into registers as soon as this task's are in
    // LDS, so only the first task of a workgroup waits for HBM.
    f32x4 nx[5][2], nm0[2], m0r[2];
    float nrr = 1.f;
    auto fetch_task = [&](int task) {
        const int chunk = task % nch, b = task / nch;
        const int t0 = a.t_start + chunk * kHC, L = min(kHC, a.t_end - t0);
        const size_t tok = (size_t)b * a.seq_len + t0;
        const float *src[5] = {a.k + tok * 64, a.v + tok * 64, a.q + tok * 64, a.d_y + tok * 64,
                               Sc + (size_t)task * 4096};
        const float *m0 = a.m_states + ((size_t)b * (seg + 1) + (t0 - a.t_start)) * 4096;
#pragma unroll
        for (int it = 0; it < 2; it++) {
            const int e = tid + it * kHebGradThr, row = e >> 4, j = (e & 15) * 4;
#pragma unroll
            for (int m = 0; m < 5; m++)
                nx[m][it] = (m == 4 || row < L) ? *reinterpret_cast<const f32x4 *>(src[m] + (size_t)row * 64 + j)
                                                : f32x4{0.f, 0.f, 0.f, 0.f};
            nm0[it] = *reinterpret_cast<const f32x4 *>(m0 + (size_t)row * 64 + j);
        }
        if (tid < 64) nrr = tid < L ? 1.f - a.alpha[tok + tid] : 1.f;
    };
    if ((int)blockIdx.x < ntask) fetch_task(blockIdx.x);
    for (int task = blockIdx.x; task < ntask; task += gridDim.x) {
    const int chunk = task % nch, b = task / nch;
    const int t0 = a.t_start + chunk * kHC, L = min(kHC, a.t_end - t0);
    const size_t tok = (size_t)b * a.seq_len + t0;
    {
        float *dst[5] = {bK, bV, bQ, bDY, bM};   // bM: S first
#pragma unroll
        for (int it = 0; it < 2; it++) {
            const int e = tid + it * kHebGradThr, row = e >> 4, j = (e & 15) * 4;
#pragma unroll
            for (int m = 0; m < 5; m++) *reinterpret_cast<f32x4 *>(dst[m] + row * kHL + j) = nx[m][it];
            m0r[it] = nm0[it];
        }
        if (tid < 64) rr[tid] = nrr;
    }
    __syncthreads();
    if (task + (int)gridDim.x < ntask) fetch_task(task + gridDim.x);
    if (wave == 0) {
        // lane t builds row t of R from its diagonal rightwards; tau runs in lock step over the wave
        const int t = lane;
        float p = 1.f;
#pragma unroll 8
        for (int tau = 0; tau < kHC; tau++) {
            if (tau > t) p *= rr[tau];
            bR[t * kHL + tau] = (tau >= t && tau < L && t < L) ? p : 0.f;
        }
        rhoL[t] = t < L ? bR[t * kHL + L - 1] : 0.f;
    } else if (wave == 1) {
        // A(t) for t = 0 .. 64
        float p = 1.f;
        for (int q = 0; q < lane; q++) p *= rr[q];
        aa[lane] = p;
        if (lane == 63) aa[64] = p * rr[63];
    }
    // <M_0, S>
    {
        float part = 0.f;
#pragma unroll
        for (int it = 0; it < 2; it++) {
            const int e = tid + it * kHebGradThr, row = e >> 4, j = (e & 15) * 4;
            const f32x4 mv = m0r[it];
            const f32x4 sv = *reinterpret_cast<const f32x4 *>(bM + row * kHL + j);
            part += mv[0] * sv[0] + mv[1] * sv[1] + mv[2] * sv[2] + mv[3] * sv[3];
        }
        part = wave_allreduce(part);
        if (lane == 0) red[wave] = part;
    }
    // products with S: T1 = K S^T (rows of d_v), T2 = V S (rows of d_k), g_s = v_s^T S k_s
    f32x4 dv[2], dk[2], dq[2];
    heb_clear2(dv); heb_clear2(dk); heb_clear2(dq);
    heb_half_mma<false, true>(bK, bM, dv, wr, cb, ml, kg);
    heb_half_mma<false, false>(bV, bM, dk, wr, cb, ml, kg);
    __syncthreads();   // tables, red and every read of S are done
    const float m0s = ((red[0] + red[1]) + (red[2] + red[3])) + ((red[4] + red[5]) + (red[6] + red[7]));
#pragma unroll
    for (int v = 0; v < 4; v++) {
        const int row = wr + 4 * kg + v;
        float part = 0.f;
#pragma unroll
        for (int jt = 0; jt < 2; jt++) part = fmaf(dk[jt][v], bK[row * kHL + cb + 16 * jt + ml], part);
        part = group_allreduce<16>(part);
        if (ml == 0) gs[64 * half + row] = part;
        const float sL = rhoL[row];
#pragma unroll
        for (int jt = 0; jt < 2; jt++) { dv[jt][v] *= sL; dk[jt][v] *= sL; }
    }
#pragma unroll
    for (int it = 0; it < 2; it++) {   // M_0
        const int e = tid + it * kHebGradThr, row = e >> 4, j = (e & 15) * 4;
        *reinterpret_cast<f32x4 *>(bM + row * kHL + j) = m0r[it];
    }
    __syncthreads();
    // T3 = dY M_0: d_q starts as A(t+1) T3, and A1_tau = dy_tau^T M_0 q_tau
    heb_half_mma<false, false>(bDY, bM, dq, wr, cb, ml, kg);
#pragma unroll
    for (int v = 0; v < 4; v++) {
        const int row = wr + 4 * kg + v;
        float part = 0.f;
#pragma unroll
        for (int jt = 0; jt < 2; jt++) part = fmaf(dq[jt][v], bQ[row * kHL + cb + 16 * jt + ml], part);
        part = group_allreduce<16>(part);
        if (ml == 0) A1[64 * half + row] = part;
        const float sA = aa[row + 1];
#pragma unroll
        for (int jt = 0; jt < 2; jt++) dq[jt][v] *= sA;
    }
    // G1 = K Q^T, G2 = V dY^T (token x token); W1 = R o G1, W2 = R o G2, and G1 o G2 for d_alpha
    f32x4 g1[2], g2[2];
    heb_clear2(g1); heb_clear2(g2);
    heb_half_mma<false, true>(bK, bQ, g1, wr, cb, ml, kg);
    heb_half_mma<false, true>(bV, bDY, g2, wr, cb, ml, kg);
    __syncthreads();   // M_0 has been read
#pragma unroll
    for (int jt = 0; jt < 2; jt++) {
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const int o = (wr + 4 * kg + v) * kHL + cb + 16 * jt + ml;
            const float rv = bR[o];
            bW1[o] = rv * g1[jt][v];
            bW2[o] = rv * g2[jt][v];
            bM[o] = g1[jt][v] * g2[jt][v];
        }
    }
    __syncthreads();
    heb_half_mma<false, false>(bW1, bDY, dv, wr, cb, ml, kg);
    heb_half_mma<false, false>(bW2, bQ, dk, wr, cb, ml, kg);
    heb_half_mma<true, false>(bW2, bK, dq, wr, cb, ml, kg);
    // U[s][t] = sum_{tau >= t} rho(tau, t) (v_s . dy_tau)(k_s . q_tau)
    f32x4 u[2];
    heb_clear2(u);
    heb_half_mma<false, true>(bM, bR, u, wr, cb, ml, kg);
    float *dvo = a.d_v + tok * 64, *dko = a.d_k + tok * 64, *dqo = a.d_q + tok * 64;
#pragma unroll
    for (int v = 0; v < 4; v++) {
        const int row = wr + 4 * kg + v;
        if (row < L) {
#pragma unroll
            for (int jt = 0; jt < 2; jt++) {
                dvo[(size_t)row * 64 + cb + 16 * jt + ml] = dv[jt][v];
                dko[(size_t)row * 64 + cb + 16 * jt + ml] = dk[jt][v];
                dqo[(size_t)row * 64 + cb + 16 * jt + ml] = dq[jt][v];
            }
        }
    }
    // sum_{s < t} rho(t - 1, s) U[s][t]: columns of the wave's 16 rows, then over the four row strips
#pragma unroll
    for (int jt = 0; jt < 2; jt++) {
        const int t = cb + 16 * jt + ml;
        float part = 0.f;
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const int srow = wr + 4 * kg + v;
            if (srow < t) part = fmaf(bR[srow * kHL + t - 1], u[jt][v], part);
        }
        part = stride_allreduce<16>(part);
        if (kg == 0) colp[strip * 64 + t] = part;
    }
    __syncthreads();
    if (tid < L) {
        // d_alpha_t = -<M_t, E_t> = -( A(t) [sum_{tau>=t} rho(tau,t) A1_tau + rho_L(t) <M_0,S>]
        //                             + sum_{s<t} rho(t-1,s) [U[s][t] + rho_L(t) g_s] )
        const int t = tid;
        float s1 = 0.f, s4 = 0.f;
        for (int tau = t; tau < L; tau++) s1 = fmaf(bR[t * kHL + tau], A1[tau] + A1[64 + tau], s1);
        for (int s2 = 0; s2 < t; s2++) s4 = fmaf(bR[s2 * kHL + t - 1], gs[s2] + gs[64 + s2], s4);
        const float s3 = colp[t] + colp[64 + t] + colp[128 + t] + colp[192 + t];
        const float x = aa[t] * fmaf(rhoL[t], m0s, s1) + s3 + rhoL[t] * s4;
        a.d_alpha[tok + t] = -x;
    }
    __syncthreads();   // the next task's matrices and tables replace this one's
    }
}

// d = 64 only; false if the shape is not covered (the caller falls back to the sweep kernel).
bool launch_bwd_chunks(const HebBwdArgs &a, int batch) {
    const ErrorScope es;
    const int seg = a.t_end - a.t_start;
    if (seg <= 0) return false;
    const int nch = (seg + kHC - 1) / kHC;
    const size_t chunks = (size_t)batch * nch;
    float *P = scratch(5, chunks * 4096 * sizeof(float));
    float *gamma = scratch(6, chunks * sizeof(float));
    float *S = scratch(7, chunks * 4096 * sizeof(float));
    if (es.failed()) return true;
    hipLaunchKernelGGL(heb_chunk_seed_kernel, dim3((unsigned)chunks), dim3(256), 0, stream(), a, P, gamma, nch);
    check_launch("heb_chunk_seed_kernel");
    hipLaunchKernelGGL(heb_chunk_scan_kernel, dim3(16, batch), dim3(256), 0, stream(), P, gamma, a.d_m_seed, S,
                       a.d_m_out, nch);
    check_launch("heb_chunk_scan_kernel");
    check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(heb_chunk_grads_kernel),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, kHebGradLds), "dynamic LDS size");
    {
        KernelTimer kt("hebbian_bwd_kernel");
        const unsigned grid = (unsigned)std::min<size_t>(chunks, (size_t)compute_units());   // one workgroup fits a compute unit
        hipLaunchKernelGGL(heb_chunk_grads_kernel, dim3(grid), dim3(kHebGradThr), kHebGradLds, stream(), a, S, nch,
                           (int)chunks);
        check_launch("heb_chunk_grads_kernel");
    }
    return true;
}

__global__ __launch_bounds__(256) void heb_chunk_fwd_seed_kernel(HebFwdArgs a, float *P, float *gamma, int nch) {
    __shared__ __align__(16) float sV[kHC * kHL];
    __shared__ __align__(16) float sK[kHC * kHL];
    __shared__ float sb[kHC + 1];
    const int tid = threadIdx.x, lane = tid & 63, wr = 16 * (tid >> 6), ml = lane & 15, kg = lane >> 4;
    const int chunk = blockIdx.x % nch, b = blockIdx.x / nch;
    const int t0 = chunk * kHC, L = min(kHC, a.seq_len - t0);
    const size_t tok = (size_t)b * a.input_stride + t0;
    heb_stage_rows(sV, a.v + tok * 64, L, tid);
    heb_stage_rows(sK, a.k + tok * 64, L, tid);
    if (tid < 64) {
        // sb[s] = rho(L-1, s) = prod_{s < r <= L-1} (1 - alpha_r); sb[kHC] = A(L): a suffix scan over the first wave
        float x = tid < L ? 1.f - a.alpha[tok + tid] : 1.f;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const float y = __shfl_down(x, o);
            if (tid + o < 64) x *= y;
        }
        const float behind = __shfl_down(x, 1);   // prod_{r > s}
        sb[tid] = tid < L ? (tid == 63 ? 1.f : behind) : 0.f;
        if (tid == 0) sb[kHC] = x;
    }
    __syncthreads();
    f32x4 acc[4];
    heb_clear(acc);
#pragma unroll 4
    for (int k0 = 0; k0 < kHC; k0 += 4) {
        const float av = sV[(k0 + kg) * kHL + wr + ml] * sb[k0 + kg];
#pragma unroll
        for (int jt = 0; jt < 4; jt++)
            acc[jt] = __builtin_amdgcn_mfma_f32_16x16x4f32(av, sK[(k0 + kg) * kHL + 16 * jt + ml], acc[jt], 0, 0, 0);
    }
    float *dst = P + (size_t)blockIdx.x * 4096;
#pragma unroll
    for (int jt = 0; jt < 4; jt++) {
#pragma unroll
        for (int v = 0; v < 4; v++) dst[(wr + 4 * kg + v) * 64 + 16 * jt + ml] = acc[jt][v];
    }
    if (tid == 0) gamma[blockIdx.x] = sb[kHC];
}

__global__ __launch_bounds__(256) void heb_chunk_fwd_scan_kernel(const float *P, const float *gamma,
                                                                 const float *m_initial, int m_stride, float *Mstart,
                                                                 int nch) {
    const int b = blockIdx.y, e = blockIdx.x * 256 + threadIdx.x;
    float m = m_initial[(size_t)b * m_stride + e];
    for (int c = 0; c < nch; c++) {
        const size_t o = ((size_t)b * nch + c) * 4096 + e;
        Mstart[o] = m;
        m = fmaf(gamma[b * nch + c], m, P[o]);
    }
}

bool launch_fwd_chunks(HebFwdArgs a, int batch) {
    const ErrorScope es;
    const int nch = (a.seq_len + kHC - 1) / kHC;
    const size_t chunks = (size_t)batch * nch;
    float *P = scratch(5, chunks * 4096 * sizeof(float));
    float *gamma = scratch(6, chunks * sizeof(float));
    float *Mstart = scratch(7, chunks * 4096 * sizeof(float));
    if (es.failed()) return true;
    hipLaunchKernelGGL(heb_chunk_fwd_seed_kernel, dim3((unsigned)chunks), dim3(256), 0, stream(), a, P, gamma, nch);
    check_launch("heb_chunk_fwd_seed_kernel");
    hipLaunchKernelGGL(heb_chunk_fwd_scan_kernel, dim3(16, batch), dim3(256), 0, stream(), P, gamma, a.m_initial,
                       a.m_stride, Mstart, nch);
    check_launch("heb_chunk_fwd_scan_kernel");
    a.m_initial = Mstart;
    a.chunks = nch;
    return launch_fwd<HEB_TRAJ>(a, 64, batch);
}

bool launch_bwd(HebBwdArgs a, int d, int batch) {
    const ErrorScope es;
    if (d != 8 && d != 16 && d != 32 && d != 64 && d != 128) return false;
    if (d == 64 && launch_bwd_chunks(a, batch)) return true;
    a.rows = rows_per_workgroup(d, batch);
    const int parts = d / a.rows;
    if (parts > 1) {
        const size_t n = (size_t)parts * batch * a.seq_len;
        a.ws_dq = scratch(2, n * d * sizeof(float));
        a.ws_dk = scratch(3, n * d * sizeof(float));
        a.ws_gate = scratch(4, n * 4 * sizeof(float));
        if (es.failed()) return true;
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

}  // namespace
}  // namespace nlh

using namespace nlh;

extern "C" {

void hebbian_forward_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem, const float *alpha,
                              const float *m_initial, float *m_states, float *y, int seq_len, int d,
                              int batch_size, int input_stride, int m_stride) {
    if (!check_dims("hebbian_forward_f32_cuda", seq_len, d, batch_size) || batch_size == 0) return;
    const HebFwdArgs a{k_mem, v_mem, q_mem, alpha, m_initial, m_states, y, seq_len, input_stride, m_stride, 1, 0,
                       (long long)seq_len + 1, 0};
    if (launch_fwd<HEB_TRAJ>(a, d, batch_size)) return;
    if (hebbian_generic_check("hebbian_forward_f32_cuda", d))
        hebbian_forward_generic(k_mem, v_mem, q_mem, alpha, m_initial, m_states, y, seq_len, d, batch_size, input_stride,
                                m_stride, 0, (long long)seq_len + 1);
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
                       checkpoint_interval, 0, (long long)n_ckpt_count(seq_len, checkpoint_interval), 0};
    if (launch_fwd<HEB_CKPT>(a, d, 1)) return;
    if (hebbian_generic_check("hebbian_forward_ckpt_f32_cuda", d))
        hebbian_forward_generic(k_mem, v_mem, q_mem, alpha, m_initial, m_states, y, seq_len, d, 1, seq_len, d * d,
                                checkpoint_interval, (long long)n_ckpt_count(seq_len, checkpoint_interval));
}

void hebbian_backward_f32_cuda(const float *k_mem, const float *v_mem, const float *q_mem, const float *alpha,
                               const float *m_states, const float *d_y, float *d_k_mem, float *d_v_mem,
                               float *d_q_mem, float *d_alpha, float *d_m_initial, int seq_len, int d) {
    if (!check_dims("hebbian_backward_f32_cuda", seq_len, d, 1)) return;
    const HebBwdArgs a{k_mem, v_mem, q_mem, alpha, m_states, d_y, nullptr, d_k_mem, d_v_mem, d_q_mem, d_alpha,
                       d_m_initial, nullptr, nullptr, nullptr, seq_len, 0, seq_len, 0};
    if (launch_bwd(a, d, 1)) return;
    if (hebbian_generic_check("hebbian_backward_f32_cuda", d))
        hebbian_backward_generic(k_mem, v_mem, q_mem, alpha, m_states, d_y, nullptr, d_k_mem, d_v_mem, d_q_mem, d_alpha,
                                 d_m_initial, seq_len, 0, seq_len, d, 1);
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
    if (launch_bwd(a, d, batch_size)) return;
    if (hebbian_generic_check("hebbian_backward_segment_f32_cuda", d))
        hebbian_backward_generic(k_mem, v_mem, q_mem, alpha, m_states, d_y, d_m_seed, d_k_mem, d_v_mem, d_q_mem, d_alpha,
                                 d_m_out, seq_len, t_start, t_end, d, batch_size);
}

}  // extern "C"
