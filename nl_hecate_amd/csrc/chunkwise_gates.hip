// Backward of the frozen-M0 chunkwise Titans / Delta rule: the gate gradients d_alpha, d_eta.
//
//   d_alpha_s = -<M_(s-1), A_s>,   d_eta_s = <S_(s-1), B_s>
// with A_s, B_s the adjoints of M_s, S_s inside the chunk (core/kernels/titans_chunkwise_backward.cu:
// 118-358 accumulates the same inner products token by token on full d x d matrices):
//   A_s = sum_(t >= s) r[s][t] dy_t q_t^T + r[s][L-1] dMo
//   B_s = sum_(t >= s) c[t][s] dy_t q_t^T + c[L-1][s] dMo + bb[s][L-1] dSo
// Every inner product of a state with a rank-1 term is a scalar that obeys the rule's own recurrence:
// with u_s(t) = <M_s, dy_t q_t^T>, v_s(t) = <S_s, dy_t q_t^T>,
//   v_s(t) = eta_s v_(s-1)(t) + xs[s][t],   u_s(t) = keep_s u_(s-1)(t) + v_s(t),   u_(-1) = p0[t], v_(-1) = ps[t]
// where xs[s][t] = -theta_s (dy_t . e_s)(q_t . k_s) and p0, ps come from the gradient pass; the same holds
// for <M_s, dMo>, <S_s, dMo>, <S_s, dSo> with -theta_s e_s^T dMo k_s and -theta_s e_s^T dSo k_s as the
// per-token terms.  The weights r, c, bb obey forward recurrences in t.  So a chunk costs two sweeps of
// 64 steps on ONE wave and no matrix product, no coefficient table and no division:
//   sweep 1 (lane = t): u, v for s = 0..63, parked in LDS as rows s + 1
//   sweep 2 (lane = s): the weighted sums over t >= s with the weights advanced step by step.
// Row s is only ever read at t >= s, so the rows are packed as a triangle (row s starts at
// 64 s - s (s - 1) / 2 and holds t = s .. 63): half the LDS of a square, which is what decides how many
// chunks a compute unit works on at once.  Sweep 1 writes a row at consecutive addresses; in sweep 2
// lane s reads address 63 s - s (s - 1) / 2 + t, whose bank is t minus a triangular number: the
// triangular numbers of 32 consecutive s fall on 32 different banks.
// Gates travel as wave-uniform values (v_readlane); tokens beyond a short chunk carry keep = 1, eta = 0
// and zero terms.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "chunkwise_grads.h"
#include "runtime.h"

namespace nlh {
namespace {

constexpr int GW = 64;            // tokens per chunk tile
constexpr int GTRI = GW * (GW + 1) / 2 + GW;   // floats of one packed triangle, and a spare row behind it
constexpr int kGateWaves = 4;     // chunks per workgroup, one wave each
__host__ __device__ constexpr int tri_row(int r) { return GW * r - r * (r - 1) / 2; }

__device__ __forceinline__ float bcast(float x, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), lane));
}

// The launch carries a second, unrelated piece of the same backward in its last workgroups: the first stage of
// the sum over the batch of the gradient of the initial state (it depends on the adjoint scan only, is far too
// small for a launch of its own, and runs beside the sweeps): workgroup (e, y, z) adds `per` chains' matrices
// z (0: M, 1: S), elements 256 e .. 256 e + 255, into tmp[z][y]; a second launch adds the rows of tmp in a fixed order.
struct FirstSum {
    const float *src[2];   // [batch][chain_stride]: gradient of the initial M / S per chain
    float *tmp;            // [nsum][rows][d*d]
    size_t chain_stride;
    int batch, per, rows, nsum;
};
constexpr int kSumElems = 64 * 64;

template <bool HAS_S>
__global__ __launch_bounds__(64 * kGateWaves) void cw_gates_sweep_kernel(
    const float *__restrict__ alpha, const float *__restrict__ eta, const float *__restrict__ pvec,
    const float *__restrict__ xs, const float *__restrict__ scal, float *__restrict__ d_alpha,
    float *__restrict__ d_eta, int s, int C, int nc, int ntask, int sweep_blocks, FirstSum fs) {
    extern __shared__ float smem[];
    if ((int)blockIdx.x >= sweep_blocks) {
        const int bid = blockIdx.x - sweep_blocks, eb = bid % (kSumElems / 256), y = (bid / (kSumElems / 256)) % fs.rows,
                  z = bid / ((kSumElems / 256) * fs.rows);
        const float *st = fs.src[z];
        const int e = eb * 256 + threadIdx.x, b0 = y * fs.per, b1 = min(fs.batch, b0 + fs.per);
        float x = 0.f;
        for (int b = b0; b < b1; b++) x += st[(size_t)b * fs.chain_stride + e];
        fs.tmp[((size_t)z * fs.rows + y) * kSumElems + e] = x;
        return;
    }
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int task = blockIdx.x * kGateWaves + wv;
    if (task >= ntask) return;   // no barrier below: waves are independent
    float *U = smem + (size_t)wv * (HAS_S ? 2 : 1) * GTRI, *V = U + GTRI;
    const int chain = task / nc, ci = task % nc, t0 = ci * C, L = min(C, s - t0);
    const size_t tok = (size_t)chain * s + t0;
    const bool in = lane < L;
    const float keep_l = in ? 1.f - alpha[tok + lane] : 1.f;
    const float eta_l = (HAS_S && in) ? eta[tok + lane] : 0.f;
    const float4 pv = in ? *reinterpret_cast<const float4 *>(pvec + (tok + lane) * 4) : make_float4(0.f, 0.f, 0.f, 0.f);
    const float m0dm = scal[(size_t)task * 4 + 0], s0dm = scal[(size_t)task * 4 + 1], s0ds = scal[(size_t)task * 4 + 2];
    const float *x = xs + (size_t)task * GW * GW + lane;

    // ── sweep 1: lane = t ──
    float u = pv.x, v = pv.y;              // <M_s, dy_t q_t^T>, <S_s, dy_t q_t^T>
    float um = m0dm, vm = s0dm, vs = s0ds; // <M_s, dMo>, <S_s, dMo>, <S_s, dSo> (wave-uniform)
    float pum = um, pvm = vm, pvs = vs;    // their values at s = lane - 1
    U[lane] = u;
    if (HAS_S) V[lane] = v;
    // The whole column of per-token terms is requested up front.  Row s is used at t >= s only, and the
    // producer leaves out the 16 x 16 tiles that lie entirely below that: those are neither read nor used.
    float xr[GW];
#pragma unroll
    for (int i = 0; i < GW; i++) xr[i] = 0.f;
#pragma unroll
    for (int b = 0; b < GW / 16; b++)
        if ((lane >> 4) >= b) {
#pragma unroll
            for (int i = 16 * b; i < 16 * b + 16; i++) xr[i] = x[i * GW];
        }
#pragma unroll
    for (int sx = 0; sx < GW; sx++) {
        const float xv = xr[sx];
        const float kp = bcast(keep_l, sx), g1 = bcast(pv.z, sx);
        if (HAS_S) {
            const float et = bcast(eta_l, sx), g2 = bcast(pv.w, sx);
            v = fmaf(et, v, xv);
            vm = fmaf(et, vm, g1);
            vs = fmaf(et, vs, g2);
        } else {
            v = xv;
            vm = g1;
        }
        u = fmaf(kp, u, v);
        um = fmaf(kp, um, vm);
        if (sx + 1 < GW) {
            // row sx + 1, columns t >= sx + 1; the other lanes store to the spare row (no branch in the sweep)
            const int dst = lane >= sx + 1 ? tri_row(sx + 1) - (sx + 1) + lane : GTRI - GW + lane;
            U[dst] = u;
            if (HAS_S) V[dst] = v;
            if (lane == sx + 1) { pum = um; pvm = vm; pvs = vs; }
        }
    }
    // the rows are read back by other lanes of the same wave
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();

    // ── sweep 2: lane = s; weights r[s][t], c[t][s], bb[s][t] advance with t ──
    float rho = 1.f, cc = 1.f, bb = 1.f, accA = 0.f, accE = 0.f;
    // row s seen from column 0: what it reads at t < s belongs to earlier rows and is weighted by zero
    const float *Ur = U + tri_row(lane) - lane, *Vr = V + tri_row(lane) - lane;
    // unrolled by 8 only: fully unrolled, the lane reads of both sweeps (four scalars per step) overflowed the scalar
    // register file and were spilled
#pragma unroll 8
    for (int t = 0; t < GW; t++) {
        const float kp = bcast(keep_l, t);
        const bool after = t > lane && t < L, on = t >= lane;   // tokens beyond a short chunk change no weight
        rho *= after ? kp : 1.f;
        accA = fmaf(on ? rho : 0.f, Ur[t], accA);
        if (HAS_S) {
            const float et = bcast(eta_l, t);
            bb *= after ? et : 1.f;
            cc = after ? fmaf(kp, cc, bb) : cc;
            accE = fmaf(on ? cc : 0.f, Vr[t], accE);
        }
    }
    if (in) {
        d_alpha[tok + lane] = -fmaf(rho, pum, accA);
        if (HAS_S) d_eta[tok + lane] = accE + cc * pvm + bb * pvs;
    }
}

}  // namespace

void chunkwise_gate_gradients(const float *alpha, const float *eta, const float *pvec, const float *xs,
                              const float *scal, float *d_alpha, float *d_eta, int seq_len, int batch,
                              int chunk_size, bool has_s, const float *dm_first, const float *ds_first,
                              size_t chain_stride, int per, int nsum, float *tmp) {
    const ErrorScope es;
    const int nc = ceil_div(seq_len, chunk_size), ntask = batch * nc;
    const size_t lds = (size_t)kGateWaves * (has_s ? 2 : 1) * GTRI * sizeof(float);
    static bool attr_set = false;
    if (!attr_set) {
        check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(cw_gates_sweep_kernel<true>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)(kGateWaves * 2 * GTRI * 4)),
                  "dynamic LDS size");
        check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(cw_gates_sweep_kernel<false>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)(kGateWaves * GTRI * 4)),
                  "dynamic LDS size");
        attr_set = true;
    }
    if (es.failed()) return;
    static_assert(64 * kGateWaves == 256, "the sum workgroups take 256 elements each");
    const int sweep_blocks = ceil_div(ntask, kGateWaves), rows = ceil_div(batch, per);
    const FirstSum fs{{dm_first, ds_first}, tmp, chain_stride, batch, per, rows, nsum};
    const dim3 grid(sweep_blocks + (kSumElems / 256) * rows * nsum), block(64 * kGateWaves);
    KernelTimer kt("cw_gates_sweep_kernel");
    if (has_s)
        hipLaunchKernelGGL(cw_gates_sweep_kernel<true>, grid, block, lds, stream(), alpha, eta, pvec, xs, scal, d_alpha,
                           d_eta, seq_len, chunk_size, nc, ntask, sweep_blocks, fs);
    else
        hipLaunchKernelGGL(cw_gates_sweep_kernel<false>, grid, block, lds, stream(), alpha, nullptr, pvec, xs, scal,
                           d_alpha, nullptr, seq_len, chunk_size, nc, ntask, sweep_blocks, fs);
    check_launch("cw_gates_sweep_kernel");
}

}  // namespace nlh
