// The level step of a CMS layer behind the C ABI: what the reference's caller of the rule kernels does
// per level around them (gpu_memory_forward, core/src/gpu_forward.rs:1197-1382: projections, row L2 norm
// of k and q at model width, the three gate projections, head split; gpu_memory_backward and
// accumulate_projection_grads, core/src/gpu_backward.rs:459-640, 2047-2115), for a stack of Titans levels
// on the chunkwise rule with bf16 tokens.
//
// Forward: ONE kernel computes every projection of x (the attention branch's plain ones and k, v, q of
// every level) on the bf16 matrix cores and finishes them in registers: a workgroup keeps its 128 tokens
// of x as bf16 in LDS for the whole kernel, each of its eight waves owns 64 output columns and streams
// the weights of those columns from L2 in the order the matrix instruction wants them (packed once per
// call), so a weight element is read by exactly one wave of the workgroup and never touches LDS.  The
// epilogue of a level's k / v / q takes the row norms and the gate dot products from the accumulators
// (four consecutive columns of one token per lane), normalises, rounds once to bf16 and writes the
// head-major operands of the rule kernels: no fp32 projection output exists.
// Backward: the rule's head-major gradients go through one streaming pass (head merge, backward of the
// two normalisations, gate projections' weight sums) into ONE bf16 operand G [tokens, all projections],
// and d_x = G W, d_W = G^T x are two library GEMMs with fp32 accumulation.
#include <hip/hip_runtime.h>
#include <math.h>
#include <rocblas/rocblas.h>
#include <stdint.h>

#include "../../include/nl_hecate_ffi.h"
#include "bf16_tiles.h"
#include "chunkwise_grads.h"
#include "lane_ops.h"
#include "runtime.h"

namespace nlh {
namespace {

constexpr int PT = 128;       // tokens per workgroup of the projection kernel
constexpr int kPThr = 512;    // 8 waves
constexpr int kMaxLevels = 8;
constexpr int kMaxExtra = 4;
constexpr int kSThr = 256;    // streaming kernels
constexpr int kGThr = 768;    // the backward glue pass: 12 waves (three per SIMD at its 140 registers) share one partial row

__device__ __forceinline__ float sigmoid_(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float softplus_(float x) { return x > 20.0f ? x : logf(1.0f + expf(x)); }
__device__ __forceinline__ float dotv(const f32x4 &a, const float4 &b) { return a[0] * b.x + a[1] * b.y + a[2] * b.z + a[3] * b.w; }
__device__ __forceinline__ float sum_rows(float x) {   // over the four 16-lane rows of a wave, to every lane
    x = swapadd16(x, x);
    return swapadd32(x, x);
}
__device__ __forceinline__ void fma4(float4 &acc, float s, const float4 &x) {
    acc.x = fmaf(s, x.x, acc.x); acc.y = fmaf(s, x.y, acc.y); acc.z = fmaf(s, x.z, acc.z); acc.w = fmaf(s, x.w, acc.w);
}
__device__ __forceinline__ float4 bf4_to_f4(const bf16x4 &h) {
    return make_float4((float)h[0], (float)h[1], (float)h[2], (float)h[3]);
}
__device__ __forceinline__ bf16x4 f4_to_bf4(const float4 &x) {
    return bf16x4{(__bf16)x.x, (__bf16)x.y, (__bf16)x.z, (__bf16)x.w};
}


struct ProjArgs {
    const float *x;            // [n, D]
    u16 *x_bf16;               // [n, D]: x rounded to bf16 (the backward's GEMM operand); may be null
    const u16 *wfrag;          // packed weights, projection p at p * D * D (wfrag_pack_kernel)
    const u16 *ufrag;          // folded gate vectors of every level, [levels][D / 32][64][8] (gate_fold_kernel)
    u16 *extra_out[kMaxExtra]; // plain projections, bf16 [n, D] each
    const float *bias[kMaxLevels][3];   // b_alpha, b_theta, b_eta
    u16 *kh, *vh, *qh;         // [levels * bs * nh, s, hd]
    float *ah, *th, *eh;       // [levels * bs * nh, s]
    float *k_norms, *q_norms, *alpha, *theta, *eta;   // [levels, n]
    long long n;
    int bs, s, nh, n_extra, levels;
    float eps;
};

// Packs P matrices W_p [D, D] (row = output column, contraction index contiguous) into the order in which
// the projection kernel's waves read them, as A operands of v_mfma_f32_32x32x16_bf16:
// [p][column block of 64][k step of 16][tile of 32 columns][lane][8], lane l holding column 32 * tile + l % 32,
// contraction indices 16 * step + 8 * (l / 32) .. + 8: one 16-byte load per lane and tile, 2 KB contiguous per
// wave and step.
__global__ void wfrag_pack_kernel(const float *__restrict__ W, u16 *__restrict__ out, int P, int D) {
    const long long total = (long long)P * D * D / 8;
    const int KS = D / 16, CB = D / 64;
    for (long long o = (long long)blockIdx.x * blockDim.x + threadIdx.x; o < total; o += (long long)gridDim.x * blockDim.x) {
        const int lane = (int)(o & 63), c32 = (int)((o >> 6) & 1);
        long long r = o >> 7;
        const int ks = (int)(r % KS);
        r /= KS;
        const int cb = (int)(r % CB);
        const long long p = r / CB;
        const int row = 64 * cb + 32 * c32 + (lane & 31), k0 = 16 * ks + 8 * (lane >> 5);
        const float *src = W + (p * D + row) * D + k0;
        const float4 a = *reinterpret_cast<const float4 *>(src), b = *reinterpret_cast<const float4 *>(src + 4);
        const bf16x8 v = {(__bf16)a.x, (__bf16)a.y, (__bf16)a.z, (__bf16)a.w, (__bf16)b.x, (__bf16)b.y, (__bf16)b.z, (__bf16)b.w};
        *reinterpret_cast<bf16x8 *>(out + o * 8) = v;
    }
}

// The gate projections see k and v, which are projections of x themselves: [k | v] . w = x . (Wk^T w[:D] + Wv^T w[D:])
// up to the normalisation of k, a scalar per token.  This kernel folds the three gate vectors of a level through
// the level's (bf16-rounded, as the projection kernel multiplies them) Wk and Wv into six D-vectors u_q,
// q = (alpha, theta, eta) x (k part, v part), so that the projection kernel gets all six dot products of a token
// from ONE extra tile of 16 output columns instead of 6 D multiply-adds per token and phase in its epilogue.
// Each u is stored as a hi + lo pair of bf16 (the sums keep fp32 accuracy), as the A operand of that tile:
// row 2 q' = hi, row 2 q' + 1 = lo with q' = (k.alpha, k.theta, k.eta, v.alpha, v.theta, v.eta), rows 12..15 zero;
// element (row r, contraction index j) at [j / 32][lane = 16 ((j % 32) / 8) + r][j % 8].
struct FoldArgs { const float *w[kMaxLevels][3]; };
constexpr int kFoldSlices = 16;   // the sum over the D columns is cut into slices that run as separate workgroups
// part [levels][kFoldSlices][6][D]: slice sl's share of u_q[j]
__global__ __launch_bounds__(64) void gate_fold_partial_kernel(const float *__restrict__ w_levels, FoldArgs g,
                                                               float *__restrict__ part, int D) {
    const int lvl = blockIdx.y, sl = blockIdx.z, j = blockIdx.x * 64 + threadIdx.x;
    const int per = D / kFoldSlices, c0 = sl * per;
    if (j >= D) return;
    const float *Wk = w_levels + (size_t)lvl * 3 * D * D, *Wv = Wk + (size_t)D * D;
    float u[6] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll 8
    for (int c = c0; c < c0 + per; c++) {
        const float wk = (float)(__bf16)Wk[(size_t)c * D + j], wv = (float)(__bf16)Wv[(size_t)c * D + j];
#pragma unroll
        for (int q = 0; q < 3; q++) {
            u[q] = fmaf(wk, g.w[lvl][q][c], u[q]);
            u[3 + q] = fmaf(wv, g.w[lvl][q][D + c], u[3 + q]);
        }
    }
#pragma unroll
    for (int q = 0; q < 6; q++) part[(((size_t)lvl * kFoldSlices + sl) * 6 + q) * D + j] = u[q];
}
__global__ __launch_bounds__(64) void gate_fold_finish_kernel(const float *__restrict__ part, u16 *__restrict__ ufrag, int D) {
    const int lvl = blockIdx.y, j = blockIdx.x * 64 + threadIdx.x;
    if (j >= D) return;
    u16 *base = ufrag + ((size_t)lvl * (D / 32) + j / 32) * 512 + (size_t)16 * ((j % 32) / 8) * 8 + j % 8;
    __bf16 *out = reinterpret_cast<__bf16 *>(base);
#pragma unroll
    for (int q = 0; q < 6; q++) {
        float u = 0.f;
        for (int sl = 0; sl < kFoldSlices; sl++) u += part[(((size_t)lvl * kFoldSlices + sl) * 6 + q) * D + j];
        const __bf16 hi = (__bf16)u;
        out[(2 * q) * 8] = hi;
        out[(2 * q + 1) * 8] = (__bf16)(u - (float)hi);
    }
#pragma unroll
    for (int r = 12; r < 16; r++) out[r * 8] = (__bf16)0.f;
}

typedef float f32x16 __attribute__((ext_vector_type(16)));
constexpr int T32 = PT / 32;   // token tiles of 32 per workgroup

// acc[t32][c32][i] = sum_k W[col][k] x[token][k] with token = 32 t32 + lane % 32 of the workgroup's 128 and
// col = 32 c32 + 8 (i / 4) + 4 (lane / 32) + i % 4 of the wave's 64 columns, on v_mfma_f32_32x32x16_bf16 (measured
// on this part: 98 % of the data-sheet rate, where the 16 x 16 x 32 shape issues at 54 %).  The weights are the A
// operand straight from global memory (a ring of four 32-wide steps, requested three steps ahead), x the B operand
// from LDS (two token tiles per unit of four products, the next unit's pair requested before this unit's products
// are issued).  Fully unrolled, with the order of requests and products pinned: left to itself the scheduler sinks
// every load to its first use and the wave then waits a full memory latency per step.
template <int D>
__device__ __forceinline__ void project_block(const u16 *Xs, const u16 *wf, f32x16 (&acc)[T32][2]) {
    constexpr int XS = D + 8, KS = D / 32, RING = 4, UPK = 2 * (T32 / 2), UNITS = KS * UPK;   // units per 32-wide step
    const int lane = threadIdx.x & 63;
    const bf16x8 *wp = reinterpret_cast<const bf16x8 *>(wf) + lane;   // step ks: [2 k halves][2 column tiles][64 lanes]
    const u16 *xb = Xs + (lane & 31) * XS + 8 * (lane >> 5);
#pragma unroll
    for (int t = 0; t < T32; t++)
#pragma unroll
        for (int c = 0; c < 2; c++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[t][c][i] = 0.f;
    bf16x8 w[RING][4], b[2][2];
#pragma unroll
    for (int p = 0; p < RING - 1 && p < KS; p++)
#pragma unroll
        for (int f = 0; f < 4; f++) w[p][f] = wp[(p * 4 + f) * 64];
    b[0][0] = *reinterpret_cast<const bf16x8 *>(xb);
    b[0][1] = *reinterpret_cast<const bf16x8 *>(xb + 32 * XS);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < UNITS; u++) {
        // unit u: k half kh of step ks, token tiles 2 pr and 2 pr + 1
        const int ks = u / UPK, kh = (u % UPK) / (T32 / 2), pr = u % (T32 / 2);
        if (u % UPK == 0 && ks + RING - 1 < KS) {
#pragma unroll
            for (int f = 0; f < 4; f++) w[(ks + RING - 1) % RING][f] = wp[((ks + RING - 1) * 4 + f) * 64];
        }
        if (u + 1 < UNITS) {
            const int nks = (u + 1) / UPK, nkh = ((u + 1) % UPK) / (T32 / 2), npr = (u + 1) % (T32 / 2);
            b[(u + 1) & 1][0] = *reinterpret_cast<const bf16x8 *>(xb + 64 * npr * XS + 32 * nks + 16 * nkh);
            b[(u + 1) & 1][1] = *reinterpret_cast<const bf16x8 *>(xb + (64 * npr + 32) * XS + 32 * nks + 16 * nkh);
        }
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int c = 0; c < 2; c++)
                acc[2 * pr + h][c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(w[ks % RING][2 * kh + c], b[u & 1][h], acc[2 * pr + h][c], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
    }
}

// The wave's 32 x 64 tile of one token tile leaves through a small LDS buffer so that a store instruction writes
// whole rows: a lane holds, of ONE token, eight 4-column pieces (8 bytes each, 16 bytes apart); parked eight tokens
// at a time as [8 tokens][64 columns] and read back with lane l taking the 16-byte piece l % 8 of token l / 8, one
// instruction stores eight complete 128-byte rows.  A compute unit's store path moved the 8-byte pieces at about
// half the rate.  tb: the wave's own [8][72] bf16; row_ptr(R): where the wave's 64 columns of token R (0 .. 31 of
// this tile) go, or null past the end.
__device__ __forceinline__ void lanes_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
template <class RowPtr>
__device__ __forceinline__ void store_tile_rows(const f32x16 (&t)[2], float scale, u16 *tb, RowPtr row_ptr) {
    const int lane = threadIdx.x & 63, l32 = lane & 31, hf = lane >> 5;
#pragma unroll
    for (int h = 0; h < 4; h++) {
        if ((l32 >> 3) == h) {
#pragma unroll
            for (int c = 0; c < 2; c++)
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const f32x4 v = {t[c][4 * j] * scale, t[c][4 * j + 1] * scale, t[c][4 * j + 2] * scale, t[c][4 * j + 3] * scale};
                    bf16_store(tb, (l32 & 7) * 72 + 32 * c + 8 * j + 4 * hf, v);
                }
        }
        // lanes exchange data here: to the compiler a lane that skipped the writes above has nothing to wait for and
        // its read may run before the other lanes' writes (it did); the wave barrier keeps the order for all lanes
        lanes_sync();
        const bf16x8 r = *reinterpret_cast<const bf16x8 *>(tb + (lane >> 3) * 72 + (lane & 7) * 8);
        lanes_sync();
        u16 *dst = row_ptr(8 * h + (lane >> 3));
        if (dst) *reinterpret_cast<bf16x8 *>(dst + (lane & 7) * 8) = r;
    }
}

__device__ __forceinline__ float gate_act(int q, float pre) { return q == 1 ? softplus_(pre) : sigmoid_(pre); }

template <int D>
__global__ __launch_bounds__(kPThr) void level_project_kernel(ProjArgs a) {
    constexpr int XS = D + 8, CB = D / 64, D4 = D / 4, KS = D / 32;
    extern __shared__ __align__(16) unsigned char smem[];
    u16 *Xs = reinterpret_cast<u16 *>(smem);                                   // [PT][XS]
    float *red = reinterpret_cast<float *>(smem + (size_t)PT * XS * 2);         // [2][8][PT]: per-wave sums of squares
    float *gdot = red + 2 * 8 * PT;                                             // [2][PT][8]: x . u_q (6 used)
    float *tot = gdot + 2 * PT * 8;                                             // [PT]: 1 / max(|k|, eps)
    int *rowoff = reinterpret_cast<int *>(tot + PT);                            // [PT]: b * nh * s + t of the token
    u16 *tb = reinterpret_cast<u16 *>(rowoff + PT) + (threadIdx.x >> 6) * 8 * 72;  // per wave: [8][72], see store_tile_rows
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l16 = lane & 15, g = lane >> 4;
    const long long tok0 = (long long)blockIdx.x * PT, n = a.n;
    const bool wave_on = wave < CB;

    // x tile: fp32 -> bf16, into LDS (and out as the backward's operand)
    for (int i0 = 0; i0 < PT * D4; i0 += kPThr * 8) {
        float4 v[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int e = i0 + j * kPThr + tid, row = e / D4, c4 = e % D4;
            v[j] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (e < PT * D4 && tok0 + row < n) v[j] = *reinterpret_cast<const float4 *>(a.x + (tok0 + row) * D + 4 * c4);
        }
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int e = i0 + j * kPThr + tid, row = e / D4, c4 = e % D4;
            if (e >= PT * D4) continue;
            const bf16x4 h = f4_to_bf4(v[j]);
            *reinterpret_cast<bf16x4 *>(Xs + row * XS + 4 * c4) = h;
            if (a.x_bf16 && tok0 + row < n) *reinterpret_cast<bf16x4 *>(a.x_bf16 + (tok0 + row) * D + 4 * c4) = h;
        }
    }
    if (tid < PT) {
        const unsigned tok = (unsigned)(tok0 + tid), b = tok / (unsigned)a.s;
        rowoff[tid] = (int)(b * (unsigned)(a.nh * a.s) + (tok - b * (unsigned)a.s));
    }
    __syncthreads();

    f32x16 acc[T32][2];
    const size_t wave_frag = (size_t)wave * 64 * D;
    const int l32 = lane & 31, hf = lane >> 5;

    // plain projections: rounded once, token-major
    if (wave_on)
        for (int e = 0; e < a.n_extra; e++) {
            project_block<D>(Xs, a.wfrag + (size_t)e * D * D + wave_frag, acc);
            u16 *out = a.extra_out[e];
#pragma unroll
            for (int tt = 0; tt < T32; tt++)
                store_tile_rows(acc[tt], 1.0f, tb, [&](int r) -> u16 * {
                    const long long tok = tok0 + 32 * tt + r;
                    return tok < n ? out + tok * D + 64 * wave : nullptr;
                });
        }

    for (int lvl = 0; lvl < a.levels; lvl++) {
        const size_t pbase = (size_t)(a.n_extra + 3 * lvl) * D * D;
        const size_t chain0 = (size_t)lvl * a.bs * a.nh;
        float *gd = gdot + (lvl & 1) * PT * 8;
        {   // the six gate dot products of the wave's 16 tokens (token tile `wave`): one tile of 16 columns
            const bf16x8 *up = reinterpret_cast<const bf16x8 *>(a.ufrag) + (size_t)lvl * KS * 64 + lane;
            const u16 *xb = Xs + (16 * wave + l16) * XS + 8 * g;
            f32x4 ga = zero4();
#pragma unroll 4
            for (int ks = 0; ks < KS; ks++)
                ga = mfma32(up[ks * 64], *reinterpret_cast<const bf16x8 *>(xb + 32 * ks), ga);
            // lane group g holds rows 4g .. 4g + 3 = (hi, lo) of quantities 2g and 2g + 1
            if (g < 3) *reinterpret_cast<float2 *>(gd + (16 * wave + l16) * 8 + 2 * g) = make_float2(ga[0] + ga[1], ga[2] + ga[3]);
        }
#pragma unroll 1
        for (int p = 0; p < 3; p++) {   // k, v, q
            if (wave_on) project_block<D>(Xs, a.wfrag + pbase + (size_t)p * D * D + wave_frag, acc);
            if (p == 1) {   // v leaves as it is
                if (wave_on) {
#pragma unroll
                    for (int tt = 0; tt < T32; tt++)
                        store_tile_rows(acc[tt], 1.0f, tb, [&](int r) -> u16 * {
                            return tok0 + 32 * tt + r < n ? a.vh + (chain0 * a.s + rowoff[32 * tt + r] + (size_t)wave * a.s) * 64 : nullptr;
                        });
                }
                continue;
            }
            // k, q: the row norm over all D columns = over the eight waves.  The two half-waves hold different columns
            // of the same 32 tokens: one exchange per pair of token tiles leaves tile t32's totals in half t32 % 2, which
            // parks them as red[token][wave]; behind the barrier every lane reads the eight waves' sums of its own four
            // tokens as two 16-byte pieces each.
            float *rd = red + (p >> 1) * 8 * PT;
            if (wave_on) {
                float ss[T32];
#pragma unroll
                for (int tt = 0; tt < T32; tt++) {
                    ss[tt] = 0.f;
#pragma unroll
                    for (int c = 0; c < 2; c++)
#pragma unroll
                        for (int i = 0; i < 16; i++) ss[tt] += acc[tt][c][i] * acc[tt][c][i];
                }
                rd[(32 * hf + l32) * 8 + wave] = swapadd32(ss[0], ss[1]);          // lower half: tile 0, upper half: tile 1
                rd[(32 * (2 + hf) + l32) * 8 + wave] = swapadd32(ss[2], ss[3]);
            }
            __syncthreads();
            float inv[T32];
            {
                float4 pa[T32], pb[T32];
#pragma unroll
                for (int tt = 0; tt < T32; tt++) {
                    pa[tt] = *reinterpret_cast<const float4 *>(rd + (32 * tt + l32) * 8);
                    pb[tt] = *reinterpret_cast<const float4 *>(rd + (32 * tt + l32) * 8 + 4);
                }
#pragma unroll
                for (int tt = 0; tt < T32; tt++) {
                    float ssum = pa[tt].x;   // waves that own no columns (D < 512) never wrote their slot
                    if (CB > 1) ssum += pa[tt].y;
                    if (CB > 2) ssum += pa[tt].z;
                    if (CB > 3) ssum += pa[tt].w;
                    if (CB > 4) ssum += pb[tt].x;
                    if (CB > 5) ssum += pb[tt].y;
                    if (CB > 6) ssum += pb[tt].z;
                    if (CB > 7) ssum += pb[tt].w;
                    const float nrm = sqrtf(ssum);
                    inv[tt] = 1.0f / fmaxf(nrm, a.eps);
                    if (wave == 0 && hf == 0) {
                        const long long tok = tok0 + 32 * tt + l32;
                        if (p == 0) tot[32 * tt + l32] = inv[tt];
                        if (tok < n) (p == 0 ? a.k_norms : a.q_norms)[lvl * n + tok] = nrm;
                    }
                }
            }
            if (wave_on) {
                u16 *dst = p == 0 ? a.kh : a.qh;
#pragma unroll
                for (int tt = 0; tt < T32; tt++)
                    store_tile_rows(acc[tt], inv[tt], tb, [&](int r) -> u16 * {
                        return tok0 + 32 * tt + r < n ? dst + (chain0 * a.s + rowoff[32 * tt + r] + (size_t)wave * a.s) * 64 : nullptr;
                    });
            }
            if (p == 2 && tid < 3 * PT) {
                // the gates: one (token, gate) per thread; the q phase's barrier lies between wave 0's write of the
                // k norms' inverses, every wave's write of the gate dot products, and this read
                const int token = tid & (PT - 1), q = tid >> 7;   // PT = 128
                const long long tok = tok0 + token;
                const float pre = gd[token * 8 + q] * tot[token] + gd[token * 8 + 3 + q] + a.bias[lvl][q][0];
                const float val = gate_act(q, pre);
                if (tok < n) {
                    float *tm = q == 0 ? a.alpha : (q == 1 ? a.theta : a.eta), *hm = q == 0 ? a.ah : (q == 1 ? a.th : a.eh);
                    tm[lvl * n + tok] = val;
                    hm += chain0 * a.s + rowoff[token];
                    for (int h = 0; h < a.nh; h++) hm[(size_t)h * a.s] = val;
                }
            }
        }
    }
}

// ── backward glue ────────────────────────────────────────────────────────────────────────────────────
struct GateGradOut { float *w_alpha, *b_alpha, *w_theta, *b_theta, *w_eta, *b_eta; };

struct GradArgs {
    const float *dah, *dth, *deh;                            // the rule's gate gradients, [levels * bs * nh, s]
    const u16 *kh, *vh, *qh;                                 // the forward's head-major operands (k, q normalised)
    const float *k_norms, *q_norms, *alpha, *theta, *eta;    // [levels, n]
    u16 *G;                                                  // [n, g_ld]: level lvl's d_k, d_v, d_q at col0 + 3 lvl d + {0, d, 2d}
    long long g_ld, col0;
    float *part;                                             // [levels][gridDim.x][3][2d + 1]
    int bs, s, nh, levels;
    float eps;
};

// What is left between the rule's backward and the GEMMs once the rule writes d_k, d_v, d_q as bf16 columns of G
// itself (token-major, every head in its own 64 columns): one wave per token and level reads the token's d_k and d_q
// rows, takes them through the backward of the two row normalisations in place (from the normalised bf16 rows the
// forward wrote and the stored norms; d_v needs nothing), sums the gate gradients over the heads, applies the gate
// activations' derivatives, and accumulates the gate projections' weight and bias gradients per wave in registers
// (one partial row per workgroup, summed afterwards in a fixed order).  A lane owns 8 consecutive columns.
__global__ __launch_bounds__(kGThr) void level_grads_bf16_kernel(GradArgs a) {
    extern __shared__ float redg[];   // [3][2d + 1]
    const int lane = threadIdx.x & 63, wave_l = threadIdx.x >> 6, d = a.nh * 64, lvl = blockIdx.y, c0 = 8 * lane;
    const bool on = c0 < d;
    const int wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6, nwaves = (gridDim.x * blockDim.x) >> 6;
    const long long n = (long long)a.bs * a.s;
    const size_t chain0 = (size_t)lvl * a.bs * a.nh;
    const float inv_eps = 1.0f / a.eps;
    float acc[3][2][8];
    float accb[3] = {0.f, 0.f, 0.f};
#pragma unroll
    for (int gi = 0; gi < 3; gi++)
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int e = 0; e < 8; e++) acc[gi][h][e] = 0.f;
    auto widen = [](const bf16x8 &v, float (&f)[8]) {
#pragma unroll
        for (int e = 0; e < 8; e++) f[e] = (float)v[e];
    };
    // a wave owns a run of consecutive tokens: their gate gradients share cache lines (4 bytes per token and chain)
    const long long per = (n + nwaves - 1) / nwaves, tok_hi = min(n, (wave + 1) * per);
    for (long long tok = wave * per; tok < tok_hi; tok++) {
        const long long b = tok / a.s, t = tok - b * a.s;
        // every load of the token first: one memory round trip per token and wave
        u16 *grow = a.G + tok * a.g_ld + a.col0 + 3LL * lvl * d + c0;
        bf16x8 rgk{}, rgq{}, rk{}, rq{}, rv{};
        if (on) {
            const size_t o = ((chain0 + b * a.nh + c0 / 64) * a.s + t) * 64 + c0 % 64;
            rgk = *reinterpret_cast<const bf16x8 *>(grow);
            rgq = *reinterpret_cast<const bf16x8 *>(grow + 2 * d);
            rk = *reinterpret_cast<const bf16x8 *>(a.kh + o);
            rq = *reinterpret_cast<const bf16x8 *>(a.qh + o);
            rv = *reinterpret_cast<const bf16x8 *>(a.vh + o);
        }
        float dg[3] = {0.f, 0.f, 0.f};
        for (int h = lane; h < a.nh; h += 64) {
            const size_t o = (chain0 + b * a.nh + h) * a.s + t;
            dg[0] += a.dah[o]; dg[1] += a.dth[o]; dg[2] += a.deh[o];
        }
        const float al = a.alpha[lvl * n + tok], th = a.theta[lvl * n + tok], et = a.eta[lvl * n + tok];
        const float kn = a.k_norms[lvl * n + tok], qn = a.q_norms[lvl * n + tok];
#pragma unroll
        for (int gi = 0; gi < 3; gi++) dg[gi] = wave_allreduce(dg[gi]);
        dg[0] *= al * (1.0f - al);
        dg[1] *= 1.0f - expf(-th);
        dg[2] *= et * (1.0f - et);
#pragma unroll
        for (int gi = 0; gi < 3; gi++) accb[gi] += dg[gi];
        const float ki = 1.0f / fmaxf(kn, a.eps), qi = 1.0f / fmaxf(qn, a.eps);
        float gk[8], gq[8], kk[8], qq[8], vv[8];
        widen(rgk, gk);
        widen(rgq, gq);
        widen(rk, kk);
        widen(rq, qq);
        widen(rv, vv);
        float dk_dot = 0.f, dq_dot = 0.f;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            dk_dot += gk[e] * kk[e];
            dq_dot += gq[e] * qq[e];
#pragma unroll
            for (int gi = 0; gi < 3; gi++) {
                acc[gi][0][e] = fmaf(dg[gi], kk[e], acc[gi][0][e]);
                acc[gi][1][e] = fmaf(dg[gi], vv[e], acc[gi][1][e]);
            }
        }
        dk_dot = wave_allreduce(dk_dot);
        dq_dot = wave_allreduce(dq_dot);
        if (on) {
            bf16x8 ok, oq;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                ok[e] = (__bf16)(kn >= a.eps ? (gk[e] - kk[e] * dk_dot) * ki : gk[e] * inv_eps);
                oq[e] = (__bf16)(qn >= a.eps ? (gq[e] - qq[e] * dq_dot) * qi : gq[e] * inv_eps);
            }
            *reinterpret_cast<bf16x8 *>(grow) = ok;
            *reinterpret_cast<bf16x8 *>(grow + 2 * d) = oq;
        }
    }
    // the workgroup's partial row: the waves add their sums into LDS one after the other (fixed order)
    const int stride = 2 * d + 1;
    for (int w = 0; w < kGThr / 64; w++) {
        if (wave_l == w) {
#pragma unroll
            for (int gi = 0; gi < 3; gi++) {
                if (on) {
#pragma unroll
                    for (int h = 0; h < 2; h++)
#pragma unroll
                        for (int e = 0; e < 8; e++) {
                            float *r = redg + gi * stride + h * d + c0 + e;
                            if (w == 0) *r = acc[gi][h][e];
                            else *r += acc[gi][h][e];
                        }
                }
                if (lane == 0) {
                    if (w == 0) redg[gi * stride + 2 * d] = accb[gi];
                    else redg[gi * stride + 2 * d] += accb[gi];
                }
            }
        }
        __syncthreads();
    }
    float *pb = a.part + ((size_t)lvl * gridDim.x + blockIdx.x) * 3 * stride;
    for (int i = threadIdx.x; i < 3 * stride; i += kGThr) pb[i] = redg[i];
}

struct GateGradOuts { GateGradOut lv[kMaxLevels]; };

// Sums the workgroups' partial rows [levels][nblk][3][2d + 1] in a fixed order: a workgroup per (64 columns, gate,
// level), 16 thread groups that each take every 16th row, combined in order.
__global__ __launch_bounds__(1024) void level_gate_partials_kernel(const float *__restrict__ part, int nblk, int twoD,
                                                                   GateGradOuts out) {
    __shared__ float red[16][64];
    const int col = threadIdx.x & 63, seg = threadIdx.x >> 6, gi = blockIdx.y, lvl = blockIdx.z;
    const int i = blockIdx.x * 64 + col;
    const size_t stride = (size_t)twoD + 1;
    const float *p = part + (size_t)lvl * nblk * 3 * stride;
    float sum = 0.f;
    if (i <= twoD)
        for (int b = seg; b < nblk; b += 16) sum += p[((size_t)b * 3 + gi) * stride + i];
    red[seg][col] = sum;
    __syncthreads();
    if (seg != 0 || i > twoD) return;
#pragma unroll
    for (int q = 1; q < 16; q++) sum += red[q][col];
    const GateGradOut o = out.lv[lvl];
    float *w = gi == 0 ? o.w_alpha : (gi == 1 ? o.w_theta : o.w_eta);
    float *bias = gi == 0 ? o.b_alpha : (gi == 1 ? o.b_theta : o.b_eta);
    if (i < twoD) w[i] = sum;
    else bias[0] = sum;
}

// fp32 [n, d] sources side by side into bf16 columns of G (row stride ld), source i at column i * d
struct ColSrcs { const float *p[kMaxExtra]; };
__global__ void cols_to_bf16_kernel(ColSrcs src, int count, long long n, int d, u16 *__restrict__ G, long long ld) {
    const int d4 = d / 4;
    const long long total = n * count * d4;
    for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (long long)gridDim.x * blockDim.x) {
        const int c4 = (int)(e % d4), si = (int)((e / d4) % count);
        const long long r = e / ((long long)d4 * count);
        const float4 x = *reinterpret_cast<const float4 *>(src.p[si] + r * d + 4 * c4);
        *reinterpret_cast<bf16x4 *>(G + r * ld + (long long)si * d + 4 * c4) = f4_to_bf4(x);
    }
}

__global__ void f32_to_bf16_vec_kernel(const float *__restrict__ x, u16 *__restrict__ out, long long n4) {
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += (long long)gridDim.x * blockDim.x)
        *reinterpret_cast<bf16x4 *>(out + 4 * i) = f4_to_bf4(*reinterpret_cast<const float4 *>(x + 4 * i));
}

// last slot of every chain's chunk states -> the carried context memories (copy_final_m_batch, gpu_forward.rs:2824)
__global__ void final_states_kernel(const float *__restrict__ mc, const float *__restrict__ sc, float *__restrict__ m_ctx,
                                    float *__restrict__ s_ctx, long long chains, int slots, int dd4) {
    const long long total = chains * dd4;
    for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (long long)gridDim.x * blockDim.x) {
        const long long c = e / dd4;
        const int i = (int)(e % dd4);
        const size_t src = ((size_t)c * slots + slots - 1) * dd4 + i;
        reinterpret_cast<float4 *>(m_ctx)[e] = reinterpret_cast<const float4 *>(mc)[src];
        reinterpret_cast<float4 *>(s_ctx)[e] = reinterpret_cast<const float4 *>(sc)[src];
    }
}

// gate = sigmoid(scale * sum_l y_l); gated = attn * gate as bf16 (the output projection's operand)
struct LevelYs { const float *y[kMaxLevels]; };
__global__ void combine_gate_x1_kernel(LevelYs lv, int k, float scale, const u16 *__restrict__ attn, float *__restrict__ gate,
                                       u16 *__restrict__ gated, long long n4) {
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += (long long)gridDim.x * blockDim.x) {
        float4 sum = *reinterpret_cast<const float4 *>(lv.y[0] + 4 * i);
        for (int l = 1; l < k; l++) {
            const float4 y = *reinterpret_cast<const float4 *>(lv.y[l] + 4 * i);
            sum.x += y.x; sum.y += y.y; sum.z += y.z; sum.w += y.w;
        }
        const float4 at = bf4_to_f4(*reinterpret_cast<const bf16x4 *>(attn + 4 * i));
        float4 gt, o;
        gt.x = sigmoid_(sum.x * scale); gt.y = sigmoid_(sum.y * scale); gt.z = sigmoid_(sum.z * scale); gt.w = sigmoid_(sum.w * scale);
        o.x = at.x * gt.x; o.y = at.y * gt.y; o.z = at.z * gt.z; o.w = at.w * gt.w;
        *reinterpret_cast<float4 *>(gate + 4 * i) = gt;
        *reinterpret_cast<bf16x4 *>(gated + 4 * i) = f4_to_bf4(o);
    }
}

inline int stream_blocks(long long items, int cap) {
    long long b = (items + kSThr - 1) / kSThr;
    return (int)(b < 1 ? 1 : (b > cap ? cap : b));
}
inline bool al16(const void *p) { return (((uintptr_t)p) & 15) == 0; }

rocblas_handle blas() {
    static rocblas_handle h = nullptr;
    if (!h && rocblas_create_handle(&h) != rocblas_status_success) {
        h = nullptr;
        fail("level step: rocblas_create_handle failed.");
        return nullptr;
    }
    if (rocblas_set_stream(h, stream()) != rocblas_status_success) {
        fail("level step: rocblas_set_stream failed.");
        return nullptr;
    }
    return h;
}

// C (m x n, column-major, ldc, fp32) = op(A) op(B) + beta C with bf16 A, B and fp32 accumulation
bool gemm_bf16(const char *what, rocblas_operation ta, rocblas_operation tb, long long m, long long n, long long k, const u16 *A,
               long long lda, const u16 *B, long long ldb, float beta, float *C, long long ldc) {
    rocblas_handle h = blas();
    if (!h) return false;
    const float one = 1.0f;
    KernelTimer kt(what);
    const rocblas_status st = rocblas_gemm_ex(h, ta, tb, (rocblas_int)m, (rocblas_int)n, (rocblas_int)k, &one, A,
                                              rocblas_datatype_bf16_r, (rocblas_int)lda, B, rocblas_datatype_bf16_r,
                                              (rocblas_int)ldb, &beta, C, rocblas_datatype_f32_r, (rocblas_int)ldc, C,
                                              rocblas_datatype_f32_r, (rocblas_int)ldc, rocblas_datatype_f32_r,
                                              rocblas_gemm_algo_standard, 0, 0);
    if (st != rocblas_status_success) {
        fail("level step: rocblas_gemm_ex (%s) failed with status %d.", what, (int)st);
        return false;
    }
    return true;
}

// sum of `parts` buffers of count floats, in order
__global__ void sum_parts_kernel(const float *__restrict__ part, float *__restrict__ out, long long count4, int parts) {
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < count4; i += (long long)gridDim.x * blockDim.x) {
        float4 s = reinterpret_cast<const float4 *>(part)[i];
        for (int p = 1; p < parts; p++) {
            const float4 v = reinterpret_cast<const float4 *>(part)[p * count4 + i];
            s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
        }
        reinterpret_cast<float4 *>(out)[i] = s;
    }
}

// Weight gradient C [rows, m] (row-major) = G^T a over `tokens` tokens, a [tokens, m] (lda), G [tokens, rows] (ldb).
// A small output leaves most of the chip idle in one GEMM over all tokens: the tokens are then cut into slabs that
// run as one batched GEMM into partial outputs, added in a fixed order.
bool gemm_weight_grad(const char *what, long long m, long long rows, long long tokens, const u16 *a, long long lda, const u16 *G,
                      long long ldb, float *C) {
    const long long tiles = ((m + 127) / 128) * ((rows + 127) / 128);
    int parts = 1;
    while (parts < 16 && tiles * parts < 384 && tokens % (2 * parts) == 0 && tokens / (2 * parts) >= 1024) parts *= 2;
    if (parts == 1 || (m * rows) % 4)
        return gemm_bf16(what, rocblas_operation_none, rocblas_operation_transpose, m, rows, tokens, a, lda, G, ldb, 0.f, C, m);
    const ErrorScope es;
    float *part = scratch(30, (size_t)parts * m * rows * sizeof(float));
    rocblas_handle h = blas();
    if (es.failed() || !h) return false;
    const float one = 1.0f, zero = 0.0f;
    const long long kp = tokens / parts;
    {
        KernelTimer kt(what);
        const rocblas_status st = rocblas_gemm_strided_batched_ex(
            h, rocblas_operation_none, rocblas_operation_transpose, (rocblas_int)m, (rocblas_int)rows, (rocblas_int)kp, &one, a,
            rocblas_datatype_bf16_r, (rocblas_int)lda, kp * lda, G, rocblas_datatype_bf16_r, (rocblas_int)ldb, kp * ldb, &zero, part,
            rocblas_datatype_f32_r, (rocblas_int)m, m * rows, part, rocblas_datatype_f32_r, (rocblas_int)m, m * rows, parts,
            rocblas_datatype_f32_r, rocblas_gemm_algo_standard, 0, 0);
        if (st != rocblas_status_success) {
            fail("level step: rocblas_gemm_strided_batched_ex (%s) failed with status %d.", what, (int)st);
            return false;
        }
    }
    KernelTimer kt("sum_parts_kernel");
    hipLaunchKernelGGL(sum_parts_kernel, dim3(stream_blocks(m * rows / 4, 1024)), dim3(kSThr), 0, stream(), part, C, m * rows / 4, parts);
    check_launch("sum_parts_kernel");
    return true;
}

void to_bf16(const float *x, u16 *out, long long count) {
    KernelTimer kt("f32_to_bf16_vec_kernel");
    hipLaunchKernelGGL(f32_to_bf16_vec_kernel, dim3(stream_blocks(count / 4, 4096)), dim3(kSThr), 0, stream(), x, out, count / 4);
    check_launch("f32_to_bf16_vec_kernel");
}

bool step_dims_ok(const char *fn, int bs, int s, int nh, int hd, int levels, int n_extra, int chunk) {
    const int d = nh * hd;
    if (bs <= 0 || s <= 0 || nh <= 0 || hd != 64 || levels < 0 || levels > kMaxLevels || n_extra < 0 ||
        n_extra > kMaxExtra || (levels == 0 && n_extra == 0) || (d != 256 && d != 512) || chunk < 1 || chunk > 64 ||
        (long long)bs * s > 0x7fffffffLL / (long long)((3 * levels + n_extra) * d)) {
        fail("%s: needs head_dim = 64 (got %d), heads * head_dim in {256, 512} (got %d), 0 <= levels <= %d (got %d), "
             "0 <= n_extra <= %d (got %d), 1 <= chunk_size <= 64 (got %d), bs = %d and seq_len = %d positive and "
             "bs * seq_len * (projections * d) below 2^31.",
             fn, hd, d, kMaxLevels, levels, kMaxExtra, n_extra, chunk, bs, s);
        return false;
    }
    return true;
}

}  // namespace
}  // namespace nlh

using namespace nlh;

extern "C" {

void level_project_forward_bf16_rocm(const float *x, const float *w_extra, int n_extra, uint16_t *const *extra_out,
                                     const float *w_levels, const float *const *gate_params, uint16_t *x_bf16,
                                     uint16_t *k_heads, uint16_t *v_heads, uint16_t *q_heads, float *alpha_heads,
                                     float *theta_heads, float *eta_heads, float *k_norms, float *q_norms, float *alpha,
                                     float *theta, float *eta, int bs, int seq_len, int heads, int head_dim, int levels,
                                     float eps) {
    const ErrorScope es;
    if (!step_dims_ok("level_project_forward_bf16_rocm", bs, seq_len, heads, head_dim, levels, n_extra, 1)) return;
    const int d = heads * head_dim, P = n_extra + 3 * levels;
    const long long n = (long long)bs * seq_len;
    if (!al16(x) || !al16(w_extra) || !al16(w_levels) || (x_bf16 && !al16(x_bf16)) || !al16(k_heads) || !al16(v_heads) ||
        !al16(q_heads)) {
        fail("level_project_forward_bf16_rocm: buffers must be 16-byte aligned.");
        return;
    }
    u16 *wfrag = reinterpret_cast<u16 *>(scratch(24, ((size_t)P * d * d + (size_t)levels * d * 16) * sizeof(u16)));
    if (es.failed()) return;
    u16 *ufrag = wfrag + (size_t)P * d * d;
    float *fold_part = scratch(29, (size_t)(levels ? levels : 1) * kFoldSlices * 6 * d * sizeof(float));
    if (es.failed()) return;
    ProjArgs a{};
    FoldArgs fa{};
    a.x = x; a.x_bf16 = x_bf16; a.wfrag = wfrag; a.ufrag = ufrag;
    for (int e = 0; e < n_extra; e++) {
        if (!al16(extra_out[e])) { fail("level_project_forward_bf16_rocm: output %d is not 16-byte aligned.", e); return; }
        a.extra_out[e] = extra_out[e];
    }
    for (int l = 0; l < levels; l++) {
        const float *const *g = gate_params + 6 * l;
        for (int q = 0; q < 3; q++) {
            fa.w[l][q] = g[2 * q];
            a.bias[l][q] = g[2 * q + 1];
        }
    }
    a.kh = k_heads; a.vh = v_heads; a.qh = q_heads; a.ah = alpha_heads; a.th = theta_heads; a.eh = eta_heads;
    a.k_norms = k_norms; a.q_norms = q_norms; a.alpha = alpha; a.theta = theta; a.eta = eta;
    a.n = n; a.bs = bs; a.s = seq_len; a.nh = heads; a.n_extra = n_extra; a.levels = levels; a.eps = eps;
    {
        KernelTimer kt("wfrag_pack_kernel");
        if (n_extra)
            hipLaunchKernelGGL(wfrag_pack_kernel, dim3(stream_blocks((long long)n_extra * d * d / 8, 2048)), dim3(kSThr), 0,
                               stream(), w_extra, wfrag, n_extra, d);
        if (levels)
            hipLaunchKernelGGL(wfrag_pack_kernel, dim3(stream_blocks(3LL * levels * d * d / 8, 2048)), dim3(kSThr), 0, stream(),
                               w_levels, wfrag + (size_t)n_extra * d * d, 3 * levels, d);
        check_launch("wfrag_pack_kernel");
    }
    if (levels) {
        KernelTimer kt("gate_fold_kernel");
        hipLaunchKernelGGL(gate_fold_partial_kernel, dim3(ceil_div(d, 64), levels, kFoldSlices), dim3(64), 0, stream(), w_levels,
                           fa, fold_part, d);
        hipLaunchKernelGGL(gate_fold_finish_kernel, dim3(ceil_div(d, 64), levels), dim3(64), 0, stream(), fold_part, ufrag, d);
        check_launch("gate_fold_kernel");
    }
    const size_t lds = (size_t)PT * (d + 8) * 2 + (2 * 8 * PT + 2 * PT * 8 + PT + PT) * sizeof(float) + 8 * 8 * 72 * 2;
    static bool attr_set = false;
    if (!attr_set) {
        check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(level_project_kernel<512>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)((size_t)PT * 520 * 2 + 17408 + 9216)), "dynamic LDS size");
        check_hip(hipFuncSetAttribute(reinterpret_cast<const void *>(level_project_kernel<256>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)((size_t)PT * 264 * 2 + 17408 + 9216)), "dynamic LDS size");
        attr_set = true;
    }
    if (es.failed()) return;
    KernelTimer kt("level_project_kernel");
    const dim3 grid(ceil_div(n, PT));
    if (d == 512) hipLaunchKernelGGL(level_project_kernel<512>, grid, dim3(kPThr), lds, stream(), a);
    else hipLaunchKernelGGL(level_project_kernel<256>, grid, dim3(kPThr), lds, stream(), a);
    check_launch("level_project_kernel");
}

void titans_levels_forward_bf16_rocm(const float *x, const float *w_extra, int n_extra, uint16_t *const *extra_out,
                                     const float *w_levels, const float *const *gate_params, float *m_context,
                                     float *s_context, uint16_t *x_bf16, uint16_t *k_heads, uint16_t *v_heads,
                                     uint16_t *q_heads, float *alpha_heads, float *theta_heads, float *eta_heads,
                                     float *k_norms, float *q_norms, float *alpha, float *theta, float *eta,
                                     float *m_chunk_states, float *s_chunk_states, float *y_tokens, int bs, int seq_len,
                                     int heads, int head_dim, int levels, int chunk_size, float eps) {
    const ErrorScope es;
    if (!step_dims_ok("titans_levels_forward_bf16_rocm", bs, seq_len, heads, head_dim, levels, n_extra, chunk_size)) return;
    level_project_forward_bf16_rocm(x, w_extra, n_extra, extra_out, w_levels, gate_params, x_bf16, k_heads, v_heads, q_heads,
                                    alpha_heads, theta_heads, eta_heads, k_norms, q_norms, alpha, theta, eta, bs, seq_len,
                                    heads, head_dim, levels, eps);
    if (es.failed() || levels == 0) return;
    const int chains = levels * bs * heads, nc = (seq_len + chunk_size - 1) / chunk_size;
    titans_chunkwise_forward_bf16_tokens_rocm(k_heads, v_heads, q_heads, alpha_heads, theta_heads, eta_heads, m_context,
                                              s_context, m_chunk_states, s_chunk_states, y_tokens, seq_len, head_dim, chains,
                                              chunk_size, heads, levels);
    if (es.failed()) return;
    KernelTimer kt("final_states_kernel");
    const int dd4 = head_dim * head_dim / 4;
    hipLaunchKernelGGL(final_states_kernel, dim3(stream_blocks((long long)chains * dd4, 2048)), dim3(kSThr), 0, stream(),
                       m_chunk_states, s_chunk_states, m_context, s_context, (long long)chains, nc + 1, dd4);
    check_launch("final_states_kernel");
}

uint16_t *level_grad_operand_rocm(int bs, int seq_len, int heads, int head_dim, int levels, int n_extra, long long *ld) {
    const ErrorScope es;
    if (!step_dims_ok("level_grad_operand_rocm", bs, seq_len, heads, head_dim, levels, n_extra, 1)) return nullptr;
    const long long n = (long long)bs * seq_len, R = (long long)(n_extra + 3 * levels) * heads * head_dim;
    if (ld) *ld = R;
    return reinterpret_cast<uint16_t *>(scratch(26, (size_t)n * R * sizeof(u16)));
}

void titans_levels_backward_bf16_rocm(const uint16_t *x_bf16, const float *w_extra, int n_extra, const float *const *d_extra,
                                      const float *w_levels, const uint16_t *k_heads, const uint16_t *v_heads,
                                      const uint16_t *q_heads, const float *alpha_heads, const float *theta_heads,
                                      const float *eta_heads, const float *k_norms, const float *q_norms, const float *alpha,
                                      const float *theta, const float *eta, const float *m_chunk_states,
                                      const float *s_chunk_states, const float *d_y_tokens, float *d_x, float *d_w_extra,
                                      float *d_w_levels, float *const *d_gate_params, float *d_m_initial, float *d_s_initial,
                                      int bs, int seq_len, int heads, int head_dim, int levels, int chunk_size, float eps) {
    const ErrorScope es;
    if (!step_dims_ok("titans_levels_backward_bf16_rocm", bs, seq_len, heads, head_dim, levels, n_extra, chunk_size)) return;
    const int d = heads * head_dim, P = n_extra + 3 * levels, chains = levels * bs * heads;
    const long long n = (long long)bs * seq_len, R = (long long)P * d;
    if (!al16(x_bf16) || !al16(d_x) || !al16(w_extra) || !al16(w_levels)) {
        fail("titans_levels_backward_bf16_rocm: buffers must be 16-byte aligned.");
        return;
    }
    const size_t gate_f = (size_t)chains * seq_len;
    float *hg = scratch(25, (3 * gate_f + 4) * sizeof(float));                  // d_alpha, d_theta, d_eta per chain and token
    u16 *G = reinterpret_cast<u16 *>(scratch(26, (size_t)n * R * sizeof(u16)));
    u16 *wb = reinterpret_cast<u16 *>(scratch(27, (size_t)R * d * sizeof(u16)));
    const int nblk = (int)std::min<long long>(compute_units(), (n * 64 + kGThr - 1) / kGThr);
    const size_t prow = 3 * (2 * (size_t)d + 1);
    float *part = scratch(28, (size_t)(levels ? levels : 1) * nblk * prow * sizeof(float));
    if (es.failed()) return;
    float *dah = hg, *dth = dah + gate_f, *deh = dth + gate_f;
    if (levels) {
        // the rule writes d_k, d_v, d_q straight into the level's columns of G: chain (level, batch element, head) owns
        // columns col0 + 3 level d + {0, d, 2d} + 64 head .. + 64 of the rows of its batch element
        GradOut16 out{};
        out.gk = G + (size_t)n_extra * d;
        out.gv = out.gk + d;
        out.gq = out.gk + 2 * d;
        out.rows = HeadRows{3LL * d, (long long)seq_len * R, 64, R, bs * heads, heads};
        titans_chunkwise_backward_bf16_tokens_g16(k_heads, v_heads, q_heads, alpha_heads, theta_heads, eta_heads,
                                                  m_chunk_states, s_chunk_states, d_y_tokens, out, dah, dth, deh, d_m_initial,
                                                  d_s_initial, seq_len, head_dim, chains, chunk_size, heads, levels, 0);
        if (es.failed()) return;
        GradArgs ga{};
        ga.dah = dah; ga.dth = dth; ga.deh = deh;
        ga.kh = k_heads; ga.vh = v_heads; ga.qh = q_heads;
        ga.k_norms = k_norms; ga.q_norms = q_norms; ga.alpha = alpha; ga.theta = theta; ga.eta = eta;
        ga.G = G; ga.g_ld = R; ga.col0 = (long long)n_extra * d; ga.part = part;
        ga.bs = bs; ga.s = seq_len; ga.nh = heads; ga.levels = levels; ga.eps = eps;
        {
            KernelTimer kt("level_grads_bf16_kernel");
            hipLaunchKernelGGL(level_grads_bf16_kernel, dim3(nblk, levels), dim3(kGThr), prow * sizeof(float), stream(), ga);
            check_launch("level_grads_bf16_kernel");
        }
        GateGradOuts go{};
        for (int l = 0; l < levels; l++) {
            float *const *g = d_gate_params + 6 * l;
            go.lv[l] = GateGradOut{g[0], g[1], g[2], g[3], g[4], g[5]};
        }
        KernelTimer kt("level_gate_partials_kernel");
        hipLaunchKernelGGL(level_gate_partials_kernel, dim3(ceil_div(2 * d + 1, 64), 3, levels), dim3(1024), 0, stream(), part,
                           nblk, 2 * d, go);
        check_launch("level_gate_partials_kernel");
    }
    if (n_extra) {
        int given = 0;
        for (int e = 0; e < n_extra; e++) given += d_extra[e] != nullptr;
        if (given != 0 && given != n_extra) {
            fail("titans_levels_backward_bf16_rocm: d_extra must hold %d pointers or none (gradients already in the operand).", n_extra);
            return;
        }
        if (given) {
            ColSrcs cs{};
            for (int e = 0; e < n_extra; e++) {
                if (!al16(d_extra[e])) { fail("titans_levels_backward_bf16_rocm: gradient %d is not 16-byte aligned.", e); return; }
                cs.p[e] = d_extra[e];
            }
            KernelTimer kt("cols_to_bf16_kernel");
            hipLaunchKernelGGL(cols_to_bf16_kernel, dim3(stream_blocks(n * n_extra * (d / 4), 4096)), dim3(kSThr), 0, stream(), cs,
                               n_extra, n, d, G, R);
            check_launch("cols_to_bf16_kernel");
        }
        to_bf16(w_extra, wb, (long long)n_extra * d * d);
    }
    if (levels) to_bf16(w_levels, wb + (size_t)n_extra * d * d, 3LL * levels * d * d);
    if (es.failed()) return;
    // d_x [n, d] = G [n, R] Wb [R, d];  d_W [R, d] = G^T x  (row-major buffers as column-major operands)
    if (!gemm_bf16("gemm d_x", rocblas_operation_none, rocblas_operation_none, d, n, R, wb, d, G, R, 0.f, d_x, d)) return;
    // the weight gradients: one product when the two outputs are one buffer (a layer's packed gradients)
    if (n_extra && levels && d_w_levels == d_w_extra + (size_t)n_extra * d * d) {
        gemm_weight_grad("gemm d_w", d, R, n, x_bf16, d, G, R, d_w_extra);
        return;
    }
    if (n_extra && !gemm_weight_grad("gemm d_w", d, (long long)n_extra * d, n, x_bf16, d, G, R, d_w_extra)) return;
    if (levels) gemm_weight_grad("gemm d_w", d, 3LL * levels * d, n, x_bf16, d, G + (size_t)n_extra * d, R, d_w_levels);
}

void cms_combine_gate_bf16x1_rocm(const float *const *y_levels, int k, const uint16_t *attn_out, float *gate,
                                  uint16_t *gated_bf16, long long n) {
    if (k < 1 || k > kMaxLevels) { fail("cms_combine_gate_bf16x1_rocm: k=%d must be in [1, %d].", k, kMaxLevels); return; }
    if (n <= 0) return;
    if (n % 4 || (((uintptr_t)attn_out) & 7) || !al16(gate) || (((uintptr_t)gated_bf16) & 7)) {
        fail("cms_combine_gate_bf16x1_rocm: n=%lld must be a multiple of 4 and the buffers aligned.", n);
        return;
    }
    LevelYs lv{};
    for (int l = 0; l < k; l++) {
        if (!al16(y_levels[l])) { fail("cms_combine_gate_bf16x1_rocm: level %d is not 16-byte aligned.", l); return; }
        lv.y[l] = y_levels[l];
    }
    const float scale = k > 2 ? 1.0f / sqrtf((float)k) : 1.0f;
    KernelTimer kt("combine_gate_x1_kernel");
    hipLaunchKernelGGL(combine_gate_x1_kernel, dim3(stream_blocks(n / 4, 4096)), dim3(kSThr), 0, stream(), lv, k, scale, attn_out,
                       gate, gated_bf16, n / 4);
    check_launch("combine_gate_x1_kernel");
}

void linear_forward_bf16_rocm(const uint16_t *a_bf16, const float *w, float *out, int n, int d_in, int d_out) {
    const ErrorScope es;
    if (n <= 0 || d_in <= 0 || d_out <= 0 || (d_in * (long long)d_out) % 4) {
        fail("linear_forward_bf16_rocm: invalid dims n=%d d_in=%d d_out=%d (d_in * d_out must be a multiple of 4).", n, d_in, d_out);
        return;
    }
    u16 *wb = reinterpret_cast<u16 *>(scratch(27, (size_t)d_in * d_out * sizeof(u16)));
    if (es.failed()) return;
    to_bf16(w, wb, (long long)d_in * d_out);
    // out [n, d_out] = a [n, d_in] W^T
    gemm_bf16("gemm linear", rocblas_operation_transpose, rocblas_operation_none, d_out, n, d_in, wb, d_in, a_bf16, d_in, 0.f, out,
              d_out);
}

void linear_backward_bf16_rocm(const float *d_out_f32, const uint16_t *a_bf16, const float *w, float *d_a, float *d_w, int n,
                               int d_in, int d_out) {
    const ErrorScope es;
    if (n <= 0 || d_in <= 0 || d_out <= 0 || (d_in * (long long)d_out) % 4 || ((long long)n * d_out) % 4) {
        fail("linear_backward_bf16_rocm: invalid dims n=%d d_in=%d d_out=%d (products must be multiples of 4).", n, d_in, d_out);
        return;
    }
    u16 *wb = reinterpret_cast<u16 *>(scratch(27, (size_t)d_in * d_out * sizeof(u16)));
    u16 *gb = reinterpret_cast<u16 *>(scratch(26, (size_t)n * d_out * sizeof(u16)));
    if (es.failed()) return;
    to_bf16(w, wb, (long long)d_in * d_out);
    to_bf16(d_out_f32, gb, (long long)n * d_out);
    // d_a [n, d_in] = g [n, d_out] W [d_out, d_in];  d_W [d_out, d_in] = g^T a
    if (d_a && !gemm_bf16("gemm linear d_a", rocblas_operation_none, rocblas_operation_none, d_in, n, d_out, wb, d_in, gb, d_out,
                          0.f, d_a, d_in))
        return;
    if (d_w) gemm_weight_grad("gemm linear d_w", d_in, d_out, n, a_bf16, d_in, gb, d_out, d_w);
}

}  // extern "C"
