// Sliding-window attention on the bf16 matrix cores for head sizes 64 and 32, no
// persistent prefix, window <= 512 (the production shapes).  Contract and mask
// are those of core/kernels/swa_forward.cu / swa_backward.cu; other shapes stay
// on the wave-per-query kernels of swa.hip.
//
// All products are v_mfma_f32_16x16x32_bf16 steps (a 16x16x16 step costs the same
// cycles for half the work), so every operand is 8 consecutive contraction
// elements per lane: lane (r = l % 16, g = l / 16) supplies row r, contraction
// elements 8 g .. 8 g + 7 of a 32-wide step.
//
// Every kernel works in blocks: one workgroup per 128 queries (keys in the key passes), one wave per 32, stages
// of 64 keys (queries) whose rows are staged in LDS exactly as they arrive.  A 16x16 result tile leaves rows
// 4 g + i in a lane; where two such tiles become an operand again with their rows as contraction index (the
// weights in O^T = V^T w^T, dS in d_q^T = K^T dS^T, ..), the matching operand is read from the row-major stage
// through ds_read_b64_tr_b16 with group g taking rows 32 hf + 4 g .. + 3 and 32 hf + 16 + 4 g .. + 3 — the rows
// the two tiles left in that group's lanes — so no stage is ever written transposed or in a permuted order.
// No kernel holds more than one stage of scores: the forward keeps a running maximum (two sweeps where the
// contract wants the normalised weights stored), the query passes accumulate A = sum (w dW) k, B = sum w k and
// D = sum w dW in one sweep and finish with d_q = (A - D B) / sqrt(hd).
//   contract (weights stored / read back):  swa_fwd_blocked_kernel, swa_bwd_q_blocked_kernel, swa_bwd_k_blocked_kernel
//   two statistics per query instead:       swa_fwd_stats_kernel,   swa_bwd_q_stats_kernel,   swa_bwd_k_stats_kernel
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>

#include "lane_ops.h"
#include "runtime.h"
#include "swa_mfma.h"

namespace nlh {
namespace {

typedef __bf16 bh8 __attribute__((ext_vector_type(8)));
typedef __bf16 bh2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// The kernels are templates on the head size HDV (64 or 32): NKS = HDV / 32 contraction steps over the dims, NDT = HDV / 16
// output tiles of dims; the LDS stages keep 64-wide rows either way.
constexpr int KS = 64;        // keys per LDS stage
constexpr int LDH = 72;       // LDS row stride in bf16 elements (144 B: 16-byte rows, conflict-free operand reads)

__device__ __forceinline__ f32x4 mfma32(uint4 a, uint4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bh8, a), __builtin_bit_cast(bh8, b), c, 0, 0, 0);
}
// two floats -> two bf16 (round to nearest even) in one dword, x in the low half
__device__ __forceinline__ unsigned pack2(float x, float y) {
    const bh2 p = {(__bf16)x, (__bf16)y};
    return __builtin_bit_cast(unsigned, p);
}
__device__ __forceinline__ float bf_lo(unsigned w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf_hi(unsigned w) { return __uint_as_float(w & 0xffff0000u); }
// x, y = hi + lo with hi, lo bf16: the pair carries 16 mantissa bits through a bf16 product
__device__ __forceinline__ void split2(float x, float y, unsigned &hi, unsigned &lo) {
    hi = pack2(x, y);
    lo = pack2(x - bf_lo(hi), y - bf_hi(hi));
}
__device__ __forceinline__ void split8(f32x4 a, f32x4 b, uint4 &hi, uint4 &lo) {
    split2(a[0], a[1], hi.x, lo.x);
    split2(a[2], a[3], hi.y, lo.y);
    split2(b[0], b[1], hi.z, lo.z);
    split2(b[2], b[3], hi.w, lo.w);
}
// Workgroup -> (block of the sequence, head * batch) with all blocks of one head on one XCD.
// Workgroups go to the 8 XCDs round robin in linear order, and each XCD has its own L2; blocks
// of one head share K and V rows, so they are given linear ids that are equal modulo 8.
struct BlockCoord { int x, h, b; };
__device__ __forceinline__ BlockCoord xcd_block_coord(int H) {
    const int gx = gridDim.x, heads = gridDim.y * gridDim.z;
    const int lin = blockIdx.x + gx * (blockIdx.y + gridDim.y * blockIdx.z);
    int x = blockIdx.x, bh = blockIdx.y + gridDim.y * blockIdx.z;
    if ((heads & 7) == 0) {
        const int xcd = lin & 7, slot = lin >> 3;
        bh = (slot / gx) * 8 + xcd;
        x = slot % gx;
    }
    return BlockCoord{x, bh % H, bh / H};
}

// Cooperative load of one stage (64 rows of 64 bf16 = 512 chunks of 16 B, two per thread of a
// 256-thread block): chunk = (row, 8 dims), consecutive lanes along a row.
struct StageSrc { const unsigned short *p; size_t row0; int total, hoff, s; };
// OUT16 instantiations of the backward passes: the gradients leave as bf16 into columns of a wider row-major matrix
// (row stride ld elements, the head's dims at the same column offset as in q, k, v), written, not accumulated.
struct Out16 { unsigned short *q, *k, *v; long long ld; };
template <int HDV>
__device__ __forceinline__ void load_rows(const StageSrc &m, int first, uint4 (&regs)[2]) {
    const int tid = threadIdx.x;
#pragma unroll
    for (int c = 0; c < 2; c++) {
        const int chunk = tid + 256 * c, row = first + (chunk >> 3);
        regs[c] = make_uint4(0, 0, 0, 0);
        if (row >= 0 && row < m.s && 8 * (chunk & 7) < HDV)
            regs[c] = *reinterpret_cast<const uint4 *>(m.p + (m.row0 + row) * m.total + m.hoff + 8 * (chunk & 7));
    }
}
// operand of a 32-wide step: row r of the tile at row0, contraction elements 32 ks + 8 g .. + 7
__device__ __forceinline__ uint4 ld_op(unsigned short (*T)[LDH], int row0, int ks) {
    const int l = threadIdx.x & 63;
    return *reinterpret_cast<const uint4 *>(&T[row0 + (l & 15)][32 * ks + 8 * (l >> 4)]);
}

// Forward that keeps statistics instead of weights, in blocks of keys with a running maximum (no score
// outlives its 64-key stage, so a lane holds 32 scores instead of 144 and four workgroups fit a compute unit
// instead of two).  One workgroup per (128 queries, head, batch), one wave per 32 queries; per stage a wave
// forms S^T = K Q^T for its two query tiles (32 matrix-core steps with the products of the second half, against
// 8 per barrier in the kernel above), rescales O^T by exp2(old maximum - new maximum) and adds V^T P^T with the
// unnormalised weights; the division by the sum happens once at the end.  K and V rows are staged as they
// arrive; V^T is read through ds_read_b64_tr_b16: group g of a wave takes keys 32 hf + 4 g .. + 3 and
// 32 hf + 16 + 4 g .. + 3, which are exactly the rows that the two score tiles of that half leave in its lanes.
constexpr int FQ = 128;    // queries per workgroup
constexpr int LDV = 80;    // row stride of the V stage (160 B: the transposing reads of a group fall on 32 banks)

template <int LD>
__device__ __forceinline__ uint4 ld_tr2(const unsigned short (*T)[LD], int row_a, int row_b, int col0) {
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) s16x4 *lds_ptr;
    const int sl = threadIdx.x & 15;
    const s16x4 a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)&T[row_a + (sl >> 2)][col0 + 4 * (sl & 3)]);
    const s16x4 b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)&T[row_b + (sl >> 2)][col0 + 4 * (sl & 3)]);
    const uint2 ua = __builtin_bit_cast(uint2, a), ub = __builtin_bit_cast(uint2, b);
    return make_uint4(ua.x, ua.y, ub.x, ub.y);
}

template <int HDV>
__global__ __launch_bounds__(256, 3) void swa_fwd_stats_kernel(const unsigned short *__restrict__ q,
                                                            const unsigned short *__restrict__ k,
                                                            const unsigned short *__restrict__ v,
                                                            unsigned short *__restrict__ out,
                                                            float2 *__restrict__ stats, int s, int H, int ws) {
    __shared__ __align__(16) unsigned short Ks[2][KS][LDH];   // K stage [key][dim]
    __shared__ __align__(16) unsigned short Vs[2][KS][LDV];   // V stage [key][dim]
    const int tid = threadIdx.x, wave = tid >> 6, l = tid & 63, r = l & 15, g = l >> 4;
    const BlockCoord bc = xcd_block_coord(H);
    const int t0 = bc.x * FQ, h = bc.h, b = bc.b;
    constexpr int NKS = HDV / 32, NDT = HDV / 16;
    constexpr float kInvSqrt = HDV == 64 ? 0.125f : 0.17677669529663687f;   // 1 / sqrt(head size)
    const int total = H * HDV, hoff = h * HDV;
    const size_t row0 = (size_t)b * s;
    const int qlo = t0 + 32 * wave, qhi = qlo + 31;           // this wave's queries
    const int st_lo = max(t0 + 1 - ws, 0) / KS, st_hi = min(t0 + FQ - 1, s - 1) / KS;
    const StageSrc km{k, row0, total, hoff, s}, vm{v, row0, total, hoff, s};

    uint4 qf[2][2];   // B operand: query qlo + 16 qt + r, dims 32 ks + 8 g ..
#pragma unroll
    for (int qt = 0; qt < 2; qt++)
#pragma unroll
        for (int ks = 0; ks < NKS; ks++) {
            const int tq = qlo + 16 * qt + r;
            qf[qt][ks] = make_uint4(0, 0, 0, 0);
            if (tq < s) qf[qt][ks] = *reinterpret_cast<const uint4 *>(q + (row0 + tq) * total + hoff + 32 * ks + 8 * g);
        }
    f32x4 o[2][4];
#pragma unroll
    for (int qt = 0; qt < 2; qt++)
#pragma unroll
        for (int dt = 0; dt < NDT; dt++) o[qt][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    float mrun[2] = {-INFINITY, -INFINITY}, lsum[2] = {0.f, 0.f};   // running maximum (exp2 units), this lane's share of the sum
    const float c2 = kInvSqrt * 1.44269504088896340736f;   // log2(e) / sqrt(head size)

    uint4 kreg[2], vreg[2];
    load_rows<HDV>(km, KS * st_lo, kreg);
    load_rows<HDV>(vm, KS * st_lo, vreg);
    for (int st = st_lo; st <= st_hi; st++) {
        const int buf = (st - st_lo) & 1, k0 = KS * st;
#pragma unroll
        for (int c = 0; c < 2; c++) {
            const int chunk = tid + 256 * c;
            *reinterpret_cast<uint4 *>(&Ks[buf][chunk >> 3][8 * (chunk & 7)]) = kreg[c];
            *reinterpret_cast<uint4 *>(&Vs[buf][chunk >> 3][8 * (chunk & 7)]) = vreg[c];
        }
        __syncthreads();   // also: every wave is done with the stage before the previous one, whose buffer comes next
        if (st < st_hi) {
            load_rows<HDV>(km, k0 + KS, kreg);
            load_rows<HDV>(vm, k0 + KS, vreg);
        }
        if (k0 > qhi || k0 + KS - 1 < qlo + 1 - ws) continue;   // no key of this stage is seen by this wave's queries
        f32x4 sc[4][2];
#pragma unroll
        for (int kt = 0; kt < 4; kt++) {
            const uint4 a0 = ld_op(Ks[buf], 16 * kt, 0), a1 = ld_op(Ks[buf], 16 * kt, 1);
#pragma unroll
            for (int qt = 0; qt < 2; qt++) {
                sc[kt][qt] = mfma32(a0, qf[qt][0], f32x4{0.f, 0.f, 0.f, 0.f});
                if constexpr (NKS == 2) sc[kt][qt] = mfma32(a1, qf[qt][1], sc[kt][qt]);
            }
        }
        const bool full = k0 + KS - 1 <= qlo && k0 >= qhi + 1 - ws && qhi < s;   // wave-uniform: nothing to mask
        if (!full) {
#pragma unroll
            for (int kt = 0; kt < 4; kt++)
#pragma unroll
                for (int qt = 0; qt < 2; qt++)
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const int key = k0 + 16 * kt + 4 * g + i, tq = qlo + 16 * qt + r;
                        const bool ok = key <= tq && key >= tq + 1 - ws && tq < s;
                        sc[kt][qt][i] = ok ? sc[kt][qt][i] : -INFINITY;
                    }
        }
#pragma unroll
        for (int qt = 0; qt < 2; qt++) {
            float mx = -INFINITY;
#pragma unroll
            for (int kt = 0; kt < 4; kt++)
#pragma unroll
                for (int i = 0; i < 4; i++) mx = fmaxf(mx, sc[kt][qt][i]);
            mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            const float mnew = fmaxf(mrun[qt], mx * c2);
            const float mref = mnew == -INFINITY ? 0.f : mnew;
            const float alpha = __builtin_amdgcn_exp2f(mrun[qt] - mref);
            mrun[qt] = mnew;
            float part = 0.f;
#pragma unroll
            for (int kt = 0; kt < 4; kt++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float e = __builtin_amdgcn_exp2f(fmaf(sc[kt][qt][i], c2, -mref));
                    sc[kt][qt][i] = e;
                    part += e;
                }
            lsum[qt] = fmaf(lsum[qt], alpha, part);
#pragma unroll
            for (int dt = 0; dt < NDT; dt++) o[qt][dt] = o[qt][dt] * alpha;
        }
#pragma unroll
        for (int hf = 0; hf < 2; hf++) {
            uint4 pb[2];
#pragma unroll
            for (int qt = 0; qt < 2; qt++) {
                const f32x4 p0 = sc[2 * hf][qt], p1 = sc[2 * hf + 1][qt];
                pb[qt] = make_uint4(pack2(p0[0], p0[1]), pack2(p0[2], p0[3]), pack2(p1[0], p1[1]), pack2(p1[2], p1[3]));
            }
#pragma unroll
            for (int dt = 0; dt < NDT; dt++) {
                const uint4 av = ld_tr2<LDV>(Vs[buf], 32 * hf + 4 * g, 32 * hf + 16 + 4 * g, 16 * dt);
#pragma unroll
                for (int qt = 0; qt < 2; qt++) o[qt][dt] = mfma32(av, pb[qt], o[qt][dt]);
            }
        }
    }
#pragma unroll
    for (int qt = 0; qt < 2; qt++) {
        const int tq = qlo + 16 * qt + r;
        float sum = lsum[qt];
        sum += __shfl_xor(sum, 16, 64);
        sum += __shfl_xor(sum, 32, 64);
        const float inv = sum > 0.f ? 1.0f / sum : 0.f;
        if (tq < s) {
            if (g == 0) stats[(size_t)(b * H + h) * s + tq] = make_float2(mrun[qt] == -INFINITY ? 0.f : mrun[qt], inv);
            unsigned short *ob = out + (row0 + tq) * total + hoff;
#pragma unroll
            for (int dt = 0; dt < NDT; dt++)
                *reinterpret_cast<uint2 *>(ob + 16 * dt + 4 * g) =
                    make_uint2(pack2(o[qt][dt][0] * inv, o[qt][dt][1] * inv), pack2(o[qt][dt][2] * inv, o[qt][dt][3] * inv));
        }
    }
}

// Forward of the contract (normalised weights stored) in the same blocks: the weights need the final maximum
// and sum, so the window is swept twice — scores and running statistics first, then scores again, the weights
// w = bf16(exp2(s c - m) / sum) to their slot rows (four consecutive slots per lane and tile: 8-byte stores at
// 2-byte alignment) and O^T += V^T w^T.  Slots behind an early query's own key (t < window - 1) are zeroed at
// the end.
template <int HDV>
__global__ __launch_bounds__(256, 3) void swa_fwd_blocked_kernel(const unsigned short *__restrict__ q,
                                                              const unsigned short *__restrict__ k,
                                                              const unsigned short *__restrict__ v,
                                                              unsigned short *__restrict__ out,
                                                              unsigned short *__restrict__ attn_w, int s, int H,
                                                              int ws) {
    __shared__ __align__(16) unsigned short Ks[2][KS][LDH];   // K stage [key][dim]
    __shared__ __align__(16) unsigned short Vs[2][KS][LDV];   // V stage [key][dim]
    const int tid = threadIdx.x, wave = tid >> 6, l = tid & 63, r = l & 15, g = l >> 4;
    const BlockCoord bc = xcd_block_coord(H);
    const int t0 = bc.x * FQ, h = bc.h, b = bc.b;
    constexpr int NKS = HDV / 32, NDT = HDV / 16;
    constexpr float kInvSqrt = HDV == 64 ? 0.125f : 0.17677669529663687f;   // 1 / sqrt(head size)
    const int total = H * HDV, hoff = h * HDV;
    const size_t row0 = (size_t)b * s;
    const int qlo = t0 + 32 * wave, qhi = qlo + 31;
    const int st_lo = max(t0 + 1 - ws, 0) / KS, st_hi = min(t0 + FQ - 1, s - 1) / KS;
    const StageSrc km{k, row0, total, hoff, s}, vm{v, row0, total, hoff, s};
    const float c2 = kInvSqrt * 1.44269504088896340736f;

    uint4 qf[2][2];
#pragma unroll
    for (int qt = 0; qt < 2; qt++)
#pragma unroll
        for (int ks = 0; ks < NKS; ks++) {
            const int tq = qlo + 16 * qt + r;
            qf[qt][ks] = make_uint4(0, 0, 0, 0);
            if (tq < s) qf[qt][ks] = *reinterpret_cast<const uint4 *>(q + (row0 + tq) * total + hoff + 32 * ks + 8 * g);
        }
    // scores of one stage for this wave's two query tiles, masked keys at -inf
    auto scores = [&](int buf, int k0, f32x4 (&sc)[4][2]) {
#pragma unroll
        for (int kt = 0; kt < 4; kt++) {
            const uint4 a0 = ld_op(Ks[buf], 16 * kt, 0), a1 = ld_op(Ks[buf], 16 * kt, 1);
#pragma unroll
            for (int qt = 0; qt < 2; qt++) {
                sc[kt][qt] = mfma32(a0, qf[qt][0], f32x4{0.f, 0.f, 0.f, 0.f});
                if constexpr (NKS == 2) sc[kt][qt] = mfma32(a1, qf[qt][1], sc[kt][qt]);
            }
        }
        const bool full = k0 + KS - 1 <= qlo && k0 >= qhi + 1 - ws && qhi < s;
        if (!full) {
#pragma unroll
            for (int kt = 0; kt < 4; kt++)
#pragma unroll
                for (int qt = 0; qt < 2; qt++)
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const int key = k0 + 16 * kt + 4 * g + i, tq = qlo + 16 * qt + r;
                        const bool ok = key <= tq && key >= tq + 1 - ws && tq < s;
                        sc[kt][qt][i] = ok ? sc[kt][qt][i] : -INFINITY;
                    }
        }
    };

    // ---- sweep 1: running maximum and sum ----
    float mrun[2] = {-INFINITY, -INFINITY}, lsum[2] = {0.f, 0.f};
    uint4 kreg[2], vreg[2];
    load_rows<HDV>(km, KS * st_lo, kreg);
    for (int st = st_lo; st <= st_hi; st++) {
        const int buf = (st - st_lo) & 1, k0 = KS * st;
#pragma unroll
        for (int c = 0; c < 2; c++) {
            const int chunk = tid + 256 * c;
            *reinterpret_cast<uint4 *>(&Ks[buf][chunk >> 3][8 * (chunk & 7)]) = kreg[c];
        }
        __syncthreads();
        if (st < st_hi) load_rows<HDV>(km, k0 + KS, kreg);
        if (k0 > qhi || k0 + KS - 1 < qlo + 1 - ws) continue;
        f32x4 sc[4][2];
        scores(buf, k0, sc);
#pragma unroll
        for (int qt = 0; qt < 2; qt++) {
            float mx = -INFINITY;
#pragma unroll
            for (int kt = 0; kt < 4; kt++)
#pragma unroll
                for (int i = 0; i < 4; i++) mx = fmaxf(mx, sc[kt][qt][i]);
            mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            const float mnew = fmaxf(mrun[qt], mx * c2);
            const float mref = mnew == -INFINITY ? 0.f : mnew;
            const float alpha = __builtin_amdgcn_exp2f(mrun[qt] - mref);
            mrun[qt] = mnew;
            float part = 0.f;
#pragma unroll
            for (int kt = 0; kt < 4; kt++)
#pragma unroll
                for (int i = 0; i < 4; i++) part += __builtin_amdgcn_exp2f(fmaf(sc[kt][qt][i], c2, -mref));
            lsum[qt] = fmaf(lsum[qt], alpha, part);
        }
    }
    float mc[2], inv[2];
#pragma unroll
    for (int qt = 0; qt < 2; qt++) {
        float sum = lsum[qt];
        sum += __shfl_xor(sum, 16, 64);
        sum += __shfl_xor(sum, 32, 64);
        inv[qt] = sum > 0.f ? 1.0f / sum : 0.f;
        mc[qt] = mrun[qt] == -INFINITY ? 0.f : mrun[qt];
    }

    // ---- sweep 2: weights out, O^T = V^T w^T ----
    f32x4 o[2][4];
#pragma unroll
    for (int qt = 0; qt < 2; qt++)
#pragma unroll
        for (int dt = 0; dt < NDT; dt++) o[qt][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    unsigned short *wrow[2];
    int lsq[2];
#pragma unroll
    for (int qt = 0; qt < 2; qt++) {
        const int tq = qlo + 16 * qt + r;
        lsq[qt] = max(tq + 1 - ws, 0);
        wrow[qt] = attn_w + ((size_t)(b * H + h) * s + min(tq, s - 1)) * ws;
    }
    __syncthreads();   // every wave is done with the buffers of sweep 1
    load_rows<HDV>(km, KS * st_lo, kreg);
    load_rows<HDV>(vm, KS * st_lo, vreg);
    for (int st = st_lo; st <= st_hi; st++) {
        const int buf = (st - st_lo) & 1, k0 = KS * st;
#pragma unroll
        for (int c = 0; c < 2; c++) {
            const int chunk = tid + 256 * c;
            *reinterpret_cast<uint4 *>(&Ks[buf][chunk >> 3][8 * (chunk & 7)]) = kreg[c];
            *reinterpret_cast<uint4 *>(&Vs[buf][chunk >> 3][8 * (chunk & 7)]) = vreg[c];
        }
        __syncthreads();
        if (st < st_hi) {
            load_rows<HDV>(km, k0 + KS, kreg);
            load_rows<HDV>(vm, k0 + KS, vreg);
        }
        if (k0 > qhi || k0 + KS - 1 < qlo + 1 - ws) continue;
        f32x4 sc[4][2];
        scores(buf, k0, sc);
#pragma unroll
        for (int hf = 0; hf < 2; hf++) {
            uint4 pb[2];
#pragma unroll
            for (int qt = 0; qt < 2; qt++) {
                const int tq = qlo + 16 * qt + r;
                unsigned wp[2][2];
#pragma unroll
                for (int c = 0; c < 2; c++) {
                    const f32x4 x = sc[2 * hf + c][qt];
                    float w[4];
#pragma unroll
                    for (int i = 0; i < 4; i++) w[i] = __builtin_amdgcn_exp2f(fmaf(x[i], c2, -mc[qt])) * inv[qt];
                    wp[c][0] = pack2(w[0], w[1]);
                    wp[c][1] = pack2(w[2], w[3]);
                    // keys key0 .. key0 + 3 of query tq sit in slots key0 - lsq ..; only keys of the window have one
                    const int key0 = k0 + 16 * (2 * hf + c) + 4 * g;
                    if (tq < s) {
                        if (key0 >= lsq[qt] && key0 + 3 <= tq) {
                            const uint2 pr = make_uint2(wp[c][0], wp[c][1]);
                            __builtin_memcpy(wrow[qt] + (key0 - lsq[qt]), &pr, 8);
                        } else if (key0 + 3 >= lsq[qt] && key0 <= tq) {
#pragma unroll
                            for (int i = 0; i < 4; i++)
                                if (key0 + i >= lsq[qt] && key0 + i <= tq)
                                    wrow[qt][key0 + i - lsq[qt]] = (unsigned short)(wp[c][i >> 1] >> (16 * (i & 1)));
                        }
                    }
                }
                pb[qt] = make_uint4(wp[0][0], wp[0][1], wp[1][0], wp[1][1]);
            }
#pragma unroll
            for (int dt = 0; dt < NDT; dt++) {
                const uint4 av = ld_tr2<LDV>(Vs[buf], 32 * hf + 4 * g, 32 * hf + 16 + 4 * g, 16 * dt);
#pragma unroll
                for (int qt = 0; qt < 2; qt++) o[qt][dt] = mfma32(av, pb[qt], o[qt][dt]);
            }
        }
    }
    // early queries: the slots behind the query's own key hold zeros
    if (qlo < ws - 1) {
        unsigned short *awb = attn_w + ((size_t)(b * H + h) * s) * ws;
        for (int qi = 0; qi < 32; qi++) {
            const int tt = qlo + qi;
            if (tt >= s || tt >= ws - 1) break;
            for (int slot = tt + 1 + l; slot < ws; slot += 64) awb[(size_t)tt * ws + slot] = 0;
        }
    }
#pragma unroll
    for (int qt = 0; qt < 2; qt++) {
        const int tq = qlo + 16 * qt + r;
        if (tq < s) {
            unsigned short *ob = out + (row0 + tq) * total + hoff;
#pragma unroll
            for (int dt = 0; dt < NDT; dt++)
                *reinterpret_cast<uint2 *>(ob + 16 * dt + 4 * g) =
                    make_uint2(pack2(o[qt][dt][0], o[qt][dt][1]), pack2(o[qt][dt][2], o[qt][dt][3]));
        }
    }
}

// Query pass on statistics, in key blocks like swa_fwd_stats_kernel (one workgroup per 128 queries, one wave per
// 32), in ONE sweep over the window.  dS = w (dW - D) needs D_t = sum_j w dW of the whole window, so the sweep
// accumulates the two sums that do not:  A^T = K^T (w dW)^T and B^T = K^T w^T, and D itself, and ends with
//   d_q = (A - D B) / sqrt(hd)
// (the same numbers as sum_j dS k_j; no sweep that rebuilds O first, and D as exact as before — taking D from
// the forward's bf16 output instead moves it by 2^-9 and, where the window holds few keys, d_q by 5e-3).
// Per stage a wave forms S^T = K Q^T, the weights w = bf16(exp2(s c - m) / sum) as the weight tensor would hold
// them, dW^T = V dO^T; dO and w dW enter as hi + lo pairs, w is exact in bf16.  K^T is read from the K rows
// through ds_read_b64_tr_b16 in the key order that the score tiles leave in the lanes.  D goes to dvec.
template <int HDV, bool OUT16>
__global__ __launch_bounds__(256, 2) void swa_bwd_q_stats_kernel(const unsigned short *__restrict__ q,
                                                                 const unsigned short *__restrict__ k,
                                                                 const unsigned short *__restrict__ v,
                                                                 const float2 *__restrict__ stats,
                                                                 const float *__restrict__ d_out,
                                                                 float *__restrict__ d_q, float *__restrict__ dvec,
                                                                 int s, int H, int ws, Out16 o16) {
    __shared__ __align__(16) unsigned short Ks[2][KS][LDH], Vs[2][KS][LDH];   // stages [key][dim]
    const int tid = threadIdx.x, wave = tid >> 6, l = tid & 63, r = l & 15, g = l >> 4;
    const BlockCoord bc = xcd_block_coord(H);
    const int t0 = bc.x * FQ, h = bc.h, b = bc.b;
    constexpr int NKS = HDV / 32, NDT = HDV / 16;
    constexpr float kInvSqrt = HDV == 64 ? 0.125f : 0.17677669529663687f;   // 1 / sqrt(head size)
    const int total = H * HDV, hoff = h * HDV;
    const size_t row0 = (size_t)b * s;
    const int qlo = t0 + 32 * wave, qhi = qlo + 31;
    const int st_lo = max(t0 + 1 - ws, 0) / KS, st_hi = min(t0 + FQ - 1, s - 1) / KS;
    const StageSrc km{k, row0, total, hoff, s}, vm{v, row0, total, hoff, s};
    const float c2 = kInvSqrt * 1.44269504088896340736f, scale = kInvSqrt;

    uint4 qf[2][2], doh[2][2], dol[2][2];
    float mc[2], inv[2], dpart[2] = {0.f, 0.f};
#pragma unroll
    for (int qt = 0; qt < 2; qt++) {
        const int tq = qlo + 16 * qt + r;
        mc[qt] = 0.f; inv[qt] = 0.f;
#pragma unroll
        for (int ks = 0; ks < NKS; ks++) {
            qf[qt][ks] = make_uint4(0, 0, 0, 0);
            f32x4 x0 = f32x4{0.f, 0.f, 0.f, 0.f}, x1 = x0;
            if (tq < s) {
                const size_t o = (row0 + tq) * total + hoff + 32 * ks + 8 * g;
                qf[qt][ks] = *reinterpret_cast<const uint4 *>(q + o);
                x0 = *reinterpret_cast<const f32x4 *>(d_out + o);
                x1 = *reinterpret_cast<const f32x4 *>(d_out + o + 4);
            }
            split8(x0, x1, doh[qt][ks], dol[qt][ks]);
        }
        if (tq < s) {
            const float2 st2 = stats[(size_t)(b * H + h) * s + tq];
            mc[qt] = st2.x;
            inv[qt] = st2.y;
        }
    }
    f32x4 aq[2][4], bq[2][4];
#pragma unroll
    for (int qt = 0; qt < 2; qt++)
#pragma unroll
        for (int dt = 0; dt < NDT; dt++) { aq[qt][dt] = f32x4{0.f, 0.f, 0.f, 0.f}; bq[qt][dt] = f32x4{0.f, 0.f, 0.f, 0.f}; }

    uint4 kreg[2], vreg[2];
    load_rows<HDV>(km, KS * st_lo, kreg);
    load_rows<HDV>(vm, KS * st_lo, vreg);
    for (int st = st_lo; st <= st_hi; st++) {
        const int buf = (st - st_lo) & 1, k0 = KS * st;
#pragma unroll
        for (int c = 0; c < 2; c++) {
            const int chunk = tid + 256 * c;
            *reinterpret_cast<uint4 *>(&Ks[buf][chunk >> 3][8 * (chunk & 7)]) = kreg[c];
            *reinterpret_cast<uint4 *>(&Vs[buf][chunk >> 3][8 * (chunk & 7)]) = vreg[c];
        }
        __syncthreads();
        if (st < st_hi) {
            load_rows<HDV>(km, k0 + KS, kreg);
            load_rows<HDV>(vm, k0 + KS, vreg);
        }
        if (k0 > qhi || k0 + KS - 1 < qlo + 1 - ws) continue;
        const bool full = k0 + KS - 1 <= qlo && k0 >= qhi + 1 - ws && qhi < s;
#pragma unroll
        for (int hf = 0; hf < 2; hf++) {
            uint4 xh[2], xl[2], wb[2];
#pragma unroll
            for (int qt = 0; qt < 2; qt++) {
                f32x4 x[2];
                unsigned wp[2][2];
#pragma unroll
                for (int c = 0; c < 2; c++) {
                    const int kt = 2 * hf + c;
                    const uint4 ak0 = ld_op(Ks[buf], 16 * kt, 0), ak1 = ld_op(Ks[buf], 16 * kt, 1);
                    const uint4 av0 = ld_op(Vs[buf], 16 * kt, 0), av1 = ld_op(Vs[buf], 16 * kt, 1);
                    f32x4 sc = mfma32(ak0, qf[qt][0], f32x4{0.f, 0.f, 0.f, 0.f});
                    if constexpr (NKS == 2) sc = mfma32(ak1, qf[qt][1], sc);
                    f32x4 dw = mfma32(av0, doh[qt][0], f32x4{0.f, 0.f, 0.f, 0.f});
                    dw = mfma32(av0, dol[qt][0], dw);
                    if constexpr (NKS == 2) dw = mfma32(av1, doh[qt][1], dw);
                    if constexpr (NKS == 2) dw = mfma32(av1, dol[qt][1], dw);
                    f32x4 w;
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const int key = k0 + 16 * kt + 4 * g + i, tq = qlo + 16 * qt + r;
                        const bool ok = full || (key <= tq && key >= tq + 1 - ws && tq < s);
                        w[i] = ok ? __builtin_amdgcn_exp2f(fmaf(sc[i], c2, -mc[qt])) * inv[qt] : 0.f;
                    }
                    wp[c][0] = pack2(w[0], w[1]);   // as the weight tensor holds them
                    wp[c][1] = pack2(w[2], w[3]);
                    x[c][0] = bf_lo(wp[c][0]) * dw[0];
                    x[c][1] = bf_hi(wp[c][0]) * dw[1];
                    x[c][2] = bf_lo(wp[c][1]) * dw[2];
                    x[c][3] = bf_hi(wp[c][1]) * dw[3];
                    dpart[qt] += (x[c][0] + x[c][1]) + (x[c][2] + x[c][3]);
                }
                split8(x[0], x[1], xh[qt], xl[qt]);
                wb[qt] = make_uint4(wp[0][0], wp[0][1], wp[1][0], wp[1][1]);
            }
#pragma unroll
            for (int dt = 0; dt < NDT; dt++) {
                const uint4 a = ld_tr2<LDH>(Ks[buf], 32 * hf + 4 * g, 32 * hf + 16 + 4 * g, 16 * dt);
#pragma unroll
                for (int qt = 0; qt < 2; qt++) {
                    aq[qt][dt] = mfma32(a, xh[qt], aq[qt][dt]);
                    aq[qt][dt] = mfma32(a, xl[qt], aq[qt][dt]);
                    bq[qt][dt] = mfma32(a, wb[qt], bq[qt][dt]);
                }
            }
        }
    }
#pragma unroll
    for (int qt = 0; qt < 2; qt++) {
        const int tq = qlo + 16 * qt + r;
        float dsum = dpart[qt];
        dsum += __shfl_xor(dsum, 16, 64);
        dsum += __shfl_xor(dsum, 32, 64);
        if (tq < s) {
            if (g == 0) dvec[(size_t)(b * H + h) * s + tq] = dsum;
            if (OUT16) {
                unsigned short *ob = o16.q + (row0 + tq) * o16.ld + hoff;
#pragma unroll
                for (int dt = 0; dt < NDT; dt++) {
                    const f32x4 x = (aq[qt][dt] - dsum * bq[qt][dt]) * scale;
                    *reinterpret_cast<uint2 *>(ob + 16 * dt + 4 * g) = make_uint2(pack2(x[0], x[1]), pack2(x[2], x[3]));
                }
            } else {
                float *ob = d_q + (row0 + tq) * total + hoff;
#pragma unroll
                for (int dt = 0; dt < NDT; dt++)
                    *reinterpret_cast<f32x4 *>(ob + 16 * dt + 4 * g) = (aq[qt][dt] - dsum * bq[qt][dt]) * scale;
            }
        }
    }
}

// Query pass of the contract (weights read back from the tensor) in the same blocks and the same single sweep as
// swa_bwd_q_stats_kernel: A = sum_j (w dW) k_j, B = sum_j w k_j and D = sum_j w dW together, d_q = (A - D B)/sqrt(hd).
// A lane's four keys of a tile are four consecutive slots of its query's row: one 8-byte load (2-byte aligned),
// requested a stage ahead; only the stages at the two ends of the window go slot by slot.
template <int HDV>
__global__ __launch_bounds__(256, 2) void swa_bwd_q_blocked_kernel(const unsigned short *__restrict__ k,
                                                                   const unsigned short *__restrict__ v,
                                                                   const unsigned short *__restrict__ attn_w,
                                                                   const float *__restrict__ d_out,
                                                                   float *__restrict__ d_q, float *__restrict__ dvec,
                                                                   int s, int H, int ws) {
    __shared__ __align__(16) unsigned short Ks[2][KS][LDH], Vs[2][KS][LDH];   // stages [key][dim]
    const int tid = threadIdx.x, wave = tid >> 6, l = tid & 63, r = l & 15, g = l >> 4;
    const BlockCoord bc = xcd_block_coord(H);
    const int t0 = bc.x * FQ, h = bc.h, b = bc.b;
    constexpr int NKS = HDV / 32, NDT = HDV / 16;
    constexpr float kInvSqrt = HDV == 64 ? 0.125f : 0.17677669529663687f;   // 1 / sqrt(head size)
    const int total = H * HDV, hoff = h * HDV;
    const size_t row0 = (size_t)b * s;
    const int qlo = t0 + 32 * wave, qhi = qlo + 31;
    const int st_lo = max(t0 + 1 - ws, 0) / KS, st_hi = min(t0 + FQ - 1, s - 1) / KS;
    const StageSrc km{k, row0, total, hoff, s}, vm{v, row0, total, hoff, s};
    const float scale = kInvSqrt;

    uint4 doh[2][2], dol[2][2];
    const unsigned short *wrow[2];
    int lsq[2], tqs[2];
    float dpart[2] = {0.f, 0.f};
#pragma unroll
    for (int qt = 0; qt < 2; qt++) {
        const int tq = qlo + 16 * qt + r;
        tqs[qt] = tq < s ? tq : -1;   // -1: no key passes "key <= tq"
        lsq[qt] = max(tq + 1 - ws, 0);
        wrow[qt] = attn_w + ((size_t)(b * H + h) * s + min(tq, s - 1)) * ws;
#pragma unroll
        for (int ks = 0; ks < NKS; ks++) {
            f32x4 x0 = f32x4{0.f, 0.f, 0.f, 0.f}, x1 = x0;
            if (tq < s) {
                const size_t o = (row0 + tq) * total + hoff + 32 * ks + 8 * g;
                x0 = *reinterpret_cast<const f32x4 *>(d_out + o);
                x1 = *reinterpret_cast<const f32x4 *>(d_out + o + 4);
            }
            split8(x0, x1, doh[qt][ks], dol[qt][ks]);
        }
    }
    f32x4 aq[2][4], bq[2][4];
#pragma unroll
    for (int qt = 0; qt < 2; qt++)
#pragma unroll
        for (int dt = 0; dt < NDT; dt++) { aq[qt][dt] = f32x4{0.f, 0.f, 0.f, 0.f}; bq[qt][dt] = f32x4{0.f, 0.f, 0.f, 0.f}; }

    // weights of a stage for this lane: wreg[kt][qt] = keys k0 + 16 kt + 4 g .. + 3 of query qt, zero outside the window
    uint2 wreg[4][2];
    auto fetch_weights = [&](int k0) {
        const bool skip = k0 > qhi || k0 + KS - 1 < qlo + 1 - ws;
        const bool full = k0 + KS - 1 <= qlo && k0 >= qhi + 1 - ws && qhi < s;
#pragma unroll
        for (int kt = 0; kt < 4; kt++)
#pragma unroll
            for (int qt = 0; qt < 2; qt++) {
                const int key0 = k0 + 16 * kt + 4 * g;
                wreg[kt][qt] = make_uint2(0u, 0u);
                if (skip) continue;
                if (full || (key0 >= lsq[qt] && key0 + 3 <= tqs[qt])) {
                    __builtin_memcpy(&wreg[kt][qt], wrow[qt] + (key0 - lsq[qt]), 8);
                } else {
                    unsigned d[2] = {0u, 0u};
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const int key = key0 + e;
                        unsigned x = 0;
                        if (key >= lsq[qt] && key <= tqs[qt]) x = wrow[qt][key - lsq[qt]];
                        d[e >> 1] |= x << (16 * (e & 1));
                    }
                    wreg[kt][qt] = make_uint2(d[0], d[1]);
                }
            }
    };

    uint4 kreg[2], vreg[2];
    load_rows<HDV>(km, KS * st_lo, kreg);
    load_rows<HDV>(vm, KS * st_lo, vreg);
    fetch_weights(KS * st_lo);
    for (int st = st_lo; st <= st_hi; st++) {
        const int buf = (st - st_lo) & 1, k0 = KS * st;
#pragma unroll
        for (int c = 0; c < 2; c++) {
            const int chunk = tid + 256 * c;
            *reinterpret_cast<uint4 *>(&Ks[buf][chunk >> 3][8 * (chunk & 7)]) = kreg[c];
            *reinterpret_cast<uint4 *>(&Vs[buf][chunk >> 3][8 * (chunk & 7)]) = vreg[c];
        }
        uint2 wcur[4][2];
#pragma unroll
        for (int kt = 0; kt < 4; kt++)
#pragma unroll
            for (int qt = 0; qt < 2; qt++) wcur[kt][qt] = wreg[kt][qt];
        __syncthreads();
        if (st < st_hi) {
            load_rows<HDV>(km, k0 + KS, kreg);
            load_rows<HDV>(vm, k0 + KS, vreg);
            fetch_weights(k0 + KS);
        }
        if (k0 > qhi || k0 + KS - 1 < qlo + 1 - ws) continue;
#pragma unroll
        for (int hf = 0; hf < 2; hf++) {
            uint4 xh[2], xl[2], wb[2];
#pragma unroll
            for (int qt = 0; qt < 2; qt++) {
                f32x4 x[2];
#pragma unroll
                for (int c = 0; c < 2; c++) {
                    const int kt = 2 * hf + c;
                    const uint4 av0 = ld_op(Vs[buf], 16 * kt, 0), av1 = ld_op(Vs[buf], 16 * kt, 1);
                    f32x4 dw = mfma32(av0, doh[qt][0], f32x4{0.f, 0.f, 0.f, 0.f});
                    dw = mfma32(av0, dol[qt][0], dw);
                    if constexpr (NKS == 2) dw = mfma32(av1, doh[qt][1], dw);
                    if constexpr (NKS == 2) dw = mfma32(av1, dol[qt][1], dw);
                    const uint2 wp = wcur[kt][qt];
                    x[c][0] = bf_lo(wp.x) * dw[0];
                    x[c][1] = bf_hi(wp.x) * dw[1];
                    x[c][2] = bf_lo(wp.y) * dw[2];
                    x[c][3] = bf_hi(wp.y) * dw[3];
                    dpart[qt] += (x[c][0] + x[c][1]) + (x[c][2] + x[c][3]);
                }
                split8(x[0], x[1], xh[qt], xl[qt]);
                wb[qt] = make_uint4(wcur[2 * hf][qt].x, wcur[2 * hf][qt].y, wcur[2 * hf + 1][qt].x, wcur[2 * hf + 1][qt].y);
            }
#pragma unroll
            for (int dt = 0; dt < NDT; dt++) {
                const uint4 a = ld_tr2<LDH>(Ks[buf], 32 * hf + 4 * g, 32 * hf + 16 + 4 * g, 16 * dt);
#pragma unroll
                for (int qt = 0; qt < 2; qt++) {
                    aq[qt][dt] = mfma32(a, xh[qt], aq[qt][dt]);
                    aq[qt][dt] = mfma32(a, xl[qt], aq[qt][dt]);
                    bq[qt][dt] = mfma32(a, wb[qt], bq[qt][dt]);
                }
            }
        }
    }
#pragma unroll
    for (int qt = 0; qt < 2; qt++) {
        const int tq = qlo + 16 * qt + r;
        float dsum = dpart[qt];
        dsum += __shfl_xor(dsum, 16, 64);
        dsum += __shfl_xor(dsum, 32, 64);
        if (tq < s) {
            if (g == 0) dvec[(size_t)(b * H + h) * s + tq] = dsum;
            float *ob = d_q + (row0 + tq) * total + hoff;
#pragma unroll
            for (int dt = 0; dt < NDT; dt++)
                *reinterpret_cast<f32x4 *>(ob + 16 * dt + 4 * g) = (aq[qt][dt] - dsum * bq[qt][dt]) * scale;
        }
    }
}

// Key pass on statistics, in query blocks (one workgroup per 128 keys, one wave per 32): over the stages of 64
// queries that see the block's keys, a wave forms S = Q K^T for its two key tiles (rows = queries, column = the
// lane's key), the weights from the queries' statistics, dW = dO V^T, dS = w (dW - D_t) / sqrt(hd), and
// accumulates d_v^T += dO^T w and d_k^T += Q^T dS.  The Q and dO rows of a stage are staged as they arrive (dO as
// hi + lo); the products that contract over queries read them through ds_read_b64_tr_b16 in the query order
// that the score tiles leave in the lanes.  K and V of the wave's keys sit in registers.
template <int HDV, bool OUT16>
__global__ __launch_bounds__(256, 2) void swa_bwd_k_stats_kernel(const unsigned short *__restrict__ q,
                                                                 const unsigned short *__restrict__ k,
                                                                 const unsigned short *__restrict__ v,
                                                                 const float2 *__restrict__ stats,
                                                                 const float *__restrict__ d_out,
                                                                 const float *__restrict__ dvec,
                                                                 float *__restrict__ d_k, float *__restrict__ d_v,
                                                                 int s, int H, int ws, Out16 o16) {
    __shared__ __align__(16) unsigned short Qs[2][KS][LDH], Dh[2][KS][LDH], Dl[2][KS][LDH];   // [query][dim]
    __shared__ __align__(16) float Mc[2][KS], Iv[2][KS], Dd[2][KS];   // the stage's queries: maximum, 1 / sum, D
    const int tid = threadIdx.x, wave = tid >> 6, l = tid & 63, r = l & 15, g = l >> 4;
    const BlockCoord bc = xcd_block_coord(H);
    const int j0 = bc.x * FQ, h = bc.h, b = bc.b;
    constexpr int NKS = HDV / 32, NDT = HDV / 16;
    constexpr float kInvSqrt = HDV == 64 ? 0.125f : 0.17677669529663687f;   // 1 / sqrt(head size)
    const int total = H * HDV, hoff = h * HDV;
    const size_t row0 = (size_t)b * s;
    const int jlo = j0 + 32 * wave, jhi = jlo + 31;            // this wave's keys
    const int st_lo = j0 / KS, st_hi = min(s - 1, j0 + FQ - 1 + ws - 1) / KS;
    const float *dvb = dvec + (size_t)(b * H + h) * s;
    const float2 *stb = stats + (size_t)(b * H + h) * s;
    const StageSrc qm{q, row0, total, hoff, s};
    const float c2 = kInvSqrt * 1.44269504088896340736f, scale = kInvSqrt;

    uint4 kf[2][2], vf[2][2];   // B operands: key jlo + 16 jt + r, dims 32 ks + 8 g ..
#pragma unroll
    for (int jt = 0; jt < 2; jt++)
#pragma unroll
        for (int ks = 0; ks < NKS; ks++) {
            const int key = jlo + 16 * jt + r;
            kf[jt][ks] = make_uint4(0, 0, 0, 0);
            vf[jt][ks] = make_uint4(0, 0, 0, 0);
            if (key < s) {
                const size_t o = (row0 + key) * total + hoff + 32 * ks + 8 * g;
                kf[jt][ks] = *reinterpret_cast<const uint4 *>(k + o);
                vf[jt][ks] = *reinterpret_cast<const uint4 *>(v + o);
            }
        }
    f32x4 dk[2][4], dv[2][4];   // d_k^T, d_v^T: rows = dims 16 dt + 4 g + i, column = key
#pragma unroll
    for (int jt = 0; jt < 2; jt++)
#pragma unroll
        for (int dt = 0; dt < NDT; dt++) { dk[jt][dt] = f32x4{0.f, 0.f, 0.f, 0.f}; dv[jt][dt] = f32x4{0.f, 0.f, 0.f, 0.f}; }

    // one stage ahead in registers: Q rows (two 16-byte pieces per thread), dO rows (thread = quarter row)
    uint4 qreg[2];
    f32x4 dreg[4];
    float2 streg = make_float2(0.f, 0.f);
    float ddreg = 0.f;
    const int drow = tid >> 2, dcol = 16 * (tid & 3);
    auto fetch_stage = [&](int t_lo) {
        load_rows<HDV>(qm, t_lo, qreg);
        const int t = t_lo + drow;
#pragma unroll
        for (int c = 0; c < 4; c++) {
            dreg[c] = f32x4{0.f, 0.f, 0.f, 0.f};
            if (t < s && dcol < HDV) dreg[c] = *reinterpret_cast<const f32x4 *>(d_out + (row0 + t) * total + hoff + dcol + 4 * c);
        }
        streg = make_float2(0.f, 0.f);
        ddreg = 0.f;
        if (tid < KS && t_lo + tid < s) { streg = stb[t_lo + tid]; ddreg = dvb[t_lo + tid]; }
    };
    fetch_stage(KS * st_lo);
    for (int st = st_lo; st <= st_hi; st++) {
        const int buf = (st - st_lo) & 1, t_lo = KS * st;
#pragma unroll
        for (int c = 0; c < 2; c++) {
            const int chunk = tid + 256 * c;
            *reinterpret_cast<uint4 *>(&Qs[buf][chunk >> 3][8 * (chunk & 7)]) = qreg[c];
            uint4 hi, lo;
            split8(dreg[2 * c], dreg[2 * c + 1], hi, lo);
            *reinterpret_cast<uint4 *>(&Dh[buf][drow][dcol + 8 * c]) = hi;
            *reinterpret_cast<uint4 *>(&Dl[buf][drow][dcol + 8 * c]) = lo;
        }
        if (tid < KS) { Mc[buf][tid] = streg.x; Iv[buf][tid] = streg.y; Dd[buf][tid] = ddreg; }
        __syncthreads();
        if (st < st_hi) fetch_stage(t_lo + KS);
        if (t_lo + KS - 1 < jlo || t_lo > jhi + ws - 1) continue;   // no query of this stage sees a key of this wave
        const bool full = t_lo >= jhi && t_lo + KS - 1 <= jlo + ws - 1 && t_lo + KS - 1 < s && jhi < s;
#pragma unroll
        for (int hq = 0; hq < 2; hq++) {
            uint4 wpk[2], dsh[2], dsl[2];
            f32x4 ds[2][2];
            unsigned wp[2][2][2];
#pragma unroll
            for (int c = 0; c < 2; c++) {
                const int qt = 2 * hq + c;
                const uint4 aq0 = ld_op(Qs[buf], 16 * qt, 0), aq1 = ld_op(Qs[buf], 16 * qt, 1);
                const uint4 ah0 = ld_op(Dh[buf], 16 * qt, 0), ah1 = ld_op(Dh[buf], 16 * qt, 1);
                const uint4 al0 = ld_op(Dl[buf], 16 * qt, 0), al1 = ld_op(Dl[buf], 16 * qt, 1);
                const f32x4 m4 = *reinterpret_cast<const f32x4 *>(&Mc[buf][16 * qt + 4 * g]);
                const f32x4 i4 = *reinterpret_cast<const f32x4 *>(&Iv[buf][16 * qt + 4 * g]);
                const f32x4 d4 = *reinterpret_cast<const f32x4 *>(&Dd[buf][16 * qt + 4 * g]);
#pragma unroll
                for (int jt = 0; jt < 2; jt++) {
                    f32x4 sc = mfma32(aq0, kf[jt][0], f32x4{0.f, 0.f, 0.f, 0.f});
                    if constexpr (NKS == 2) sc = mfma32(aq1, kf[jt][1], sc);
                    f32x4 dw = mfma32(ah0, vf[jt][0], f32x4{0.f, 0.f, 0.f, 0.f});
                    dw = mfma32(al0, vf[jt][0], dw);
                    if constexpr (NKS == 2) dw = mfma32(ah1, vf[jt][1], dw);
                    if constexpr (NKS == 2) dw = mfma32(al1, vf[jt][1], dw);
                    f32x4 w;
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const int t = t_lo + 16 * qt + 4 * g + i, key = jlo + 16 * jt + r;
                        const bool ok = full || (key <= t && t <= key + ws - 1 && t < s && key < s);
                        w[i] = ok ? __builtin_amdgcn_exp2f(fmaf(sc[i], c2, -m4[i])) * i4[i] : 0.f;
                    }
                    wp[jt][c][0] = pack2(w[0], w[1]);   // as the weight tensor holds them
                    wp[jt][c][1] = pack2(w[2], w[3]);
                    ds[jt][c][0] = bf_lo(wp[jt][c][0]) * (dw[0] - d4[0]) * scale;
                    ds[jt][c][1] = bf_hi(wp[jt][c][0]) * (dw[1] - d4[1]) * scale;
                    ds[jt][c][2] = bf_lo(wp[jt][c][1]) * (dw[2] - d4[2]) * scale;
                    ds[jt][c][3] = bf_hi(wp[jt][c][1]) * (dw[3] - d4[3]) * scale;
                }
            }
#pragma unroll
            for (int jt = 0; jt < 2; jt++) {
                wpk[jt] = make_uint4(wp[jt][0][0], wp[jt][0][1], wp[jt][1][0], wp[jt][1][1]);
                split8(ds[jt][0], ds[jt][1], dsh[jt], dsl[jt]);
            }
#pragma unroll
            for (int dt = 0; dt < NDT; dt++) {
                const int ra = 32 * hq + 4 * g, rb = ra + 16;
                const uint4 aq = ld_tr2<LDH>(Qs[buf], ra, rb, 16 * dt);    // Q^T [dim][query]
                const uint4 ah = ld_tr2<LDH>(Dh[buf], ra, rb, 16 * dt);    // dO^T hi / lo
                const uint4 al = ld_tr2<LDH>(Dl[buf], ra, rb, 16 * dt);
#pragma unroll
                for (int jt = 0; jt < 2; jt++) {
                    dk[jt][dt] = mfma32(aq, dsh[jt], dk[jt][dt]);
                    dk[jt][dt] = mfma32(aq, dsl[jt], dk[jt][dt]);
                    dv[jt][dt] = mfma32(ah, wpk[jt], dv[jt][dt]);
                    dv[jt][dt] = mfma32(al, wpk[jt], dv[jt][dt]);
                }
            }
        }
    }
    // accumulate: column = key jlo + 16 jt + r, rows = dims 16 dt + 4 g ..
#pragma unroll
    for (int jt = 0; jt < 2; jt++) {
        const int key = jlo + 16 * jt + r;
        if (key >= s) continue;
        if (OUT16) {
            unsigned short *pk = o16.k + (row0 + key) * o16.ld + hoff, *pv = o16.v + (row0 + key) * o16.ld + hoff;
#pragma unroll
            for (int dt = 0; dt < NDT; dt++) {
                const f32x4 a = dk[jt][dt], c = dv[jt][dt];
                *reinterpret_cast<uint2 *>(pk + 16 * dt + 4 * g) = make_uint2(pack2(a[0], a[1]), pack2(a[2], a[3]));
                *reinterpret_cast<uint2 *>(pv + 16 * dt + 4 * g) = make_uint2(pack2(c[0], c[1]), pack2(c[2], c[3]));
            }
            continue;
        }
        float *pk = d_k + (row0 + key) * total + hoff, *pv = d_v + (row0 + key) * total + hoff;
#pragma unroll
        for (int dt = 0; dt < NDT; dt++) {
            f32x4 *ck = reinterpret_cast<f32x4 *>(pk + 16 * dt + 4 * g), *cv = reinterpret_cast<f32x4 *>(pv + 16 * dt + 4 * g);
            *ck = *ck + dk[jt][dt];
            *cv = *cv + dv[jt][dt];
        }
    }
}

// Key pass of the contract in query blocks, like swa_bwd_k_stats_kernel, with the weights read back from the tensor:
// the stage's 64 query rows x the block's 128 keys are 256 contiguous bytes per query where the window covers them;
// they are staged in LDS as [query][key] and a lane takes its two tiles (rows = queries, column = its key) with one
// transposing read, which is both the B operand of d_v^T += dO^T w and the w of dS = w (dW - D_t) / sqrt(hd).
constexpr int LDW = 144;   // row stride of the weight stage (288 B: the transposing reads of a group fall on 32 banks)

template <int HDV>
__global__ __launch_bounds__(256, 2) void swa_bwd_k_blocked_kernel(const unsigned short *__restrict__ q,
                                                                   const unsigned short *__restrict__ v,
                                                                   const unsigned short *__restrict__ attn_w,
                                                                   const float *__restrict__ d_out,
                                                                   const float *__restrict__ dvec,
                                                                   float *__restrict__ d_k, float *__restrict__ d_v,
                                                                   int s, int H, int ws) {
    __shared__ __align__(16) unsigned short Qs[2][KS][LDH], Dh[2][KS][LDH], Dl[2][KS][LDH];   // [query][dim]
    __shared__ __align__(16) unsigned short Wt[KS][LDW];                                       // [query][key of the block]
    __shared__ __align__(16) float Dd[2][KS];
    const int tid = threadIdx.x, wave = tid >> 6, l = tid & 63, r = l & 15, g = l >> 4;
    const BlockCoord bc = xcd_block_coord(H);
    const int j0 = bc.x * FQ, h = bc.h, b = bc.b;
    constexpr int NKS = HDV / 32, NDT = HDV / 16;
    constexpr float kInvSqrt = HDV == 64 ? 0.125f : 0.17677669529663687f;   // 1 / sqrt(head size)
    const int total = H * HDV, hoff = h * HDV;
    const size_t row0 = (size_t)b * s;
    const int jlo = j0 + 32 * wave, jhi = jlo + 31;
    const int st_lo = j0 / KS, st_hi = min(s - 1, j0 + FQ - 1 + ws - 1) / KS;
    const float *dvb = dvec + (size_t)(b * H + h) * s;
    const unsigned short *awb = attn_w + ((size_t)(b * H + h) * s) * ws;
    const StageSrc qm{q, row0, total, hoff, s};
    const float scale = kInvSqrt;

    uint4 vf[2][2];
#pragma unroll
    for (int jt = 0; jt < 2; jt++)
#pragma unroll
        for (int ks = 0; ks < NKS; ks++) {
            const int key = jlo + 16 * jt + r;
            vf[jt][ks] = make_uint4(0, 0, 0, 0);
            if (key < s) vf[jt][ks] = *reinterpret_cast<const uint4 *>(v + (row0 + key) * total + hoff + 32 * ks + 8 * g);
        }
    f32x4 dk[2][4], dv[2][4];
#pragma unroll
    for (int jt = 0; jt < 2; jt++)
#pragma unroll
        for (int dt = 0; dt < NDT; dt++) { dk[jt][dt] = f32x4{0.f, 0.f, 0.f, 0.f}; dv[jt][dt] = f32x4{0.f, 0.f, 0.f, 0.f}; }

    uint4 qreg[2], wreg[4];
    f32x4 dreg[4];
    float ddreg = 0.f;
    const int drow = tid >> 2, dcol = 16 * (tid & 3);
    auto fetch_stage = [&](int t_lo) {
        load_rows<HDV>(qm, t_lo, qreg);
        const int t = t_lo + drow;
#pragma unroll
        for (int c = 0; c < 4; c++) {
            dreg[c] = f32x4{0.f, 0.f, 0.f, 0.f};
            if (t < s && dcol < HDV) dreg[c] = *reinterpret_cast<const f32x4 *>(d_out + (row0 + t) * total + hoff + dcol + 4 * c);
        }
        ddreg = (tid < KS && t_lo + tid < s) ? dvb[t_lo + tid] : 0.f;
        // weights of query t for keys j0 + 32 (tid % 4) .. + 31: four pieces of 8 keys
        const int lsq = max(t + 1 - ws, 0), thi = t < s ? t : -1;
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const int key0 = j0 + 32 * (tid & 3) + 8 * c;
            wreg[c] = make_uint4(0, 0, 0, 0);
            if (key0 >= lsq && key0 + 7 <= thi) {
                __builtin_memcpy(&wreg[c], awb + (size_t)t * ws + (key0 - lsq), 16);
            } else if (key0 + 7 >= lsq && key0 <= thi) {
                unsigned d[4] = {0u, 0u, 0u, 0u};
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const int key = key0 + e;
                    unsigned x = 0;
                    if (key >= lsq && key <= thi) x = awb[(size_t)t * ws + (key - lsq)];
                    d[e >> 1] |= x << (16 * (e & 1));
                }
                wreg[c] = make_uint4(d[0], d[1], d[2], d[3]);
            }
        }
    };
    fetch_stage(KS * st_lo);
    for (int st = st_lo; st <= st_hi; st++) {
        const int buf = (st - st_lo) & 1, t_lo = KS * st;
#pragma unroll
        for (int c = 0; c < 2; c++) {
            const int chunk = tid + 256 * c;
            *reinterpret_cast<uint4 *>(&Qs[buf][chunk >> 3][8 * (chunk & 7)]) = qreg[c];
            uint4 hi, lo;
            split8(dreg[2 * c], dreg[2 * c + 1], hi, lo);
            *reinterpret_cast<uint4 *>(&Dh[buf][drow][dcol + 8 * c]) = hi;
            *reinterpret_cast<uint4 *>(&Dl[buf][drow][dcol + 8 * c]) = lo;
        }
#pragma unroll
        for (int c = 0; c < 4; c++) *reinterpret_cast<uint4 *>(&Wt[drow][32 * (tid & 3) + 8 * c]) = wreg[c];
        if (tid < KS) Dd[buf][tid] = ddreg;
        __syncthreads();
        if (st < st_hi) fetch_stage(t_lo + KS);
        if (!(t_lo + KS - 1 < jlo || t_lo > jhi + ws - 1)) {   // a query of this stage sees a key of this wave
#pragma unroll
            for (int hq = 0; hq < 2; hq++) {
                const int ra = 32 * hq + 4 * g, rb = ra + 16;
                uint4 wpk[2], dsh[2], dsl[2];
                f32x4 ds[2][2];
#pragma unroll
                for (int jt = 0; jt < 2; jt++) wpk[jt] = ld_tr2<LDW>(Wt, ra, rb, 32 * wave + 16 * jt);
#pragma unroll
                for (int c = 0; c < 2; c++) {
                    const int qt = 2 * hq + c;
                    const uint4 ah0 = ld_op(Dh[buf], 16 * qt, 0), ah1 = ld_op(Dh[buf], 16 * qt, 1);
                    const uint4 al0 = ld_op(Dl[buf], 16 * qt, 0), al1 = ld_op(Dl[buf], 16 * qt, 1);
                    const f32x4 d4 = *reinterpret_cast<const f32x4 *>(&Dd[buf][16 * qt + 4 * g]);
#pragma unroll
                    for (int jt = 0; jt < 2; jt++) {
                        f32x4 dw = mfma32(ah0, vf[jt][0], f32x4{0.f, 0.f, 0.f, 0.f});
                        dw = mfma32(al0, vf[jt][0], dw);
                        if constexpr (NKS == 2) dw = mfma32(ah1, vf[jt][1], dw);
                        if constexpr (NKS == 2) dw = mfma32(al1, vf[jt][1], dw);
                        const unsigned w01 = c ? wpk[jt].z : wpk[jt].x, w23 = c ? wpk[jt].w : wpk[jt].y;
                        ds[jt][c][0] = bf_lo(w01) * (dw[0] - d4[0]) * scale;
                        ds[jt][c][1] = bf_hi(w01) * (dw[1] - d4[1]) * scale;
                        ds[jt][c][2] = bf_lo(w23) * (dw[2] - d4[2]) * scale;
                        ds[jt][c][3] = bf_hi(w23) * (dw[3] - d4[3]) * scale;
                    }
                }
#pragma unroll
                for (int jt = 0; jt < 2; jt++) split8(ds[jt][0], ds[jt][1], dsh[jt], dsl[jt]);
#pragma unroll
                for (int dt = 0; dt < NDT; dt++) {
                    const uint4 aq = ld_tr2<LDH>(Qs[buf], ra, rb, 16 * dt);    // Q^T [dim][query]
                    const uint4 ah = ld_tr2<LDH>(Dh[buf], ra, rb, 16 * dt);    // dO^T hi / lo
                    const uint4 al = ld_tr2<LDH>(Dl[buf], ra, rb, 16 * dt);
#pragma unroll
                    for (int jt = 0; jt < 2; jt++) {
                        dk[jt][dt] = mfma32(aq, dsh[jt], dk[jt][dt]);
                        dk[jt][dt] = mfma32(aq, dsl[jt], dk[jt][dt]);
                        dv[jt][dt] = mfma32(ah, wpk[jt], dv[jt][dt]);
                        dv[jt][dt] = mfma32(al, wpk[jt], dv[jt][dt]);
                    }
                }
            }
        }
        __syncthreads();   // the weight stage has one buffer: every wave is done with it before the next one lands
    }
#pragma unroll
    for (int jt = 0; jt < 2; jt++) {
        const int key = jlo + 16 * jt + r;
        if (key >= s) continue;
        float *pk = d_k + (row0 + key) * total + hoff, *pv = d_v + (row0 + key) * total + hoff;
#pragma unroll
        for (int dt = 0; dt < NDT; dt++) {
            f32x4 *ck = reinterpret_cast<f32x4 *>(pk + 16 * dt + 4 * g), *cv = reinterpret_cast<f32x4 *>(pv + 16 * dt + 4 * g);
            *ck = *ck + dk[jt][dt];
            *cv = *cv + dv[jt][dt];
        }
    }
}

}  // namespace

bool swa_forward_mfma(const uint16_t *q, const uint16_t *k, const uint16_t *v, uint16_t *out, uint16_t *attn_weights,
                      int seq_len, int num_heads, int head_dim, int window, int batch, int n_persistent, float *stats) {
    if ((head_dim != 64 && head_dim != 32) || n_persistent != 0 || window > 512 || window < 1) return false;
    if (stats) {
        KernelTimer kt("swa_fwd_stats_kernel");
        if (head_dim == 64) hipLaunchKernelGGL(swa_fwd_stats_kernel<64>, dim3((seq_len + FQ - 1) / FQ, num_heads, batch), dim3(256), 0, stream(), q,
                           k, v, out, reinterpret_cast<float2 *>(stats), seq_len, num_heads, window);
        else hipLaunchKernelGGL(swa_fwd_stats_kernel<32>, dim3((seq_len + FQ - 1) / FQ, num_heads, batch), dim3(256), 0, stream(), q,
                           k, v, out, reinterpret_cast<float2 *>(stats), seq_len, num_heads, window);
        check_launch("swa_fwd_stats_kernel");
        return true;
    }
    KernelTimer kt("swa_fwd_blocked_kernel");
    if (head_dim == 64) hipLaunchKernelGGL(swa_fwd_blocked_kernel<64>, dim3((seq_len + FQ - 1) / FQ, num_heads, batch), dim3(256), 0, stream(), q,
                       k, v, out, attn_weights, seq_len, num_heads, window);
    else hipLaunchKernelGGL(swa_fwd_blocked_kernel<32>, dim3((seq_len + FQ - 1) / FQ, num_heads, batch), dim3(256), 0, stream(), q,
                       k, v, out, attn_weights, seq_len, num_heads, window);
    check_launch("swa_fwd_blocked_kernel");
    return true;
}

bool swa_backward_mfma(const uint16_t *q, const uint16_t *k, const uint16_t *v, const uint16_t *attn_weights,
                       const float *d_attn_out, float *d_q, float *d_k, float *d_v, int seq_len, int num_heads,
                       int head_dim, int window, int batch, int n_persistent, const float *stats, const SwaGradCols *cols) {
    const ErrorScope es;
    if ((head_dim != 64 && head_dim != 32) || n_persistent != 0 || window > 512 || window < 1) return false;
    float *dvec = scratch(1, (size_t)batch * num_heads * seq_len * sizeof(float));
    if (es.failed()) return true;
    if (stats) {
        const float2 *st2 = reinterpret_cast<const float2 *>(stats);
        const dim3 grid((seq_len + FQ - 1) / FQ, num_heads, batch);
        const Out16 o16 = cols ? Out16{cols->q, cols->k, cols->v, cols->ld} : Out16{nullptr, nullptr, nullptr, 0};
#define NLH_SWA_BWD_STATS(HDV, O16)                                                                                       \
    {                                                                                                                     \
        {                                                                                                                 \
            KernelTimer kt("swa_bwd_q_stats_kernel");                                                                     \
            hipLaunchKernelGGL((swa_bwd_q_stats_kernel<HDV, O16>), grid, dim3(256), 0, stream(), q, k, v, st2, d_attn_out, d_q, \
                               dvec, seq_len, num_heads, window, o16);                                                    \
            check_launch("swa_bwd_q_stats_kernel");                                                                       \
        }                                                                                                                 \
        KernelTimer kt("swa_bwd_k_stats_kernel");                                                                         \
        hipLaunchKernelGGL((swa_bwd_k_stats_kernel<HDV, O16>), grid, dim3(256), 0, stream(), q, k, v, st2, d_attn_out, dvec,   \
                           d_k, d_v, seq_len, num_heads, window, o16);                                                    \
        check_launch("swa_bwd_k_stats_kernel");                                                                           \
    }
        if (head_dim == 64) { if (cols) NLH_SWA_BWD_STATS(64, true) else NLH_SWA_BWD_STATS(64, false) }
        else { if (cols) NLH_SWA_BWD_STATS(32, true) else NLH_SWA_BWD_STATS(32, false) }
#undef NLH_SWA_BWD_STATS
        return true;
    }
    if (cols) return false;   // bf16 column output exists for the statistics pair only
    {
        KernelTimer kt("swa_bwd_q_blocked_kernel");
        if (head_dim == 64) hipLaunchKernelGGL(swa_bwd_q_blocked_kernel<64>, dim3((seq_len + FQ - 1) / FQ, num_heads, batch), dim3(256), 0,
                           stream(), k, v, attn_weights, d_attn_out, d_q, dvec, seq_len, num_heads, window);
        else hipLaunchKernelGGL(swa_bwd_q_blocked_kernel<32>, dim3((seq_len + FQ - 1) / FQ, num_heads, batch), dim3(256), 0,
                           stream(), k, v, attn_weights, d_attn_out, d_q, dvec, seq_len, num_heads, window);
        check_launch("swa_bwd_q_blocked_kernel");
    }
    KernelTimer kt("swa_bwd_k_blocked_kernel");
    if (head_dim == 64) hipLaunchKernelGGL(swa_bwd_k_blocked_kernel<64>, dim3((seq_len + FQ - 1) / FQ, num_heads, batch), dim3(256), 0, stream(), q,
                       v, attn_weights, d_attn_out, dvec, d_k, d_v, seq_len, num_heads, window);
    else hipLaunchKernelGGL(swa_bwd_k_blocked_kernel<32>, dim3((seq_len + FQ - 1) / FQ, num_heads, batch), dim3(256), 0, stream(), q,
                       v, attn_weights, d_attn_out, dvec, d_k, d_v, seq_len, num_heads, window);
    check_launch("swa_bwd_k_blocked_kernel");
    return true;
}

}  // namespace nlh
