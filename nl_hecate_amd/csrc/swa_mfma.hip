// Sliding-window attention on the bf16 matrix cores for head size 64, no
// persistent prefix, window <= 512 (the production shape).  Contract and mask
// are those of core/kernels/swa_forward.cu / swa_backward.cu; other shapes stay
// on the wave-per-query kernels of swa.hip.
//
// Forward.  One workgroup per (64 queries, head, batch), one wave per 16 queries.
// The wave computes S^T = K Q^T for its 16 queries against the 576 keys
// [t0-512, t0+64) that the block can see, 36 tiles of 16x16 kept in registers
// (v_mfma_f32_16x16x16_bf16: A = 16 keys x 16 dims from an LDS-staged K tile,
// B = the wave's Q fragment).  In this orientation a lane owns ONE query column
// and 144 of its keys, so the softmax is a per-lane reduction plus two
// exchanges, and the normalised tile is already laid out as the B operand of
// O^T = V^T P^T: no shuffles between the two products.  V tiles are staged
// transposed in LDS.  The normalised weights (part of the contract) leave
// through a per-wave LDS tile so that each store instruction writes 128
// contiguous bytes of one query's slot row.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>

#include "lane_ops.h"
#include "runtime.h"
#include "swa_mfma.h"

namespace nlh {
namespace {

typedef short bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int HD = 64;        // head size
constexpr int QB = 64;        // queries per workgroup
constexpr int KS = 64;        // keys per LDS stage
constexpr int NS = 9;         // stages: 576 keys
constexpr int NT = 36;        // 16-key tiles
constexpr int LDH = 72;       // LDS row stride in bf16 elements (144 B: 16-byte aligned rows)

__device__ __forceinline__ unsigned short f2bf(float f) {
    unsigned u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (unsigned short)((u >> 16) | 0x40);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (unsigned short)(u >> 16);
}
__device__ __forceinline__ bf16x4 pack4(f32x4 x) {
    bf16x4 r;
    r[0] = (short)f2bf(x[0]); r[1] = (short)f2bf(x[1]); r[2] = (short)f2bf(x[2]); r[3] = (short)f2bf(x[3]);
    return r;
}
__device__ __forceinline__ f32x4 mfma16(bf16x4 a, bf16x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, b, c, 0, 0, 0);
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

__global__ __launch_bounds__(256) void swa_fwd_mfma_kernel(const unsigned short *__restrict__ q,
                                                           const unsigned short *__restrict__ k,
                                                           const unsigned short *__restrict__ v,
                                                           unsigned short *__restrict__ out,
                                                           unsigned short *__restrict__ attn_w, int s, int H,
                                                           int ws) {
    __shared__ __align__(16) unsigned short Ks[2][KS][LDH];   // K stage (row-major), then V^T stage [d][key]
    __shared__ __align__(16) unsigned short Pw[4][16][KS];    // per wave: normalised weights of one stage
    const int tid = threadIdx.x, wave = tid >> 6, l = tid & 63, r = l & 15, g = l >> 4;
    const BlockCoord bc = xcd_block_coord(H);
    const int t0 = bc.x * QB, h = bc.h, b = bc.b;
    const int total = H * HD, hoff = h * HD;
    const int base = t0 + QB - NS * KS;               // first key of stage 0 (may be negative)
    const int tq = t0 + 16 * wave + r;                // this lane's query (column of S^T)
    const size_t row0 = (size_t)b * s;
    const int first_key = max(t0 + 1 - ws, 0);        // smallest key any query of the block sees
    const int st_lo = max(0, (first_key - base) / KS);   // stages before it hold masked keys only

    bf16x4 qf[4];
#pragma unroll
    for (int st = 0; st < 4; st++) {
        qf[st] = bf16x4{0, 0, 0, 0};
        if (tq < s) qf[st] = *reinterpret_cast<const bf16x4 *>(q + (row0 + tq) * total + hoff + 16 * st + 4 * g);
    }
    f32x4 acc[NT];
#pragma unroll
    for (int i = 0; i < NT; i++) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};

    // cooperative stage loads: 64 rows x 128 B = 512 chunks of 16 B, two per thread
    auto load_rows = [&](const unsigned short *src, int stage, uint4 (&regs)[2]) {
#pragma unroll
        for (int c = 0; c < 2; c++) {
            const int chunk = tid + 256 * c, key = base + KS * stage + (chunk >> 3);
            regs[c] = make_uint4(0, 0, 0, 0);
            if (key >= 0 && key < s)
                regs[c] = *reinterpret_cast<const uint4 *>(src + (row0 + key) * total + hoff + 8 * (chunk & 7));
        }
    };
    // rows for a transposed stage: the thread takes 8 dims of two neighbouring keys
    auto load_pairs = [&](const unsigned short *src, int stage, uint4 (&regs)[2]) {
        const int kp = tid & 31, d0 = 8 * (tid >> 5);
#pragma unroll
        for (int c = 0; c < 2; c++) {
            const int key = base + KS * stage + 2 * kp + c;
            regs[c] = make_uint4(0, 0, 0, 0);
            if (key >= 0 && key < s) regs[c] = *reinterpret_cast<const uint4 *>(src + (row0 + key) * total + hoff + d0);
        }
    };
    uint4 stg[2];

    // ---- pass A: S^T tiles ----
    load_rows(k, st_lo, stg);
#pragma unroll
    for (int st = 0; st < NS; st++) {
        if (st < st_lo) continue;
        const int buf = st & 1;
#pragma unroll
        for (int c = 0; c < 2; c++) {
            const int chunk = tid + 256 * c;
            *reinterpret_cast<uint4 *>(&Ks[buf][chunk >> 3][8 * (chunk & 7)]) = stg[c];
        }
        __syncthreads();
        if (st + 1 < NS) load_rows(k, st + 1, stg);
#pragma unroll
        for (int kt = 0; kt < 4; kt++)
#pragma unroll
            for (int sp = 0; sp < 4; sp++) {
                const bf16x4 a = *reinterpret_cast<const bf16x4 *>(&Ks[buf][16 * kt + r][16 * sp + 4 * g]);
                acc[4 * st + kt] = mfma16(a, qf[sp], acc[4 * st + kt]);
            }
    }

    // ---- mask, scale, softmax over this lane's query column ----
    const float scale = 0.125f;   // 1/sqrt(64)
    const int lsq = max(tq + 1 - ws, 0);
    float mx = -INFINITY;
#pragma unroll
    for (int T = 0; T < NT; T++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int key = base + 16 * T + 4 * g + i;
            const bool ok = key >= lsq && key <= tq && tq < s;
            const float x = ok ? acc[T][i] * scale : -INFINITY;
            acc[T][i] = x;
            mx = fmaxf(mx, x);
        }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    float sum = 0.f;
#pragma unroll
    for (int T = 0; T < NT; T++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float e = acc[T][i] == -INFINITY ? 0.f : expf(acc[T][i] - mx);
            acc[T][i] = e;
            sum += e;
        }
    sum += __shfl_xor(sum, 16, 64);
    sum += __shfl_xor(sum, 32, 64);
    const float inv = sum > 0.f ? 1.0f / sum : 0.f;

    // ---- pass B: O^T = V^T P^T, weights out ----
    f32x4 o[4];
#pragma unroll
    for (int i = 0; i < 4; i++) o[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    unsigned short *awb = attn_w + ((size_t)(b * H + h) * s) * ws;
    __syncthreads();   // every wave is done with the last K stage
    load_pairs(v, st_lo, stg);
#pragma unroll
    for (int st = 0; st < NS; st++) {
        if (st < st_lo) continue;
        const int buf = st & 1;
        // transposed staging as 32-bit key pairs (bank = key pair: no conflicts): Vt[dim][key]
        {
            const int kp = tid & 31, d0 = 8 * (tid >> 5);
            const unsigned e[4] = {stg[0].x, stg[0].y, stg[0].z, stg[0].w};
            const unsigned o2[4] = {stg[1].x, stg[1].y, stg[1].z, stg[1].w};
#pragma unroll
            for (int j = 0; j < 4; j++) {
                *reinterpret_cast<unsigned *>(&Ks[buf][d0 + 2 * j][2 * kp]) = (e[j] & 0xffffu) | (o2[j] << 16);
                *reinterpret_cast<unsigned *>(&Ks[buf][d0 + 2 * j + 1][2 * kp]) = (e[j] >> 16) | (o2[j] & 0xffff0000u);
            }
        }
        __syncthreads();
        if (st + 1 < NS) load_pairs(v, st + 1, stg);
#pragma unroll
        for (int kt = 0; kt < 4; kt++) {
            f32x4 p = acc[4 * st + kt];
#pragma unroll
            for (int i = 0; i < 4; i++) p[i] *= inv;
            const bf16x4 pb = pack4(p);
            *reinterpret_cast<bf16x4 *>(&Pw[wave][r][16 * kt + 4 * g]) = pb;
#pragma unroll
            for (int dt = 0; dt < 4; dt++) {
                const bf16x4 a = *reinterpret_cast<const bf16x4 *>(&Ks[buf][16 * dt + r][16 * kt + 4 * g]);
                o[dt] = mfma16(a, pb, o[dt]);
            }
        }
        // this stage's weights: one query row per instruction, 64 consecutive slots
        // (the tile was written by this wave only; order the LDS stores before the loads)
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll 4
        for (int qi = 0; qi < 16; qi++) {
            const int tt = t0 + 16 * wave + qi, key = base + KS * st + l;
            const int slot = key - max(tt + 1 - ws, 0);
            if (tt < s && slot >= 0 && slot < ws) awb[(size_t)tt * ws + slot] = Pw[wave][qi][l];
        }
        asm volatile("" ::: "memory");
    }
    // slots whose keys lie beyond the block's last key (early queries only): zero
    if (t0 + QB < ws) {
        for (int qi = 0; qi < 16; qi++) {
            const int tt = t0 + 16 * wave + qi;
            if (tt >= s) break;
            for (int slot = t0 + QB + l; slot < ws; slot += 64) awb[(size_t)tt * ws + slot] = 0;
        }
    }
    if (tq < s) {
        unsigned short *ob = out + (row0 + tq) * total + hoff;
#pragma unroll
        for (int dt = 0; dt < 4; dt++) *reinterpret_cast<bf16x4 *>(ob + 16 * dt + 4 * g) = pack4(o[dt]);
    }
}

__device__ __forceinline__ float bf2f(unsigned short h) { return __uint_as_float(((unsigned)h) << 16); }
// x = hi + lo with hi, lo bf16: the pair carries 16 mantissa bits through a bf16 product
__device__ __forceinline__ void split4(f32x4 x, bf16x4 &hi, bf16x4 &lo) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const unsigned short h = f2bf(x[i]);
        hi[i] = (short)h;
        lo[i] = (short)f2bf(x[i] - bf2f(h));
    }
}

// Backward, query pass (one workgroup per 64 queries, one wave per 16 queries):
//   D_t = sum_j w dW = dO_t . O_t with O_t = sum_j w[t,j] v_j recomputed from the stored (bf16) weights,
//   dW[t,j] = dO_t . v_j,  dS = w (dW - D_t) / sqrt(hd),  d_q[t] = sum_j dS[t,j] k_j.
// Two sweeps over the window: the first rebuilds O^T (four accumulators) and from it D; the second
// recomputes each dW tile next to its use, so no score tile outlives a stage.  dO and dS enter the
// bf16 products as hi + lo pairs.  D_t goes to dvec for the key pass.
//
// The weights never pass through LDS.  Within a stage of 64 keys, element i of lane group g in
// 16-key tile kt stands for key 32 (kt / 2) + 8 g + 4 (kt % 2) + i, so that the B operands of one
// query for two tiles are 8 consecutive slots of its weight row: one 16-byte load (2-byte aligned)
// per lane, kept in registers for the second sweep.  The LDS tiles of V and K are stored in that key
// order (stage_pos).  Only the last stage, the one that holds the queries themselves, is read slot
// by slot: its groups can end inside the 16 bytes, and a load that runs past the query's row would
// leave the array at its last row.
__device__ __forceinline__ int stage_pos(int key) {   // key 32 a + 8 g + 4 c + i -> 16 (2 a + c) + 4 g + i
    return (key & 0x23) | ((key & 0x18) >> 1) | ((key & 0x04) << 2);
}

__global__ __launch_bounds__(256, 2) void swa_bwd_q_mfma_kernel(const unsigned short *__restrict__ k,
                                                                const unsigned short *__restrict__ v,
                                                                const unsigned short *__restrict__ attn_w,
                                                                const float *__restrict__ d_out,
                                                                float *__restrict__ d_q, float *__restrict__ dvec,
                                                                int s, int H, int ws) {
    __shared__ __align__(16) unsigned short Vr[2][KS][LDH];   // V stage, [stage_pos(key)][dim]
    __shared__ __align__(16) unsigned short Tt[2][HD][LDH];   // transposed stage [dim][stage_pos(key)]: V (sweep 1), K (sweep 2)
    const int tid = threadIdx.x, wave = tid >> 6, l = tid & 63, r = l & 15, g = l >> 4;
    const BlockCoord bc = xcd_block_coord(H);
    const int t0 = bc.x * QB, h = bc.h, b = bc.b;
    const int total = H * HD, hoff = h * HD;
    const int base = t0 + QB - NS * KS;
    const int tq = t0 + 16 * wave + r;
    const int lsq = max(tq + 1 - ws, 0);
    const size_t row0 = (size_t)b * s;
    const int st_lo = max(0, (max(t0 + 1 - ws, 0) - base) / KS);
    const unsigned short *wrow = attn_w + ((size_t)(b * H + h) * s + min(tq, s - 1)) * ws;

    f32x4 dof[4];     // dO_t at dims 16 sp + 4 g .. +3: the positions of this lane in an O^T tile
    bf16x4 doh[4], dol[4];
#pragma unroll
    for (int sp = 0; sp < 4; sp++) {
        dof[sp] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (tq < s) dof[sp] = *reinterpret_cast<const f32x4 *>(d_out + (row0 + tq) * total + hoff + 16 * sp + 4 * g);
        split4(dof[sp], doh[sp], dol[sp]);
    }

    auto load_rows = [&](const unsigned short *src, int stage, uint4 (&regs)[2]) {
#pragma unroll
        for (int c = 0; c < 2; c++) {
            const int chunk = tid + 256 * c, key = base + KS * stage + (chunk >> 3);
            regs[c] = make_uint4(0, 0, 0, 0);
            if (key >= 0 && key < s)
                regs[c] = *reinterpret_cast<const uint4 *>(src + (row0 + key) * total + hoff + 8 * (chunk & 7));
        }
    };
    auto commit_rows = [&](int buf, const uint4 (&regs)[2]) {
#pragma unroll
        for (int c = 0; c < 2; c++) {
            const int chunk = tid + 256 * c;
            *reinterpret_cast<uint4 *>(&Vr[buf][stage_pos(chunk >> 3)][8 * (chunk & 7)]) = regs[c];
        }
    };
    // rows for a transposed stage: the thread takes 8 dims of two neighbouring keys, so that the
    // transposed tile is written as 32-bit key pairs (bank = key pair: no conflicts)
    auto load_pairs = [&](const unsigned short *src, int stage, uint4 (&regs)[2]) {
        const int kp = tid & 31, d0 = 8 * (tid >> 5);
#pragma unroll
        for (int c = 0; c < 2; c++) {
            const int key = base + KS * stage + 2 * kp + c;
            regs[c] = make_uint4(0, 0, 0, 0);
            if (key >= 0 && key < s) regs[c] = *reinterpret_cast<const uint4 *>(src + (row0 + key) * total + hoff + d0);
        }
    };
    auto commit_transposed = [&](int buf, const uint4 (&regs)[2]) {
        const int col = stage_pos(2 * (tid & 31)), d0 = 8 * (tid >> 5);
        const unsigned e[4] = {regs[0].x, regs[0].y, regs[0].z, regs[0].w};
        const unsigned o[4] = {regs[1].x, regs[1].y, regs[1].z, regs[1].w};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            *reinterpret_cast<unsigned *>(&Tt[buf][d0 + 2 * j][col]) = (e[j] & 0xffffu) | (o[j] << 16);
            *reinterpret_cast<unsigned *>(&Tt[buf][d0 + 2 * j + 1][col]) = (e[j] >> 16) | (o[j] & 0xffff0000u);
        }
    };
    // weights of this lane's query for the keys of its group in a stage: wv[stage][half] holds the
    // 8 keys 32 half + 8 g .. + 7 (B operands of tiles 2 half and 2 half + 1), zero outside the window
    uint4 wv[NS][2];
    auto fetch_weights = [&](int stage, uint4 (&w)[2]) {
#pragma unroll
        for (int hf = 0; hf < 2; hf++) {
            const int key0 = base + KS * stage + 32 * hf + 8 * g;
            w[hf] = make_uint4(0, 0, 0, 0);
            if (stage < NS - 1) {
                // keys below t0: the group never runs past the query; it may start before the window
                if (tq < s && key0 + 7 >= lsq) {
                    uint4 x;
                    __builtin_memcpy(&x, wrow + (key0 - lsq), 16);
                    const int cut = lsq - key0;   // elements below cut are outside the window
                    x.x &= (cut > 0 ? 0u : 0xffffu) | (cut > 1 ? 0u : 0xffff0000u);
                    x.y &= (cut > 2 ? 0u : 0xffffu) | (cut > 3 ? 0u : 0xffff0000u);
                    x.z &= (cut > 4 ? 0u : 0xffffu) | (cut > 5 ? 0u : 0xffff0000u);
                    x.w &= (cut > 6 ? 0u : 0xffffu) | (cut > 7 ? 0u : 0xffff0000u);
                    w[hf] = x;
                }
            } else {
                unsigned d[4] = {0u, 0u, 0u, 0u};
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const int key = key0 + e;
                    unsigned x = 0;
                    if (tq < s && key >= lsq && key <= tq) x = wrow[key - lsq];
                    d[e >> 1] |= x << (16 * (e & 1));
                }
                w[hf] = make_uint4(d[0], d[1], d[2], d[3]);
            }
        }
    };
    auto b_operand = [&](const uint4 &w, int odd) {
        const unsigned lo = odd ? w.z : w.x, hi = odd ? w.w : w.y;
        bf16x4 pb;
        pb[0] = (short)(lo & 0xffffu); pb[1] = (short)(lo >> 16); pb[2] = (short)(hi & 0xffffu); pb[3] = (short)(hi >> 16);
        return pb;
    };
    uint4 sv[2], sk[2];

    // ---- sweep 1: O^T = V^T P^T, then D = dO . O ----
    f32x4 ot[4];
#pragma unroll
    for (int i = 0; i < 4; i++) ot[i] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int st = 0; st < NS; st++) { wv[st][0] = make_uint4(0, 0, 0, 0); wv[st][1] = make_uint4(0, 0, 0, 0); }
    load_pairs(v, st_lo, sv);
#pragma unroll
    for (int st = 0; st < NS; st++) {
        if (st < st_lo) continue;
        const int buf = st & 1;
        fetch_weights(st, wv[st]);
        commit_transposed(buf, sv);
        __syncthreads();
        if (st + 1 < NS) load_pairs(v, st + 1, sv);
#pragma unroll
        for (int kt = 0; kt < 4; kt++) {
            const bf16x4 pb = b_operand(wv[st][kt >> 1], kt & 1);
#pragma unroll
            for (int dt = 0; dt < 4; dt++) {
                const bf16x4 a = *reinterpret_cast<const bf16x4 *>(&Tt[buf][16 * dt + r][16 * kt + 4 * g]);
                ot[dt] = mfma16(a, pb, ot[dt]);
            }
        }
    }
    float dsum = 0.f;
#pragma unroll
    for (int dt = 0; dt < 4; dt++)
#pragma unroll
        for (int i = 0; i < 4; i++) dsum = fmaf(dof[dt][i], ot[dt][i], dsum);
    dsum += __shfl_xor(dsum, 16, 64);
    dsum += __shfl_xor(dsum, 32, 64);
    if (g == 0 && tq < s) dvec[(size_t)(b * H + h) * s + tq] = dsum;

    // ---- sweep 2: dW^T tiles recomputed, dS, d_q^T = K^T dS^T ----
    f32x4 dq[4];
#pragma unroll
    for (int i = 0; i < 4; i++) dq[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    const float scale = 0.125f;
    __syncthreads();
    load_rows(v, st_lo, sv);
    load_pairs(k, st_lo, sk);
#pragma unroll
    for (int st = 0; st < NS; st++) {
        if (st < st_lo) continue;
        const int buf = st & 1;
        commit_rows(buf, sv);
        commit_transposed(buf, sk);
        __syncthreads();
        if (st + 1 < NS) { load_rows(v, st + 1, sv); load_pairs(k, st + 1, sk); }
#pragma unroll
        for (int kt = 0; kt < 4; kt++) {
            f32x4 dw = f32x4{0.f, 0.f, 0.f, 0.f};   // dW^T[key of (kt, g, i)][query r]
#pragma unroll
            for (int sp = 0; sp < 4; sp++) {
                const bf16x4 a = *reinterpret_cast<const bf16x4 *>(&Vr[buf][16 * kt + r][16 * sp + 4 * g]);
                dw = mfma16(a, doh[sp], dw);
                dw = mfma16(a, dol[sp], dw);
            }
            const bf16x4 pb = b_operand(wv[st][kt >> 1], kt & 1);
            f32x4 ds;
#pragma unroll
            for (int i = 0; i < 4; i++) ds[i] = bf2f((unsigned short)pb[i]) * (dw[i] - dsum) * scale;
            bf16x4 dsh, dsl;
            split4(ds, dsh, dsl);
#pragma unroll
            for (int dt = 0; dt < 4; dt++) {
                const bf16x4 a = *reinterpret_cast<const bf16x4 *>(&Tt[buf][16 * dt + r][16 * kt + 4 * g]);
                dq[dt] = mfma16(a, dsh, dq[dt]);
                dq[dt] = mfma16(a, dsl, dq[dt]);
            }
        }
    }
    if (tq < s) {
        float *ob = d_q + (row0 + tq) * total + hoff;
#pragma unroll
        for (int dt = 0; dt < 4; dt++) *reinterpret_cast<f32x4 *>(ob + 16 * dt + 4 * g) = dq[dt];
    }
}

// Backward, key pass (one workgroup per 64 keys, one wave per 16 keys): over the up to 575
// queries t in [j, j + window) that see key j,
//   d_v[j] += sum_t w[t,j] dO_t,   d_k[j] += sum_t dS[t,j] q_t,   dS recomputed from w, dO.v_j, D_t.
// A tile of dS / w in accumulator layout (rows = queries, column = the lane's key) is exactly
// the A operand of the products with Q^T / dO^T, which are staged transposed in LDS.
__global__ __launch_bounds__(256) void swa_bwd_k_mfma_kernel(const unsigned short *__restrict__ q,
                                                             const unsigned short *__restrict__ v,
                                                             const unsigned short *__restrict__ attn_w,
                                                             const float *__restrict__ d_out,
                                                             const float *__restrict__ dvec,
                                                             float *__restrict__ d_k, float *__restrict__ d_v,
                                                             int s, int H, int ws) {
    __shared__ __align__(16) unsigned short Dh[KS][LDH], Dl[KS][LDH];      // dO hi / lo, [query][dim]
    __shared__ __align__(16) unsigned short DhT[HD][LDH], DlT[HD][LDH];    // transposed, [dim][query]
    __shared__ __align__(16) unsigned short QT[HD][LDH];                   // Q^T, [dim][query]
    __shared__ __align__(16) unsigned short Pt[KS][LDH];                   // weights, [query][key of the block]
    __shared__ float Dv[KS];
    const int tid = threadIdx.x, wave = tid >> 6, l = tid & 63, r = l & 15, g = l >> 4;
    const BlockCoord bc = xcd_block_coord(H);
    const int j0 = bc.x * QB, h = bc.h, b = bc.b;
    const int total = H * HD, hoff = h * HD;
    const size_t row0 = (size_t)b * s;
    const int kj = j0 + 16 * wave + r;   // this lane's key (B-operand / accumulator column)
    const unsigned short *awb = attn_w + ((size_t)(b * H + h) * s) * ws;
    const float *dvb = dvec + (size_t)(b * H + h) * s;

    bf16x4 vf[4];
#pragma unroll
    for (int sp = 0; sp < 4; sp++) {
        vf[sp] = bf16x4{0, 0, 0, 0};
        if (kj < s) vf[sp] = *reinterpret_cast<const bf16x4 *>(v + (row0 + kj) * total + hoff + 16 * sp + 4 * g);
    }
    f32x4 dk[4], dv[4];
#pragma unroll
    for (int i = 0; i < 4; i++) { dk[i] = f32x4{0.f, 0.f, 0.f, 0.f}; dv[i] = f32x4{0.f, 0.f, 0.f, 0.f}; }
    const float scale = 0.125f;
    const int t_last = min(s - 1, j0 + QB - 1 + ws - 1);

    // global -> register fetch of one stage (64 queries), issued one stage ahead of its use
    f32x4 gdo[4];
    uint4 gq[2];
    unsigned short gw[16];
    float gd = 0.f;
    const int dpair = r + 16 * (wave & 1), dd0 = 4 * g + 16 * (wave >> 1);   // dO: query pair, first dim (+32 for the second half)
    const int qpair = tid & 31, qd0 = 8 * (tid >> 5);                        // Q: query pair, first dim
    auto fetch_stage = [&](int st) {
        const int qs0 = j0 + KS * st;
        // dO: query pair (2 rows) x 4 dims per load, Q: query pair x 8 dims; pairs so that the
        // transposed tiles are written as 32-bit words without bank conflicts
#pragma unroll
        for (int cc = 0; cc < 2; cc++)
#pragma unroll
            for (int c = 0; c < 2; c++) {
                const int t = qs0 + 2 * dpair + c;
                gdo[2 * cc + c] = f32x4{0.f, 0.f, 0.f, 0.f};
                if (t < s) gdo[2 * cc + c] = *reinterpret_cast<const f32x4 *>(d_out + (row0 + t) * total + hoff + dd0 + 32 * cc);
            }
#pragma unroll
        for (int c = 0; c < 2; c++) {
            const int t = qs0 + 2 * qpair + c;
            gq[c] = make_uint4(0, 0, 0, 0);
            if (t < s) gq[c] = *reinterpret_cast<const uint4 *>(q + (row0 + t) * total + hoff + qd0);
        }
        // weights of the block's 64 keys for the stage's 64 queries: row t, slots j - ls(t)
#pragma unroll
        for (int c = 0; c < 16; c++) {
            const int t = qs0 + 4 * c + wave, key = j0 + l;
            const int slot = key - max(t + 1 - ws, 0);
            gw[c] = 0;
            if (t < s && key <= t && slot >= 0 && slot < ws) gw[c] = awb[(size_t)t * ws + slot];
        }
        gd = (tid < KS && qs0 + tid < s) ? dvb[qs0 + tid] : 0.f;
    };
    fetch_stage(0);
    for (int st = 0; st < NS; st++) {
        const int qs0 = j0 + KS * st;
        if (qs0 > t_last) break;
        __syncthreads();   // previous stage's readers are done
#pragma unroll
        for (int cc = 0; cc < 2; cc++) {
            bf16x4 hi[2], lo[2];
#pragma unroll
            for (int c = 0; c < 2; c++) {
                split4(gdo[2 * cc + c], hi[c], lo[c]);
                *reinterpret_cast<bf16x4 *>(&Dh[2 * dpair + c][dd0 + 32 * cc]) = hi[c];
                *reinterpret_cast<bf16x4 *>(&Dl[2 * dpair + c][dd0 + 32 * cc]) = lo[c];
            }
#pragma unroll
            for (int j = 0; j < 4; j++) {
                *reinterpret_cast<unsigned *>(&DhT[dd0 + 32 * cc + j][2 * dpair]) =
                    (unsigned)(unsigned short)hi[0][j] | ((unsigned)(unsigned short)hi[1][j] << 16);
                *reinterpret_cast<unsigned *>(&DlT[dd0 + 32 * cc + j][2 * dpair]) =
                    (unsigned)(unsigned short)lo[0][j] | ((unsigned)(unsigned short)lo[1][j] << 16);
            }
        }
        {
            const unsigned e[4] = {gq[0].x, gq[0].y, gq[0].z, gq[0].w};
            const unsigned o[4] = {gq[1].x, gq[1].y, gq[1].z, gq[1].w};
#pragma unroll
            for (int j = 0; j < 4; j++) {
                *reinterpret_cast<unsigned *>(&QT[qd0 + 2 * j][2 * qpair]) = (e[j] & 0xffffu) | (o[j] << 16);
                *reinterpret_cast<unsigned *>(&QT[qd0 + 2 * j + 1][2 * qpair]) = (e[j] >> 16) | (o[j] & 0xffff0000u);
            }
        }
#pragma unroll
        for (int c = 0; c < 16; c++) Pt[4 * c + wave][l] = gw[c];
        if (tid < KS) Dv[tid] = gd;
        __syncthreads();
        if (qs0 + KS <= t_last) fetch_stage(st + 1);
#pragma unroll
        for (int qt = 0; qt < 4; qt++) {
            f32x4 dw = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int sp = 0; sp < 4; sp++) {
                const bf16x4 ah = *reinterpret_cast<const bf16x4 *>(&Dh[16 * qt + r][16 * sp + 4 * g]);
                const bf16x4 al = *reinterpret_cast<const bf16x4 *>(&Dl[16 * qt + r][16 * sp + 4 * g]);
                dw = mfma16(ah, vf[sp], dw);
                dw = mfma16(al, vf[sp], dw);
            }
            // accumulator layout: rows = queries 16 qt + 4g + i, column = key r of this wave
            bf16x4 pa;
            f32x4 ds;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int qi = 16 * qt + 4 * g + i;
                const unsigned short pw = Pt[qi][16 * wave + r];
                pa[i] = (short)pw;
                ds[i] = bf2f(pw) * (dw[i] - Dv[qi]) * scale;
            }
            bf16x4 dsh, dsl;
            split4(ds, dsh, dsl);
#pragma unroll
            for (int dt = 0; dt < 4; dt++) {
                const bf16x4 bh = *reinterpret_cast<const bf16x4 *>(&DhT[16 * dt + r][16 * qt + 4 * g]);
                const bf16x4 bl = *reinterpret_cast<const bf16x4 *>(&DlT[16 * dt + r][16 * qt + 4 * g]);
                const bf16x4 bq = *reinterpret_cast<const bf16x4 *>(&QT[16 * dt + r][16 * qt + 4 * g]);
                dv[dt] = mfma16(pa, bh, dv[dt]);
                dv[dt] = mfma16(pa, bl, dv[dt]);
                dk[dt] = mfma16(dsh, bq, dk[dt]);
                dk[dt] = mfma16(dsl, bq, dk[dt]);
            }
        }
    }
    // accumulate: rows = keys 16 wave + 4g + i, column = dim 16 dt + r
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int key = j0 + 16 * wave + 4 * g + i;
        if (key >= s) continue;
        float *pk = d_k + (row0 + key) * total + hoff, *pv = d_v + (row0 + key) * total + hoff;
#pragma unroll
        for (int dt = 0; dt < 4; dt++) {
            pk[16 * dt + r] += dk[dt][i];
            pv[16 * dt + r] += dv[dt][i];
        }
    }
}

}  // namespace

bool swa_forward_mfma(const uint16_t *q, const uint16_t *k, const uint16_t *v, uint16_t *out, uint16_t *attn_weights,
                      int seq_len, int num_heads, int head_dim, int window, int batch, int n_persistent) {
    if (head_dim != HD || n_persistent != 0 || window > 512 || window < 1) return false;
    const dim3 grid((seq_len + QB - 1) / QB, num_heads, batch);
    hipLaunchKernelGGL(swa_fwd_mfma_kernel, grid, dim3(256), 0, stream(), q, k, v, out, attn_weights, seq_len,
                       num_heads, window);
    check_launch("swa_fwd_mfma_kernel");
    return true;
}

}  // namespace nlh

namespace nlh {
bool swa_backward_mfma(const uint16_t *q, const uint16_t *k, const uint16_t *v, const uint16_t *attn_weights,
                       const float *d_attn_out, float *d_q, float *d_k, float *d_v, int seq_len, int num_heads,
                       int head_dim, int window, int batch, int n_persistent) {
    if (head_dim != HD || n_persistent != 0 || window > 512 || window < 1) return false;
    float *dvec = scratch(1, (size_t)batch * num_heads * seq_len * sizeof(float));
    if (failed()) return true;
    const dim3 grid((seq_len + QB - 1) / QB, num_heads, batch);
    hipLaunchKernelGGL(swa_bwd_q_mfma_kernel, grid, dim3(256), 0, stream(), k, v, attn_weights, d_attn_out, d_q, dvec,
                       seq_len, num_heads, window);
    check_launch("swa_bwd_q_mfma_kernel");
    hipLaunchKernelGGL(swa_bwd_k_mfma_kernel, grid, dim3(256), 0, stream(), q, v, attn_weights, d_attn_out, dvec, d_k,
                       d_v, seq_len, num_heads, window);
    check_launch("swa_bwd_k_mfma_kernel");
    return true;
}
}  // namespace nlh
