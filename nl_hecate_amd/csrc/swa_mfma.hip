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

__global__ __launch_bounds__(256) void swa_fwd_mfma_kernel(const unsigned short *__restrict__ q,
                                                           const unsigned short *__restrict__ k,
                                                           const unsigned short *__restrict__ v,
                                                           unsigned short *__restrict__ out,
                                                           unsigned short *__restrict__ attn_w, int s, int H,
                                                           int ws) {
    __shared__ __align__(16) unsigned short Ks[2][KS][LDH];   // K stage (row-major), then V^T stage [d][key]
    __shared__ __align__(16) unsigned short Pw[4][16][KS];    // per wave: normalised weights of one stage
    const int tid = threadIdx.x, wave = tid >> 6, l = tid & 63, r = l & 15, g = l >> 4;
    const int t0 = blockIdx.x * QB, h = blockIdx.y, b = blockIdx.z;
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
    load_rows(v, st_lo, stg);
#pragma unroll
    for (int st = 0; st < NS; st++) {
        if (st < st_lo) continue;
        const int buf = st & 1;
        // transposed staging: chunk = (key, 8 dims) -> Vt[dim][key]
#pragma unroll
        for (int c = 0; c < 2; c++) {
            const int chunk = tid + 256 * c, key = chunk >> 3, d0 = 8 * (chunk & 7);
            const unsigned w[4] = {stg[c].x, stg[c].y, stg[c].z, stg[c].w};
#pragma unroll
            for (int j = 0; j < 4; j++) {
                Ks[buf][d0 + 2 * j][key] = (unsigned short)(w[j] & 0xffffu);
                Ks[buf][d0 + 2 * j + 1][key] = (unsigned short)(w[j] >> 16);
            }
        }
        __syncthreads();
        if (st + 1 < NS) load_rows(v, st + 1, stg);
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
