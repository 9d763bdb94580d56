// On-device check of the cross-lane primitives against host arithmetic.
#include <hip/hip_runtime.h>

#include <stdio.h>

#include <vector>

#include "../../include/nl_hecate_ffi.h"
#include "chunk_coef.h"
#include "lane_ops.h"
#include "runtime.h"

namespace nlh {

// out[0..5][64]: group sums for G=4,16,64; stride sums for LPR=16, 2; swapadd32(a,b)
__global__ void lane_ops_kernel(const float *in, const float *in2, float *out) {
    int l = threadIdx.x;
    float x = in[l], y = in2[l];
    out[0 * 64 + l] = group_allreduce<4>(x);
    out[1 * 64 + l] = group_allreduce<16>(x);
    out[2 * 64 + l] = group_allreduce<64>(x);
    out[3 * 64 + l] = stride_allreduce<16>(x);
    out[4 * 64 + l] = stride_allreduce<2>(x);
    out[5 * 64 + l] = swapadd32(x, y);
    out[6 * 64 + l] = swapadd16(x, y);
    out[7 * 64 + l] = stride_allreduce<8>(x);
    out[8 * 64 + l] = group_allreduce<8>(x);
    out[9 * 64 + l] = group_allreduce<32>(x);
    {
        // column reduce-scatter and batched wave reduction
        float4 q4 = make_float4(x, y, x + y, x - y), k4 = make_float4(2.f * x, 3.f * y, y, x);
        float fq, fk;
        colreduce4x2(q4, k4, fq, fk);
        out[12 * 64 + l] = fq;
        out[13 * 64 + l] = fk;
        float v[8], r[2];
#pragma unroll
        for (int i = 0; i < 8; i++) v[i] = x * (float)(i + 1) + (float)i;
        wave_reduce_scatter<8>(v, r);
        out[14 * 64 + l] = r[0];
        out[15 * 64 + l] = r[1];
    }
    // The row-exchange results are read by the very next VALU instruction in
    // lane_ops.h (no padding after the swap); these two probes pin that this
    // is safe.  (A VALU write right BEFORE a swap does need 2 wait states.)
    {
        float a = x, b = y;
        asm volatile("s_nop 4\n\tv_permlane32_swap_b32 %0, %1\n\tv_add_f32 %0, %0, %1"
                     : "+v"(a), "+v"(b));
        out[10 * 64 + l] = a;
        a = x; b = y;
        asm volatile("s_nop 4\n\tv_permlane16_swap_b32 %0, %1\n\tv_add_f32 %0, %0, %1"
                     : "+v"(a), "+v"(b));
        out[11 * 64 + l] = a;
    }
}

}  // namespace nlh

extern "C" int nlh_selftest_lane_ops(void) {
    using namespace nlh;
    const int NT = 16;
    std::vector<float> a(64), b(64), o(NT * 64);
    // small integers: every sum is exact, so results compare with ==
    for (int i = 0; i < 64; i++) { a[i] = (float)((i * 37 + 11) % 23 - 9); b[i] = (float)((i * 53 + 5) % 31 - 13); }
    float *din, *din2, *dout;
    if (hipMalloc(&din, 256) != hipSuccess || hipMalloc(&din2, 256) != hipSuccess ||
        hipMalloc(&dout, NT * 256) != hipSuccess) return -1;
    (void)hipMemcpy(din, a.data(), 256, hipMemcpyHostToDevice);
    (void)hipMemcpy(din2, b.data(), 256, hipMemcpyHostToDevice);
    hipLaunchKernelGGL(lane_ops_kernel, dim3(1), dim3(64), 0, stream(), din, din2, dout);
    if (hipDeviceSynchronize() != hipSuccess) return -2;
    (void)hipMemcpy(o.data(), dout, NT * 256, hipMemcpyDeviceToHost);
    (void)hipFree(din); (void)hipFree(din2); (void)hipFree(dout);
    int bad = 0;
    std::vector<float> want(NT * 64);
    auto gsum = [&](int l, int G) { float s = 0; for (int j = (l / G) * G; j < (l / G + 1) * G; j++) s += a[j]; return s; };
    auto ssum = [&](int l, int LPR) { float s = 0; for (int j = l % LPR; j < 64; j += LPR) s += a[j]; return s; };
    for (int l = 0; l < 64; l++) {
        want[0 * 64 + l] = gsum(l, 4);
        want[1 * 64 + l] = gsum(l, 16);
        want[2 * 64 + l] = gsum(l, 64);
        want[3 * 64 + l] = ssum(l, 16);
        want[4 * 64 + l] = ssum(l, 2);
        want[5 * 64 + l] = l < 32 ? a[l] + a[l + 32] : b[l - 32] + b[l];
        int row = l / 16, c = l % 16;
        want[6 * 64 + l] = (row % 2 == 0) ? a[row * 16 + c] + a[(row + 1) * 16 + c]
                                          : b[(row - 1) * 16 + c] + b[row * 16 + c];
        want[7 * 64 + l] = ssum(l, 8);
        want[8 * 64 + l] = gsum(l, 8);
        want[9 * 64 + l] = gsum(l, 32);
        {
            int g = l / 16, cb = l % 16;
            float sq = 0, sk = 0;
            for (int gg = 0; gg < 4; gg++) {
                float xa = a[gg * 16 + cb], yb = b[gg * 16 + cb];
                float qv[4] = {xa, yb, xa + yb, xa - yb}, kv[4] = {2.f * xa, 3.f * yb, yb, xa};
                sq += qv[g];
                sk += kv[g];
            }
            want[12 * 64 + l] = sq;
            want[13 * 64 + l] = sk;
            float suma = 0;
            for (int j = 0; j < 64; j++) suma += a[j];
            for (int n = 0; n < 2; n++) {
                int i = 4 * n + 2 * (g & 1) + (g >> 1);
                want[(14 + n) * 64 + l] = suma * (float)(i + 1) + 64.f * (float)i;
            }
        }
        want[10 * 64 + l] = want[5 * 64 + l];
        want[11 * 64 + l] = want[6 * 64 + l];
    }
    for (int t = 0; t < NT; t++) {
        int nb = 0;
        for (int l = 0; l < 64; l++) nb += o[t * 64 + l] != want[t * 64 + l];
        if (nb) {
            fprintf(stderr, "lane-op selftest %d: %d lanes differ; got/want:", t, nb);
            for (int l = 0; l < 64; l++) fprintf(stderr, " %g/%g", o[t * 64 + l], want[t * 64 + l]);
            fprintf(stderr, "\n");
        }
        bad += nb;
    }
    return bad;
}

namespace nlh {
// c, bb, r of one chunk from both tile generators, as dense [kind][t][j] tables, and the vectors.
__global__ void chunk_coef_kernel(const float *alpha, const float *theta, const float *eta, int L, float *tj,
                                  float *jt, float *vecs) {
    __shared__ ChunkCoef cc;
    const int l = threadIdx.x, g = l >> 4, c16 = l & 15;
    coef_scan(cc, alpha[l], theta[l], eta[l], L);
    __syncthreads();
    for (int T = 0; T < 4; T++)
        for (int J = 0; J < 4; J++) {
            const cf32x4 a[3] = {coef_tile_tj<COEF_C>(cc, T, J, L), coef_tile_tj<COEF_BB>(cc, T, J, L),
                                 coef_tile_tj<COEF_R>(cc, T, J, L)};
            const cf32x4 b[3] = {coef_tile_jt<COEF_C>(cc, J, T, L), coef_tile_jt<COEF_BB>(cc, J, T, L),
                                 coef_tile_jt<COEF_R>(cc, J, T, L)};
            for (int kd = 0; kd < 3; kd++)
                for (int i = 0; i < 4; i++) {
                    tj[(kd * 64 + 16 * T + 4 * g + i) * 64 + 16 * J + c16] = a[kd][i];
                    jt[(kd * 64 + 16 * T + c16) * 64 + 16 * J + 4 * g + i] = b[kd][i];
                }
        }
    const float *src[9] = {cc.a, cc.beta, cc.h, cc.cl, cc.bl, cc.rl, cc.keep, cc.eta, cc.th};
    for (int v = 0; v < 9; v++) vecs[v * 64 + l] = src[v][l];
    if (l < 3) vecs[9 * 64 + l] = cc.last[l];
}
}  // namespace nlh

// tj, jt: [3][64][64] (c, bb, r indexed [t][j]); vecs: [9][64] a, beta, h, cl, bl, rl, keep, eta, theta, then a_L, beta_L, h_L
extern "C" int nlh_selftest_chunk_coef(const float *alpha, const float *theta, const float *eta, int L, float *tj,
                                       float *jt, float *vecs) {
    using namespace nlh;
    if (L < 1 || L > 64) return -1;
    hipLaunchKernelGGL(chunk_coef_kernel, dim3(1), dim3(64), 0, stream(), alpha, theta, eta, L, tj, jt, vecs);
    return hipGetLastError() == hipSuccess ? 0 : -2;
}

namespace nlh {
// The helpers of the coefficient pre-passes on one chunk: table[t][j] = theta-free c[t][j] and, with scale = -theta_j,
// the forward's W[t][j]; vecs [5][64] = a, beta, h, cl, bl of token (lane).
__global__ void chunk_coef_prepass_kernel(const float *alpha, const float *theta, const float *eta, int L,
                                          float *table, float *table_scaled, float *vecs) {
    constexpr int LD = 68;
    __shared__ __align__(16) float stage[65 * LD];
    __shared__ float gk[128], ge[128];
    const int l = threadIdx.x;
    const bool in = l < L;
    const float keep = in ? 1.f - alpha[l] : 1.f, et = in ? eta[l] : 0.f, nth = in ? -theta[l] : 0.f;
    const ChunkVectors cv = coef_vectors(keep, et, in);
    vecs[0 * 64 + l] = cv.a;
    vecs[1 * 64 + l] = cv.beta;
    vecs[2 * 64 + l] = cv.h;
    vecs[3 * 64 + l] = cv.cl;
    vecs[4 * 64 + l] = cv.bl;
    coef_table_columns<LD, false>(stage, gk, ge, keep, et, 1.f, L);
    for (int t = 0; t < 64; t++) table[t * 64 + l] = stage[t * LD + l];
    coef_table_columns<LD, true>(stage, gk, ge, keep, et, nth, L);
    for (int t = 0; t < 64; t++) table_scaled[t * 64 + l] = stage[t * LD + l];
}
}  // namespace nlh

extern "C" int nlh_selftest_chunk_coef_prepass(const float *alpha, const float *theta, const float *eta, int L,
                                               float *table, float *table_scaled, float *vecs) {
    using namespace nlh;
    if (L < 1 || L > 64) return -1;
    hipLaunchKernelGGL(chunk_coef_prepass_kernel, dim3(1), dim3(64), 0, stream(), alpha, theta, eta, L, table,
                       table_scaled, vecs);
    return hipGetLastError() == hipSuccess ? 0 : -2;
}
