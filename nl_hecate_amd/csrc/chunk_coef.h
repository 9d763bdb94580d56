// Gate coefficients of one chunk of the frozen-M0 chunkwise Titans / Delta rule, computed inside
// the kernels that use them (no table in HBM).
//
// With keep_t = 1 - alpha_t and the per-token map g_t = [[keep_t, eta_t], [0, eta_t]] acting on
// (weight in M, weight in S) of an earlier rank-1 term, a range of tokens composes to an upper
// triangular 2x2 map G(a..b) = g_b ... g_a = [[R, X], [0, H]] (R = prod keep, H = prod eta).  The
// coefficients of chunkwise_mm.hip are entries of such maps:
//   a_t = R(0..t), beta_t = X(0..t), h_t = H(0..t)
//   r[j][t] = R(j+1..t), bb[j][t] = H(j+1..t), c[t][j] = R(j+1..t) + X(j+1..t)      (j <= t)
//   cl_j = c[L-1][j], bl_j = bb[j][L-1], rl_j = r[j][L-1]
// Tokens beyond a short chunk's length L carry the identity map, so "L-1" is always token 63.
// A chunk is cut into four blocks of 16 tokens (one DPP row of a wave each).  One wave scans the
// maps inside the blocks (prefixes "head", suffixes "tail") and across them; every other quantity
// is a product of at most three maps, without a division (a saturated gate, keep = 0 or eta = 0,
// is an ordinary value):
//   tokens j < t in different blocks J < T:  G(j+1..t) = head_t . mid(J,T) . tail_j
//     => c[t][j] = A.R zc_j + A.X zh_j,  bb[j][t] = A.H zh_j,  r[j][t] = A.R zr_j,  A = head_t . mid(J,T)
//   tokens in the same block: a 16-step recurrence per lane (coef_diag_*).
#pragma once
#include <hip/hip_runtime.h>

namespace nlh {
namespace {

typedef float cf32x4 __attribute__((ext_vector_type(4)));

struct Map3 { float R, X, H; };   // [[R, X], [0, H]]
__device__ __forceinline__ Map3 map_identity() { return Map3{1.f, 0.f, 1.f}; }
// later . earlier
__device__ __forceinline__ Map3 compose(const Map3 &l, const Map3 &e) {
    return Map3{l.R * e.R, fmaf(l.R, e.X, l.X * e.H), l.H * e.H};
}

// Everything the consumers read, in LDS (one per chunk in flight).
struct ChunkCoef {
    float keep[64], eta[64], th[64];   // gates; beyond L: 1, 0, 0  (the scan itself uses the identity map there)
    float hR[64], hX[64], hH[64];      // head_t = G(16 T .. t)
    float zc[64], zh[64], zr[64];      // tail_j = G(j+1 .. 16 J + 15):  R + X, H, R
    float a[64], beta[64], h[64];      // G(0 .. t)
    float cl[64], bl[64], rl[64];      // G(j+1 .. 63): R + X, H, R
    float mid[6][4];                   // mid(J,T) for (0,1) (0,2) (0,3) (1,2) (1,3) (2,3): R, X, H, unused
    float last[4];                     // a_63, beta_63, h_63 (= a_L, beta_L, h_L), unused
};
__device__ __forceinline__ int mid_index(int J, int T) { return J == 0 ? T - 1 : (J == 1 ? T + 1 : 5); }

// value of lane (i - n) of the same 16-lane row, `fill` where that lane does not exist
template <int N>
__device__ __forceinline__ float row_shr(float x, float fill) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, fill),
                                                                 __builtin_bit_cast(int, x), 0x110 + N, 0xF, 0xF, false));
}
// value of lane (i + n) of the same row
template <int N>
__device__ __forceinline__ float row_shl(float x, float fill) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, fill),
                                                                 __builtin_bit_cast(int, x), 0x100 + N, 0xF, 0xF, false));
}
template <int N>
__device__ __forceinline__ Map3 map_shr(const Map3 &m) { return Map3{row_shr<N>(m.R, 1.f), row_shr<N>(m.X, 0.f), row_shr<N>(m.H, 1.f)}; }
template <int N>
__device__ __forceinline__ Map3 map_shl(const Map3 &m) { return Map3{row_shl<N>(m.R, 1.f), row_shl<N>(m.X, 0.f), row_shl<N>(m.H, 1.f)}; }
__device__ __forceinline__ float coef_readlane(float x, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), lane));
}

// One whole wave, lane = token of the chunk; alpha, theta, eta are that token's gates (any value
// beyond L).  Fills cc; the caller orders it against the readers with a barrier.
__device__ __forceinline__ void coef_scan(ChunkCoef &cc, float alpha, float theta, float eta, int L) {
    const int t = threadIdx.x & 63;
    const bool in = t < L;
    const float keep = in ? 1.f - alpha : 1.f, et = in ? eta : 0.f;
    cc.keep[t] = keep;
    cc.eta[t] = et;
    cc.th[t] = in ? theta : 0.f;
    const Map3 g = in ? Map3{keep, et, et} : map_identity();
    // prefixes inside the block: head_t = g_t ... g_(16 T)
    Map3 hd = g;
    hd = compose(hd, map_shr<1>(hd));
    hd = compose(hd, map_shr<2>(hd));
    hd = compose(hd, map_shr<4>(hd));
    hd = compose(hd, map_shr<8>(hd));
    // suffixes inside the block: sf_j = g_(16 J + 15) ... g_j; tail_j = sf_(j+1)
    Map3 sf = g;
    sf = compose(map_shl<1>(sf), sf);
    sf = compose(map_shl<2>(sf), sf);
    sf = compose(map_shl<4>(sf), sf);
    sf = compose(map_shl<8>(sf), sf);
    const Map3 tl = map_shl<1>(sf);
    // whole blocks (uniform values)
    Map3 blk[4];
#pragma unroll
    for (int b = 0; b < 4; b++)
        blk[b] = Map3{coef_readlane(hd.R, 16 * b + 15), coef_readlane(hd.X, 16 * b + 15), coef_readlane(hd.H, 16 * b + 15)};
    const Map3 m02 = blk[1], m13 = blk[2], m03 = compose(blk[2], blk[1]);
    const Map3 pre1 = blk[0], pre2 = compose(blk[1], blk[0]), pre3 = compose(blk[2], pre2);
    const Map3 post2 = blk[3], post1 = compose(blk[3], blk[2]), post0 = compose(post1, blk[1]);
    const int T = t >> 4;
    const Map3 pre = T == 0 ? map_identity() : (T == 1 ? pre1 : (T == 2 ? pre2 : pre3));
    const Map3 post = T == 3 ? map_identity() : (T == 2 ? post2 : (T == 1 ? post1 : post0));
    const Map3 pf = compose(hd, pre), sx = compose(post, tl);
    cc.hR[t] = hd.R; cc.hX[t] = hd.X; cc.hH[t] = hd.H;
    cc.zc[t] = tl.R + tl.X; cc.zh[t] = tl.H; cc.zr[t] = tl.R;
    cc.a[t] = pf.R; cc.beta[t] = pf.X; cc.h[t] = pf.H;
    cc.cl[t] = sx.R + sx.X; cc.bl[t] = sx.H; cc.rl[t] = sx.R;
    if (t == 63) { cc.last[0] = pf.R; cc.last[1] = pf.X; cc.last[2] = pf.H; cc.last[3] = 0.f; }
    if (t < 6) {
        const Map3 id = map_identity();
        const Map3 m = t == 1 ? m02 : (t == 2 ? m03 : (t == 4 ? m13 : id));
        cc.mid[t][0] = m.R; cc.mid[t][1] = m.X; cc.mid[t][2] = m.H; cc.mid[t][3] = 0.f;
    }
}

// Which of c, bb, r a tile function returns.
enum CoefKind { COEF_C = 0, COEF_BB = 1, COEF_R = 2 };

// Tile (T, J) in "token-major" order: element i of lane l is the coefficient between
// t = 16 T + 4 (l / 16) + i (row) and j = 16 J + l % 16 (column); zero unless j <= t < L.
template <int KIND>
__device__ __forceinline__ cf32x4 coef_tile_tj(const ChunkCoef &cc, int T, int J, int L) {
    const int l = threadIdx.x & 63, g = l >> 4, c16 = l & 15;
    cf32x4 out = {0.f, 0.f, 0.f, 0.f};
    if (J > T) return out;
    const int j = 16 * J + c16;
    if (J < T) {
        const float *md = cc.mid[mid_index(J, T)];
        const float mR = md[0], mX = md[1], mH = md[2];
        const float zc = cc.zc[j], zh = cc.zh[j], zr = cc.zr[j];
        const cf32x4 hR = *reinterpret_cast<const cf32x4 *>(cc.hR + 16 * T + 4 * g);
        const cf32x4 hX = *reinterpret_cast<const cf32x4 *>(cc.hX + 16 * T + 4 * g);
        const cf32x4 hH = *reinterpret_cast<const cf32x4 *>(cc.hH + 16 * T + 4 * g);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float aR = hR[i] * mR;
            float x;
            if (KIND == COEF_C) x = fmaf(aR, zc, fmaf(hR[i], mX, hX[i] * mH) * zh);
            else if (KIND == COEF_BB) x = hH[i] * mH * zh;
            else x = aR * zr;
            out[i] = (16 * T + 4 * g + i < L && j < L) ? x : 0.f;
        }
        return out;
    }
    // same block: run the recurrence from token j upwards, keep the steps this lane owns
    float b = 1.f, c = 1.f, r = 1.f;
#pragma unroll
    for (int u = 0; u < 16; u++) {
        const float kp = cc.keep[16 * T + u], et = cc.eta[16 * T + u];
        const bool after = u > c16;
        if (KIND != COEF_R) b *= after ? et : 1.f;
        if (KIND == COEF_C) c = after ? fmaf(kp, c, b) : c;
        if (KIND == COEF_R) r *= after ? kp : 1.f;
        if ((u >> 2) == g) {
            const float x = KIND == COEF_C ? c : (KIND == COEF_BB ? b : r);
            out[u & 3] = (u >= c16 && 16 * T + u < L && j < L) ? x : 0.f;
        }
    }
    return out;
}

// Tile (J, T) in "source-major" order: element i of lane l is the coefficient between
// j = 16 J + 4 (l / 16) + i (row) and t = 16 T + l % 16 (column); zero unless j <= t < L.
template <int KIND>
__device__ __forceinline__ cf32x4 coef_tile_jt(const ChunkCoef &cc, int J, int T, int L) {
    const int l = threadIdx.x & 63, g = l >> 4, c16 = l & 15;
    cf32x4 out = {0.f, 0.f, 0.f, 0.f};
    if (J > T) return out;
    const int t = 16 * T + c16;
    if (J < T) {
        const float *md = cc.mid[mid_index(J, T)];
        const float mR = md[0], mX = md[1], mH = md[2];
        const float hR = cc.hR[t], hX = cc.hX[t], hH = cc.hH[t];
        const float aR = hR * mR, aX = fmaf(hR, mX, hX * mH), aH = hH * mH;
        const cf32x4 zc = *reinterpret_cast<const cf32x4 *>(cc.zc + 16 * J + 4 * g);
        const cf32x4 zh = *reinterpret_cast<const cf32x4 *>(cc.zh + 16 * J + 4 * g);
        const cf32x4 zr = *reinterpret_cast<const cf32x4 *>(cc.zr + 16 * J + 4 * g);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float x;
            if (KIND == COEF_C) x = fmaf(aR, zc[i], aX * zh[i]);
            else if (KIND == COEF_BB) x = aH * zh[i];
            else x = aR * zr[i];
            out[i] = (t < L && 16 * J + 4 * g + i < L) ? x : 0.f;
        }
        return out;
    }
    // same block: four recurrences (sources j = 4 g + i), each from j + 1 up to this lane's t
    float b[4] = {1.f, 1.f, 1.f, 1.f}, c[4] = {1.f, 1.f, 1.f, 1.f}, r[4] = {1.f, 1.f, 1.f, 1.f};
#pragma unroll
    for (int u = 1; u < 16; u++) {
        const float kp = cc.keep[16 * T + u], et = cc.eta[16 * T + u];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const bool on = u > 4 * g + i && u <= c16;
            if (KIND != COEF_R) b[i] *= on ? et : 1.f;
            if (KIND == COEF_C) c[i] = on ? fmaf(kp, c[i], b[i]) : c[i];
            if (KIND == COEF_R) r[i] *= on ? kp : 1.f;
        }
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float x = KIND == COEF_C ? c[i] : (KIND == COEF_BB ? b[i] : r[i]);
        out[i] = (4 * g + i <= c16 && t < L && 16 * J + 4 * g + i < L) ? x : 0.f;
    }
    return out;
}


// ── Coefficient tables written to HBM by a pre-pass (one wave per chunk) ──
// The vectors of a chunk from two scans of composed maps instead of 64-step loops:
//   a, beta, h = R, X, H of G(0..t);  cl, bl = R + X, H of G(t+1..63)   (tokens beyond L: identity map)
struct ChunkVectors { float a, beta, h, cl, bl; };
__device__ __forceinline__ ChunkVectors coef_vectors(float keep, float et, bool in) {
    const int t = threadIdx.x & 63;
    const Map3 g = in ? Map3{keep, et, et} : map_identity();
    Map3 hd = g;
    hd = compose(hd, map_shr<1>(hd));
    hd = compose(hd, map_shr<2>(hd));
    hd = compose(hd, map_shr<4>(hd));
    hd = compose(hd, map_shr<8>(hd));
    Map3 sf = g;
    sf = compose(map_shl<1>(sf), sf);
    sf = compose(map_shl<2>(sf), sf);
    sf = compose(map_shl<4>(sf), sf);
    sf = compose(map_shl<8>(sf), sf);
    const Map3 tl = map_shl<1>(sf);
    Map3 blk[4];
#pragma unroll
    for (int b = 0; b < 4; b++)
        blk[b] = Map3{coef_readlane(hd.R, 16 * b + 15), coef_readlane(hd.X, 16 * b + 15), coef_readlane(hd.H, 16 * b + 15)};
    const Map3 pre1 = blk[0], pre2 = compose(blk[1], blk[0]), pre3 = compose(blk[2], pre2);
    const Map3 post2 = blk[3], post1 = compose(blk[3], blk[2]), post0 = compose(post1, blk[1]);
    const int T = t >> 4;
    const Map3 pre = T == 0 ? map_identity() : (T == 1 ? pre1 : (T == 2 ? pre2 : pre3));
    const Map3 post = T == 3 ? map_identity() : (T == 2 ? post2 : (T == 1 ? post1 : post0));
    const Map3 pf = compose(hd, pre), sx = compose(post, tl);
    return ChunkVectors{pf.R, pf.X, pf.H, sx.R + sx.X, sx.H};
}

// stage[t * LD + j] = scale_j c[t][j] for j <= t < L and zero elsewhere (64 rows of LD floats, LD a multiple of 4,
// and one spare row behind them).
// One wave, lane = j.  Lane j walks t = j, j + 1, .. on its own: at step i every lane multiplies (no lane waits
// for its column to start), the gates of token j + i come from LDS (gk, ge: 128 floats each, identity from 64
// on) at an immediate offset, and the destination is base + i * LD.  A step is two multiply-adds and a store
// per lane, against a dozen instructions when the lanes advance through t together.
template <int LD, bool SCALED>
__device__ __forceinline__ void coef_table_columns(float *stage, float *gk, float *ge, float keep, float et,
                                                   float scale, int L) {
    const int j = threadIdx.x & 63;
    gk[j] = keep; gk[64 + j] = 1.f;   // the caller passes keep = 1, eta = 0 beyond L
    ge[j] = et;   ge[64 + j] = 0.f;
    for (int e = j; e < 64 * LD / 4; e += 64) reinterpret_cast<cf32x4 *>(stage)[e] = cf32x4{0.f, 0.f, 0.f, 0.f};
    // the gates of tokens j + 1 .. j + 63 in registers (requested in one go: no step waits for LDS), and every
    // lane stores at every step (a lane whose column has ended stores to a spare row): no branch inside the walk
    float kk[64], ee[64];
#pragma unroll
    for (int i = 1; i < 64; i++) { kk[i] = gk[j + i]; ee[i] = ge[j + i]; }
    float b = 1.f, c = 1.f;
    float *dst = stage + j * (LD + 1), *spare = stage + 64 * LD + j;
    const bool jv = j < L;
    dst[0] = jv ? (SCALED ? scale : 1.f) : 0.f;
    if (L == 64) {
#pragma unroll
        for (int i = 1; i < 64; i++) {
            b *= ee[i];
            c = fmaf(kk[i], c, b);
            *(j < 64 - i ? dst + i * LD : spare) = SCALED ? scale * c : c;
        }
    } else {
#pragma unroll
        for (int i = 1; i < 64; i++) {
            b *= ee[i];
            c = fmaf(kk[i], c, b);
            *(j < 64 - i ? dst + i * LD : spare) = (jv && j < L - i) ? (SCALED ? scale * c : c) : 0.f;
        }
    }
}

}  // namespace
}  // namespace nlh
