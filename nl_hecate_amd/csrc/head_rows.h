// Where the row of token t of chain c sits in a tensor of per-token head vectors (y, dY):
// base + offset(c) + t * row_stride floats.  Head-major [chains, s, hd] is what the rule's entry
// points take by default; token-major [levels, bs, s, nh * hd] is what a layer's projections
// produce and consume, with chain c = (level, batch element, head) and, for an upstream gradient
// that every level shares, a level stride of zero.
#pragma once
#include <limits.h>
#include <stddef.h>

#include <hip/hip_runtime.h>

namespace nlh {

struct HeadRows {
    long long level_stride, batch_stride, head_stride, row_stride;
    int per_level, nh;
    __host__ __device__ size_t offset(int c) const {
        const int lv = c / per_level, r = c - lv * per_level;
        return (size_t)lv * level_stride + (size_t)(r / nh) * batch_stride + (size_t)(r % nh) * head_stride;
    }
};

inline HeadRows head_major_rows(int s, int hd) { return HeadRows{0, (long long)s * hd, 0, hd, INT_MAX, 1}; }

// chains_per_level = bs * nh chains per level; per_level: every level has its own [bs, s, nh * hd] block
inline HeadRows token_major_rows(int s, int hd, int nh, int chains_per_level, bool per_level) {
    const long long d = (long long)nh * hd;
    return HeadRows{per_level ? (long long)(chains_per_level / nh) * s * d : 0, (long long)s * d, hd, d,
                    chains_per_level, nh};
}

}  // namespace nlh
