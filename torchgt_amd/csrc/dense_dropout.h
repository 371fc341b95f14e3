// Shared by the two dense attention implementations (dense_attn.hip: bf16 matrix products, dense_attn_f32.hip:
// float32 arithmetic): the attention dropout that needs no mask in memory, and the float32 call descriptor.
#pragma once
#include "common.h"

namespace tgt {

// Attention dropout (models/graphormer_graph_level.py:207-209: Dropout on the softmax output).  Whether the
// probability of (graph g, head h, query q, key k) is kept is a pure function of (seed, g, h, q, k): a
// counter-based hash, so the forward, both walks of the backward and tgt_dense_attn_dropout_mask agree
// without any mask in memory.  Kept probabilities are scaled by 1 / (1 - p) like torch's Dropout.
struct DropArgs {
    uint32_t thresh;       // an element is dropped when its hash is below this (p * 2^32)
    uint32_t seed_lo, seed_hi;
    float inv_keep;        // 1 / (1 - p)
};
__host__ __device__ __forceinline__ uint32_t fmix32(uint32_t h) {
    h ^= h >> 16; h *= 0x85ebca6bu; h ^= h >> 13; h *= 0xc2b2ae35u; h ^= h >> 16;
    return h;
}
// pair = g * H + h; the row hash is formed once per query row, the key is mixed in per element
__host__ __device__ __forceinline__ uint32_t drop_row_hash(const DropArgs& da, int pair, int q) {
    return fmix32(((uint32_t)pair * 0x9e3779b1u) ^ da.seed_lo) + fmix32(((uint32_t)q * 0x85ebca77u) ^ da.seed_hi);
}
__host__ __device__ __forceinline__ bool drop_keep(const DropArgs& da, uint32_t row_hash, int k) {
    return fmix32(row_hash ^ ((uint32_t)k * 0xc2b2ae3du + 0x27d4eb2fu)) >= da.thresh;
}
inline DropArgs drop_args(float p, uint64_t seed) {
    DropArgs da{};
    const double t = (double)p * 4294967296.0;
    da.thresh = t >= 4294967295.0 ? 0xffffffffu : (uint32_t)t;
    da.seed_lo = (uint32_t)seed;
    da.seed_hi = (uint32_t)(seed >> 32);
    da.inv_keep = 1.0f / (1.0f - p);
    return da;
}

struct DenseF32Call {
    const float *q, *k, *v, *bias, *out, *dout, *lse;
    float *o_out, *o_lse, *dq, *dk, *dv, *dbias;
    int b, S, H, d;
    hipStream_t st;
    float p_drop;
    uint64_t seed;
};
// float32 arithmetic throughout (dense_attn_f32.hip)
int dense_attn_f32(const DenseF32Call& c, bool bwd);

}  // namespace tgt
