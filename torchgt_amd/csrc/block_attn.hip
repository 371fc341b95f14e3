// Block path: attention over a list of dense 16 x 16 tiles plus a remainder of
// ordinary edges, one softmax per destination.
//
// The reference's cluster reordering replaces the edges of every partition pair
// by dense bs x bs blocks of (source, destination) pairs (gt_sp/utils.py:284-299,
// create_pairs :218-220) and then feeds the expanded edge list to the same
// sparse_attention (attn_module.py:133-189).  Here a block is never expanded: a
// tile (r0, c0) stands for the 256 edges a -> b, a in [r0, r0+16), b in
// [c0, c0+16).  Its scores are one 16x16 matrix product per head on the matrix
// cores (v_mfma_f32_16x16x16_bf16_1k, K and V rows of the tile read once for 16
// destinations), and because the reference's softmax has no max subtraction the
// tile sums (sum w v, Z) simply add to the sums of the remaining edges: the tile
// kernels leave fp32 partial sums per node and the sparse kernels add them when
// they write the row (forward) or the gradient row (backward).
//
// Layouts of the matrix instruction (lane l, col = l % 16, kq = l / 16):
//   A 16x16: A[col][4kq .. 4kq+3]      B 16x16: B[4kq .. 4kq+3][col]
//   C 16x16: register r holds C[4kq + r][col]
// Scores are formed transposed (rows = sources, col = destination) so that the
// weights sit in the B layout of the next product.
#include "common.h"
#include <algorithm>
#include <vector>
#include <new>

namespace tgt {

typedef short bshort4 __attribute__((ext_vector_type(4)));
typedef float bfloat4 __attribute__((ext_vector_type(4)));
struct tbf16 { uint16_t x; };

__device__ __forceinline__ short t_f2bf(float f) {
    const __bf16 b = static_cast<__bf16>(f);
    return __builtin_bit_cast(short, b);
}
__device__ __forceinline__ bshort4 t_ld4(const tbf16* p) { return *reinterpret_cast<const bshort4*>(p); }
__device__ __forceinline__ bshort4 t_ld4(const float* p) {
    const bfloat4 f = *reinterpret_cast<const bfloat4*>(p);
    bshort4 r;
    r.x = t_f2bf(f.x); r.y = t_f2bf(f.y); r.z = t_f2bf(f.z); r.w = t_f2bf(f.w);
    return r;
}
__device__ __forceinline__ short t_ld1(const tbf16* p) { return (short)p->x; }
__device__ __forceinline__ short t_ld1(const float* p) { return t_f2bf(*p); }
__device__ __forceinline__ bshort4 t_zero4() { bshort4 z; z.x = 0; z.y = 0; z.z = 0; z.w = 0; return z; }
__device__ __forceinline__ bfloat4 t_zerof() { bfloat4 z; z.x = 0.f; z.y = 0.f; z.z = 0.f; z.w = 0.f; return z; }
__device__ __forceinline__ bfloat4 mfma16(bshort4 a, bshort4 b, bfloat4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ float t_clamp5(float x) { return x < -5.0f ? -5.0f : (x > 5.0f ? 5.0f : x); }
__device__ __forceinline__ bshort4 t_pack(const float (&x)[4]) {
    bshort4 r;
    r.x = t_f2bf(x[0]); r.y = t_f2bf(x[1]); r.z = t_f2bf(x[2]); r.w = t_f2bf(x[3]);
    return r;
}
// column `c` of four consecutive node rows starting at `row0` (the transposed operand)
template <typename T>
__device__ __forceinline__ bshort4 t_ld_col(const T* __restrict__ X, int row0, int h, int H, int D, int c, bool ok) {
    bshort4 r = t_zero4();
    if (ok) {
        r.x = t_ld1(X + ((int64_t)(row0 + 0) * H + h) * D + c);
        r.y = t_ld1(X + ((int64_t)(row0 + 1) * H + h) * D + c);
        r.z = t_ld1(X + ((int64_t)(row0 + 2) * H + h) * D + c);
        r.w = t_ld1(X + ((int64_t)(row0 + 3) * H + h) * D + c);
    }
    return r;
}

constexpr int kTile = 16;

// One wave per group of tiles that share their 16 destinations: sum w v and Z of the tiles.
template <typename T, int D>
__global__ __launch_bounds__(64) void k_tile_fwd(const int32_t* __restrict__ grp_c0, const int32_t* __restrict__ grp_off,
                                                 const int32_t* __restrict__ tile_r0, const T* __restrict__ Q,
                                                 const T* __restrict__ K, const T* __restrict__ V,
                                                 float* __restrict__ acc, float* __restrict__ Zp, int H,
                                                 float inv_scale) {
    const int g = blockIdx.x, lane = threadIdx.x;
    const int col = lane & 15, kq = lane >> 4;
    const bool kval = kq * 4 < D;
    const int c0 = grp_c0[g], t0 = grp_off[g], t1 = grp_off[g + 1];
    for (int h = 0; h < H; ++h) {
        bshort4 bq = t_zero4();
        if (kval) bq = t_ld4(Q + ((int64_t)(c0 + col) * H + h) * D + kq * 4);
        bfloat4 o = t_zerof();
        float z = 0.f;
        for (int t = t0; t < t1; ++t) {
            const int r0 = tile_r0[t];
            bshort4 ak = t_zero4();
            if (kval) ak = t_ld4(K + ((int64_t)(r0 + col) * H + h) * D + kq * 4);
            const bfloat4 sc = mfma16(ak, bq, t_zerof());          // S^T[source 4kq+r][destination col]
            float w[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                w[r] = __expf(t_clamp5(sc[r] * inv_scale));
                z += w[r];
            }
            const bshort4 av = t_ld_col<T>(V, r0 + 4 * kq, h, H, D, col, col < D);
            o = mfma16(av, t_pack(w), o);                          // O^T[dd 4kq+r][destination col]
        }
        z += __shfl_xor(z, 16);
        z += __shfl_xor(z, 32);
        if (kval) *reinterpret_cast<bfloat4*>(acc + ((int64_t)(c0 + col) * H + h) * D + kq * 4) = o;
        if (kq == 0) Zp[(int64_t)(c0 + col) * H + h] = z;
    }
}

// Same grouping: dQ of the tiles.  nd[i,h] = (1/(Z+eps), dout.out) of the FINAL output.
template <typename T, int D>
__global__ __launch_bounds__(64) void k_tile_bwd_dst(const int32_t* __restrict__ grp_c0, const int32_t* __restrict__ grp_off,
                                                     const int32_t* __restrict__ tile_r0, const T* __restrict__ Q,
                                                     const T* __restrict__ K, const T* __restrict__ V,
                                                     const T* __restrict__ dO, const float2* __restrict__ nd,
                                                     float* __restrict__ dq_part, int H, float inv_scale) {
    const int g = blockIdx.x, lane = threadIdx.x;
    const int col = lane & 15, kq = lane >> 4;
    const bool kval = kq * 4 < D;
    const int c0 = grp_c0[g], t0 = grp_off[g], t1 = grp_off[g + 1];
    for (int h = 0; h < H; ++h) {
        bshort4 bq = t_zero4(), bg = t_zero4();
        if (kval) {
            bq = t_ld4(Q + ((int64_t)(c0 + col) * H + h) * D + kq * 4);
            bg = t_ld4(dO + ((int64_t)(c0 + col) * H + h) * D + kq * 4);
        }
        const float2 ndv = nd[(int64_t)(c0 + col) * H + h];
        bfloat4 dq = t_zerof();
        for (int t = t0; t < t1; ++t) {
            const int r0 = tile_r0[t];
            bshort4 ak = t_zero4(), av = t_zero4();
            if (kval) {
                ak = t_ld4(K + ((int64_t)(r0 + col) * H + h) * D + kq * 4);
                av = t_ld4(V + ((int64_t)(r0 + col) * H + h) * D + kq * 4);
            }
            const bfloat4 sc = mfma16(ak, bq, t_zerof());          // S^T[source][destination]
            const bfloat4 dp = mfma16(av, bg, t_zerof());          // dP^T = V dout^T
            float md[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float raw = sc[r] * inv_scale;
                const float wv = __expf(t_clamp5(raw));
                const float dS = wv * ndv.x * (dp[r] - ndv.y);
                md[r] = ((raw >= -5.0f) & (raw <= 5.0f)) ? dS : 0.f;
            }
            const bshort4 akT = t_ld_col<T>(K, r0 + 4 * kq, h, H, D, col, col < D);
            dq = mfma16(akT, t_pack(md), dq);                      // dQ^T[dd][destination] += K^T (m dS)^T
        }
        if (kval) {
            bfloat4 o;
            o.x = dq.x * inv_scale; o.y = dq.y * inv_scale; o.z = dq.z * inv_scale; o.w = dq.w * inv_scale;
            *reinterpret_cast<bfloat4*>(dq_part + ((int64_t)(c0 + col) * H + h) * D + kq * 4) = o;
        }
    }
}

// One wave per group of tiles that share their 16 SOURCES: dK and dV of the tiles.
template <typename T, int D>
__global__ __launch_bounds__(64) void k_tile_bwd_src(const int32_t* __restrict__ grp_r0, const int32_t* __restrict__ grp_off,
                                                     const int32_t* __restrict__ tile_c0, const T* __restrict__ Q,
                                                     const T* __restrict__ K, const T* __restrict__ V,
                                                     const T* __restrict__ dO, const float2* __restrict__ nd,
                                                     float* __restrict__ dk_part, float* __restrict__ dv_part, int H,
                                                     float inv_scale) {
    const int g = blockIdx.x, lane = threadIdx.x;
    const int col = lane & 15, kq = lane >> 4;
    const bool kval = kq * 4 < D;
    const int r0 = grp_r0[g], t0 = grp_off[g], t1 = grp_off[g + 1];
    for (int h = 0; h < H; ++h) {
        bshort4 bk = t_zero4(), bv = t_zero4();
        if (kval) {
            bk = t_ld4(K + ((int64_t)(r0 + col) * H + h) * D + kq * 4);
            bv = t_ld4(V + ((int64_t)(r0 + col) * H + h) * D + kq * 4);
        }
        bfloat4 dk = t_zerof(), dv = t_zerof();
        for (int t = t0; t < t1; ++t) {
            const int c0 = tile_c0[t];
            bshort4 aq = t_zero4(), ag = t_zero4();
            if (kval) {
                aq = t_ld4(Q + ((int64_t)(c0 + col) * H + h) * D + kq * 4);
                ag = t_ld4(dO + ((int64_t)(c0 + col) * H + h) * D + kq * 4);
            }
            const bfloat4 sc = mfma16(aq, bk, t_zerof());          // S[destination 4kq+r][source col]
            const bfloat4 dp = mfma16(ag, bv, t_zerof());          // dP = dout V^T
            float pw[4], md[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float2 ndv = nd[(int64_t)(c0 + 4 * kq + r) * H + h];
                const float raw = sc[r] * inv_scale;
                const float p = __expf(t_clamp5(raw)) * ndv.x;
                const float dS = p * (dp[r] - ndv.y);
                pw[r] = p;
                md[r] = ((raw >= -5.0f) & (raw <= 5.0f)) ? dS : 0.f;
            }
            const bshort4 agT = t_ld_col<T>(dO, c0 + 4 * kq, h, H, D, col, col < D);
            const bshort4 aqT = t_ld_col<T>(Q, c0 + 4 * kq, h, H, D, col, col < D);
            dv = mfma16(agT, t_pack(pw), dv);                      // dV^T[dd][source] += dout^T p
            dk = mfma16(aqT, t_pack(md), dk);                      // dK^T[dd][source] += Q^T (m dS)
        }
        if (kval) {
            bfloat4 o;
            o.x = dk.x * inv_scale; o.y = dk.y * inv_scale; o.z = dk.z * inv_scale; o.w = dk.w * inv_scale;
            *reinterpret_cast<bfloat4*>(dk_part + ((int64_t)(r0 + col) * H + h) * D + kq * 4) = o;
            *reinterpret_cast<bfloat4*>(dv_part + ((int64_t)(r0 + col) * H + h) * D + kq * 4) = dv;
        }
    }
}

}  // namespace tgt

// Tiles grouped by destination block and by source block.
struct tgt_tiles {
    int64_t N = 0, T = 0;
    int32_t n_dst_groups = 0, n_src_groups = 0;
    tgt::DevBuf dst_c0, dst_off, dst_r0;     // [G], [G+1], [T]
    tgt::DevBuf src_r0, src_off, src_c0;     // [Gs], [Gs+1], [T]
    tgt::DevBuf cover_dst, cover_src;        // [N] bytes
};

namespace tgt {

static inline int64_t a256(int64_t x) { return (x + 255) & ~(int64_t)255; }

struct BlockWs { int64_t acc, Z, dq, dk, dv, sparse, total; };
static BlockWs block_ws(const tgt_tiles* tl, const tgt_plan* plan, int H, int d) {
    const int64_t nhd = a256(tl->N * H * d * 4), nh = a256(tl->N * H * 4);
    BlockWs w;
    w.acc = 0;
    w.Z = w.acc + nhd;
    w.dq = w.Z + nh;
    w.dk = w.dq + nhd;
    w.dv = w.dk + nhd;
    w.sparse = w.dv + nhd;
    w.total = w.sparse + tgt_sparse_attn_workspace_bytes(plan, H, d);
    return w;
}

// group (key, other) pairs by key; keys of different groups must be >= 16 apart
static int group_tiles(const std::vector<std::pair<int32_t, int32_t>>& pairs, int64_t N, const char* what,
                       std::vector<int32_t>& keys, std::vector<int32_t>& off, std::vector<int32_t>& others,
                       std::vector<uint8_t>& cover) {
    std::vector<std::pair<int32_t, int32_t>> s(pairs);
    std::stable_sort(s.begin(), s.end(), [](const auto& a, const auto& b) { return a.first < b.first; });
    cover.assign((size_t)N, 0);
    for (size_t i = 0; i < s.size(); ++i) {
        if (i == 0 || s[i].first != s[i - 1].first) {
            if (i > 0 && s[i].first - s[i - 1].first < kTile) {
                set_error("tiles: %s blocks starting at %d and %d overlap partially", what, s[i - 1].first, s[i].first);
                return TGT_ERR_INVALID_ARG;
            }
            keys.push_back(s[i].first);
            off.push_back((int32_t)i);
            for (int j = 0; j < kTile; ++j) cover[(size_t)s[i].first + j] = 1;
        }
        others.push_back(s[i].second);
    }
    off.push_back((int32_t)s.size());
    return TGT_OK;
}

template <typename X>
static int upload(DevBuf& b, const std::vector<X>& v, hipStream_t st) {
    TGT_HIP_CHECK(b.alloc(sizeof(X) * (v.size() + 1)));
    if (!v.empty()) TGT_HIP_CHECK(hipMemcpyAsync(b.p, v.data(), sizeof(X) * v.size(), hipMemcpyHostToDevice, st));
    return TGT_OK;
}

template <typename T>
static int tile_fwd_launch(const tgt_tiles* tl, const void* q, const void* k, const void* v, float* acc, float* Zp,
                           int H, int d, hipStream_t st) {
    if (tl->n_dst_groups == 0) return TGT_OK;
    const float inv_scale = 1.0f / sqrtf((float)d);
    KernelTimer t(KS_TILE_FWD, st);
    if (d == 8)
        hipLaunchKernelGGL((k_tile_fwd<T, 8>), dim3(tl->n_dst_groups), dim3(64), 0, st, tl->dst_c0.as<int32_t>(),
                           tl->dst_off.as<int32_t>(), tl->dst_r0.as<int32_t>(), (const T*)q, (const T*)k, (const T*)v,
                           acc, Zp, H, inv_scale);
    else
        hipLaunchKernelGGL((k_tile_fwd<T, 16>), dim3(tl->n_dst_groups), dim3(64), 0, st, tl->dst_c0.as<int32_t>(),
                           tl->dst_off.as<int32_t>(), tl->dst_r0.as<int32_t>(), (const T*)q, (const T*)k, (const T*)v,
                           acc, Zp, H, inv_scale);
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

template <typename T, int D>
static int tile_bwd_launch_d(const tgt_tiles* tl, const void* q, const void* k, const void* v, const void* dout,
                             const float2* nd, float* dq, float* dk, float* dv, int H, hipStream_t st) {
    const float inv_scale = 1.0f / sqrtf((float)D);
    KernelTimer t(KS_TILE_BWD, st);
    if (tl->n_dst_groups > 0)
        hipLaunchKernelGGL((k_tile_bwd_dst<T, D>), dim3(tl->n_dst_groups), dim3(64), 0, st, tl->dst_c0.as<int32_t>(),
                           tl->dst_off.as<int32_t>(), tl->dst_r0.as<int32_t>(), (const T*)q, (const T*)k, (const T*)v,
                           (const T*)dout, nd, dq, H, inv_scale);
    if (tl->n_src_groups > 0)
        hipLaunchKernelGGL((k_tile_bwd_src<T, D>), dim3(tl->n_src_groups), dim3(64), 0, st, tl->src_r0.as<int32_t>(),
                           tl->src_off.as<int32_t>(), tl->src_c0.as<int32_t>(), (const T*)q, (const T*)k, (const T*)v,
                           (const T*)dout, nd, dk, dv, H, inv_scale);
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

static int check_block(const tgt_tiles* tl, const tgt_plan* plan, int H, int d, int dtype, const void* ws,
                       int64_t ws_bytes) {
    if (!tl || !plan) { set_error("block attention: null tiles or plan"); return TGT_ERR_INVALID_ARG; }
    if (tl->N != plan->N) { set_error("block attention: tiles and plan disagree on N"); return TGT_ERR_INVALID_ARG; }
    if (d != 8 && d != 16) { set_error("block attention: head dim %d not in {8, 16}", d); return TGT_ERR_UNSUPPORTED; }
    if (dtype != TGT_DTYPE_F32 && dtype != TGT_DTYPE_BF16) { set_error("bad dtype %d", dtype); return TGT_ERR_INVALID_ARG; }
    if (H < 1) { set_error("H must be positive"); return TGT_ERR_INVALID_ARG; }
    const int64_t need = block_ws(tl, plan, H, d).total;
    if (!ws || ws_bytes < need || (reinterpret_cast<uintptr_t>(ws) & 255u)) {
        set_error("block attention workspace: need %lld bytes, 256-byte aligned; got %lld", (long long)need,
                  (long long)ws_bytes);
        return TGT_ERR_WORKSPACE;
    }
    return TGT_OK;
}

}  // namespace tgt

extern "C" {

int tgt_tiles_create(const int32_t* h_tiles, int64_t T, int block_size, int64_t N, void* stream,
                     tgt_tiles_t** out) {
    if (!out || T < 0 || N < 1 || (T > 0 && !h_tiles)) {
        tgt::set_error("tgt_tiles_create: bad argument");
        return TGT_ERR_INVALID_ARG;
    }
    if (block_size != tgt::kTile) {
        tgt::set_error("tgt_tiles_create: only 16 x 16 tiles (the reference's block size) have a kernel");
        return TGT_ERR_UNSUPPORTED;
    }
    std::vector<std::pair<int32_t, int32_t>> by_dst, by_src;
    for (int64_t t = 0; t < T; ++t) {
        const int32_t r0 = h_tiles[2 * t], c0 = h_tiles[2 * t + 1];
        if (r0 < 0 || c0 < 0 || (int64_t)r0 + tgt::kTile > N || (int64_t)c0 + tgt::kTile > N) {
            tgt::set_error("tgt_tiles_create: tile %lld = (%d, %d) leaves [0, %lld)", (long long)t, r0, c0, (long long)N);
            return TGT_ERR_INDEX_RANGE;
        }
        by_dst.emplace_back(c0, r0);
        by_src.emplace_back(r0, c0);
    }
    tgt_tiles* tl = new (std::nothrow) tgt_tiles();
    if (!tl) return TGT_ERR_INVALID_ARG;
    tl->N = N;
    tl->T = T;
    hipStream_t st = (hipStream_t)stream;
    std::vector<int32_t> kd, od, xd, ks, os, xs;
    std::vector<uint8_t> cd, cs;
    int rc = tgt::group_tiles(by_dst, N, "destination", kd, od, xd, cd);
    if (!rc) rc = tgt::group_tiles(by_src, N, "source", ks, os, xs, cs);
    if (!rc) rc = tgt::upload(tl->dst_c0, kd, st);
    if (!rc) rc = tgt::upload(tl->dst_off, od, st);
    if (!rc) rc = tgt::upload(tl->dst_r0, xd, st);
    if (!rc) rc = tgt::upload(tl->src_r0, ks, st);
    if (!rc) rc = tgt::upload(tl->src_off, os, st);
    if (!rc) rc = tgt::upload(tl->src_c0, xs, st);
    if (!rc) rc = tgt::upload(tl->cover_dst, cd, st);
    if (!rc) rc = tgt::upload(tl->cover_src, cs, st);
    if (!rc && hipStreamSynchronize(st) != hipSuccess) rc = TGT_ERR_HIP;
    if (rc) { delete tl; return rc; }
    tl->n_dst_groups = (int32_t)kd.size();
    tl->n_src_groups = (int32_t)ks.size();
    *out = tl;
    return TGT_OK;
}

int tgt_tiles_destroy(tgt_tiles_t* tiles) {
    delete tiles;
    return TGT_OK;
}

int64_t tgt_block_attn_workspace_bytes(const tgt_tiles_t* tiles, const tgt_plan_t* plan, int H, int d) {
    if (!tiles || !plan || H < 1 || d < 1) return -1;
    return tgt::block_ws(tiles, plan, H, d).total;
}

int tgt_block_attn_fwd(const tgt_tiles_t* tiles, const tgt_plan_t* plan, const void* d_q, const void* d_k,
                       const void* d_v, const void* d_bias, int bias_mode, int H, int d, int dtype, void* d_out,
                       float* d_Z, void* d_workspace, int64_t workspace_bytes, void* stream) {
    int rc = tgt::check_block(tiles, plan, H, d, dtype, d_workspace, workspace_bytes);
    if (rc) return rc;
    if (!d_q || !d_k || !d_v || !d_out || !d_Z) { tgt::set_error("block attention: null q/k/v/out/Z"); return TGT_ERR_INVALID_ARG; }
    const tgt::BlockWs L = tgt::block_ws(tiles, plan, H, d);
    char* ws = static_cast<char*>(d_workspace);
    float* acc = reinterpret_cast<float*>(ws + L.acc);
    float* Zp = reinterpret_cast<float*>(ws + L.Z);
    hipStream_t st = (hipStream_t)stream;
    rc = dtype == TGT_DTYPE_F32 ? tgt::tile_fwd_launch<float>(tiles, d_q, d_k, d_v, acc, Zp, H, d, st)
                                : tgt::tile_fwd_launch<tgt::tbf16>(tiles, d_q, d_k, d_v, acc, Zp, H, d, st);
    if (rc) return rc;
    tgt::TileInit init{};
    init.acc = acc; init.Z = Zp; init.cover_dst = tiles->cover_dst.as<uint8_t>();
    return tgt::sparse_attn_fwd_impl(plan, d_q, d_k, d_v, d_bias, bias_mode, H, d, dtype, d_out, d_Z, ws + L.sparse,
                                     workspace_bytes - L.sparse, stream, &init);
}

int tgt_block_attn_bwd(const tgt_tiles_t* tiles, const tgt_plan_t* plan, const void* d_q, const void* d_k,
                       const void* d_v, const void* d_bias, int bias_mode, int H, int d, int dtype,
                       const void* d_out, const float* d_Z, const void* d_dout, void* d_dq, void* d_dk, void* d_dv,
                       void* d_dbias, void* d_workspace, int64_t workspace_bytes, void* stream) {
    int rc = tgt::check_block(tiles, plan, H, d, dtype, d_workspace, workspace_bytes);
    if (rc) return rc;
    if (!d_q || !d_k || !d_v || !d_out || !d_Z || !d_dout || !d_dq || !d_dk || !d_dv) {
        tgt::set_error("block attention backward: null pointer");
        return TGT_ERR_INVALID_ARG;
    }
    const tgt::BlockWs L = tgt::block_ws(tiles, plan, H, d);
    char* ws = static_cast<char*>(d_workspace);
    hipStream_t st = (hipStream_t)stream;
    rc = tgt::sparse_attn_node_side(plan, H, d, dtype, d_out, d_Z, d_dout, ws + L.sparse, stream);
    if (rc) return rc;
    const float2* nd = tgt::sparse_attn_nd_ptr(ws + L.sparse);
    float* dq = reinterpret_cast<float*>(ws + L.dq);
    float* dk = reinterpret_cast<float*>(ws + L.dk);
    float* dv = reinterpret_cast<float*>(ws + L.dv);
    if (dtype == TGT_DTYPE_F32)
        rc = d == 8 ? tgt::tile_bwd_launch_d<float, 8>(tiles, d_q, d_k, d_v, d_dout, nd, dq, dk, dv, H, st)
                    : tgt::tile_bwd_launch_d<float, 16>(tiles, d_q, d_k, d_v, d_dout, nd, dq, dk, dv, H, st);
    else
        rc = d == 8 ? tgt::tile_bwd_launch_d<tgt::tbf16, 8>(tiles, d_q, d_k, d_v, d_dout, nd, dq, dk, dv, H, st)
                    : tgt::tile_bwd_launch_d<tgt::tbf16, 16>(tiles, d_q, d_k, d_v, d_dout, nd, dq, dk, dv, H, st);
    if (rc) return rc;
    tgt::TileInit init{};
    init.dq = dq; init.dk = dk; init.dv = dv;
    init.cover_dst = tiles->cover_dst.as<uint8_t>();
    init.cover_src = tiles->cover_src.as<uint8_t>();
    return tgt::sparse_attn_bwd_impl(plan, d_q, d_k, d_v, d_bias, bias_mode, H, d, dtype, d_out, d_Z, d_dout, d_dq,
                                     d_dk, d_dv, d_dbias, ws + L.sparse, workspace_bytes - L.sparse, stream, &init,
                                     true);
}

}  // extern "C"
