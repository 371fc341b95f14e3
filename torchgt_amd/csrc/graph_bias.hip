// The graph-level attention bias and the shortest-path preprocessing behind it.
//
//   tgt_graph_attn_bias_fwd / _bwd   GraphAttnBias.forward, simple edge-type branch
//                                    (models/graphormer_graph_level.py:94-156) and the
//                                    gradients of its three embedding tables
//   tgt_floyd_warshall               floyd_warshall of data/algos.pyx:9-54 (distance and
//                                    intermediate-node matrices) for a batch of small graphs
//
// The reference builds the [b, H, S+1, S+1] bias with six ATen passes over tensors of
// that size (clone, repeat, two embedding lookups + permutes, slice adds); here one
// kernel reads the ids once and writes the bias once.  The backward folds the bias
// gradient into the (tiny) tables: every workgroup accumulates in LDS and the
// workgroup partials are added in a fixed order.
#include "common.h"
#include <algorithm>

namespace tgt {
namespace {

struct gbf16 { uint16_t x; };
__device__ __forceinline__ float ldf(const float* p) { return *p; }
__device__ __forceinline__ float ldf(const gbf16* p) { return __uint_as_float(((uint32_t)p->x) << 16); }
__device__ __forceinline__ void stf(float* p, float v) { *p = v; }
__device__ __forceinline__ void stf(gbf16* p, float v) {
    const __bf16 b = static_cast<__bf16>(v);
    p->x = __builtin_bit_cast(uint16_t, b);
}

constexpr int kMaxHeads = 32;

struct BiasArgs {
    const void* attn_bias;        // [b, S1, S1]
    const int64_t* spatial_pos;   // [b, s, s]
    const int64_t* edge_type;     // [b, s, s, F]
    const void* spatial_table;    // [num_spatial, H]
    const void* edge_table;       // [num_edges, H]
    const void* virtual_dist;     // [H]
    int b, s, H, F, num_spatial, num_edges;
};

__device__ __forceinline__ int clamp_id(int64_t v, int n) { return v < 0 ? 0 : (v >= n ? n - 1 : (int)v); }

// one thread per (graph, row i, column j) of the [S1, S1] bias, all heads
template <typename T>
__global__ __launch_bounds__(256) void k_graph_bias_fwd(BiasArgs a, T* __restrict__ out) {
    const int S1 = a.s + 1;
    const int64_t total = (int64_t)a.b * S1 * S1;
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= total) return;
    const int j = (int)(t % S1), i = (int)((t / S1) % S1);
    const int64_t g = t / ((int64_t)S1 * S1);
    const float base = 2.f * ldf(reinterpret_cast<const T*>(a.attn_bias) + t);    // the clone plus the final re-add (:104, :153)
    const T* sp_tab = reinterpret_cast<const T*>(a.spatial_table);
    const T* e_tab = reinterpret_cast<const T*>(a.edge_table);
    const T* vd = reinterpret_cast<const T*>(a.virtual_dist);
    const bool inner = i >= 1 && j >= 1;
    const bool virt = i == 0 || j == 0;          // (i >= 1, j == 0) and the whole row 0 (:116-117)
    int sp = 0;
    const int64_t* et = nullptr;
    if (inner) {
        const int64_t pos = (g * a.s + (i - 1)) * a.s + (j - 1);
        sp = clamp_id(a.spatial_pos[pos], a.num_spatial);
        et = a.edge_type + pos * a.F;
    }
    const float inv_f = 1.f / (float)a.F;
    for (int h = 0; h < a.H; ++h) {
        float v = base;
        if (inner) {
            v += ldf(sp_tab + sp * a.H + h);
            float e = 0.f;
            for (int f = 0; f < a.F; ++f) e += ldf(e_tab + clamp_id(et[f], a.num_edges) * a.H + h);
            v += e * inv_f;                      // mean over the edge features (:150)
        }
        if (virt) v += ldf(vd + h);
        stf(out + ((g * a.H + h) * S1 + i) * S1 + j, v);
    }
}

// Position (graph, row, column) of a thread in the [b, S1, S1] index space and its step from one
// iteration of a grid-stride loop to the next, without a 64-bit division per iteration.
struct BiasPos {
    int64_t g;
    int i, j;
};
struct BiasStep {
    int64_t dg;
    int di, dj;
};
__device__ __forceinline__ BiasPos bias_pos(int64_t t, int S1) {
    const int64_t plane = (int64_t)S1 * S1;
    BiasPos p;
    p.g = t / plane;
    const int ij = (int)(t - p.g * plane);
    p.i = ij / S1;
    p.j = ij - p.i * S1;
    return p;
}
__device__ __forceinline__ BiasStep bias_step(int64_t stride, int S1) {
    const BiasPos p = bias_pos(stride, S1);
    return BiasStep{p.g, p.i, p.j};
}
__device__ __forceinline__ void bias_advance(BiasPos& p, const BiasStep& d, int S1) {
    p.j += d.dj;
    if (p.j >= S1) { p.j -= S1; ++p.i; }
    p.i += d.di;
    if (p.i >= S1) { p.i -= S1; ++p.g; }
    p.g += d.dg;
}

// The same for eight heads and tables that fit LDS: the tables are converted to float once per
// workgroup, a position reads its table rows with 16-byte LDS loads instead of one global load per
// head and feature, and the global loads of a position (bias, ids) are issued together.  Same
// arithmetic in the same order as the kernel above.
template <typename T>
__global__ __launch_bounds__(256) void k_graph_bias_fwd8(BiasArgs a, T* __restrict__ out) {
    constexpr int H = 8;
    extern __shared__ float4 tab4[];
    float* tab = reinterpret_cast<float*>(tab4);
    const int n_sp = a.num_spatial * H, n_e = a.num_edges * H;
    {
        const T* sp_tab = reinterpret_cast<const T*>(a.spatial_table);
        const T* e_tab = reinterpret_cast<const T*>(a.edge_table);
        const T* vd = reinterpret_cast<const T*>(a.virtual_dist);
        for (int k = threadIdx.x; k < n_sp + n_e + H; k += 256)
            tab[k] = k < n_sp ? ldf(sp_tab + k) : (k < n_sp + n_e ? ldf(e_tab + (k - n_sp)) : ldf(vd + (k - n_sp - n_e)));
    }
    __syncthreads();
    const float4* t_sp = tab4;
    const float4* t_e = tab4 + n_sp / 4;
    const float4* t_v = t_e + n_e / 4;
    const int S1 = a.s + 1, F = a.F;
    const int64_t plane = (int64_t)S1 * S1;
    const int64_t total = (int64_t)a.b * plane;
    const float inv_f = 1.f / (float)F;
    const T* __restrict__ bias = reinterpret_cast<const T*>(a.attn_bias);
    const int64_t stride = (int64_t)gridDim.x * 256;
    const BiasStep step = bias_step(stride, S1);
    BiasPos p = bias_pos((int64_t)blockIdx.x * 256 + threadIdx.x, S1);
    for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < total; t += stride, bias_advance(p, step, S1)) {
        const int64_t g = p.g;
        const int i = p.i, j = p.j, ij = i * S1 + j;
        const bool inner = i >= 1 && j >= 1;
        const int64_t pos = inner ? (g * a.s + (i - 1)) * a.s + (j - 1) : 0;
        const T braw = bias[t];
        float v[H];
        if (a.s > 0) {
            const int64_t spr = a.spatial_pos[pos];
            float e[H];
#pragma unroll
            for (int h = 0; h < H; ++h) e[h] = 0.f;
            for (int f0 = 0; f0 < F; f0 += 4) {
                int64_t er[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) er[u] = a.edge_type[pos * F + min(f0 + u, F - 1)];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    if (f0 + u < F) {
                        const int id = clamp_id(er[u], a.num_edges);
                        const float4 lo = t_e[id * 2], hi = t_e[id * 2 + 1];
                        e[0] += lo.x; e[1] += lo.y; e[2] += lo.z; e[3] += lo.w;
                        e[4] += hi.x; e[5] += hi.y; e[6] += hi.z; e[7] += hi.w;
                    }
                }
            }
            const int sp = clamp_id(spr, a.num_spatial);
            const float4 lo = t_sp[sp * 2], hi = t_sp[sp * 2 + 1];
            const float s8[H] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
            const float base = 2.f * ldf(&braw);
#pragma unroll
            for (int h = 0; h < H; ++h) {
                float x = base;
                if (inner) { x += s8[h]; x += e[h] * inv_f; }
                v[h] = x;
            }
        } else {
            const float base = 2.f * ldf(&braw);
#pragma unroll
            for (int h = 0; h < H; ++h) v[h] = base;
        }
        if (!inner) {
            const float4 lo = t_v[0], hi = t_v[1];
            v[0] += lo.x; v[1] += lo.y; v[2] += lo.z; v[3] += lo.w;
            v[4] += hi.x; v[5] += hi.y; v[6] += hi.z; v[7] += hi.w;
        }
        T* __restrict__ o = out + g * H * plane + ij;
#pragma unroll
        for (int h = 0; h < H; ++h) stf(o + h * plane, v[h]);
    }
}

// Table gradients.  Each workgroup keeps the three tables in LDS ([num_spatial + num_edges + 1][H]
// floats), walks its share of the positions and writes one partial.  Row 0 of the two
// embedding tables is the padding index: it receives no gradient (nn.Embedding padding_idx=0).
// All loads of a position (ids, then the gradient of eight heads at a time) are issued without a
// lane-dependent branch around them: out-of-range lanes read a clamped address and add nothing.
// Shortest-path ids are few and small (most pairs of a graph are two to four hops apart), and an LDS
// float atomic costs a few cycles per active lane whatever the address: with up to eight heads the
// ids 1..NHOT are summed in registers (one compare per id, one select + add per id and head), added
// over the wave at the end and put into LDS by one lane; only the rare other ids, the edge types
// (most pairs are not edges: id 0) and the virtual-node row and column use atomics per position.
constexpr int kBiasFeat = 4;      // edge features handled per pass over the heads (1 when there is only one)
constexpr int kBiasHot = 5;       // spatial ids 1..5 (self, one to four hops) are summed in registers

// What one lane reads for one position and one pass (up to kBiasFeat edge features, eight heads), kept
// as loaded: converting or clamping a value where it is fetched would make the wave wait for it there.
template <typename T, int FC>
struct BiasFetch {
    int64_t spr, er[FC];
    T raw[8];
    bool valid, inner;
};
template <typename T, int FC>
__device__ __forceinline__ void bias_fetch(const BiasArgs& a, const T* __restrict__ dout, const BiasPos& p, bool valid, int f0,
                                           int h0, BiasFetch<T, FC>& x) {
    const int S1 = a.s + 1;
    const int64_t plane = (int64_t)S1 * S1;
    x.valid = valid;
    const int64_t g = valid ? p.g : 0;               // past the end: element 0, nothing is added
    const int i = valid ? p.i : 0, j = valid ? p.j : 0, ij = i * S1 + j;
    x.inner = valid && i >= 1 && j >= 1;
    const int64_t pos = x.inner ? (g * a.s + (i - 1)) * a.s + (j - 1) : 0;
    x.spr = 0;
#pragma unroll
    for (int u = 0; u < FC; ++u) x.er[u] = 0;
    if (a.s > 0) {
        x.spr = a.spatial_pos[pos];
#pragma unroll
        for (int u = 0; u < FC; ++u) x.er[u] = a.edge_type[pos * a.F + min(f0 + u, a.F - 1)];
    }
    const T* __restrict__ dg = dout + g * a.H * plane + ij;          // head h of this position: dg[h * plane]
#pragma unroll
    for (int u = 0; u < 8; ++u) x.raw[u] = dg[(int64_t)min(h0 + u, a.H - 1) * plane];
}

template <typename T, int NHOT, int FC>
__device__ __forceinline__ void bias_consume(const BiasArgs& a, const BiasFetch<T, FC>& x, int f0, int h0, float* acc_sp, float* acc_e,
                                             float* acc_v, float (&hot)[NHOT > 0 ? NHOT : 1][8]) {
    const int H = a.H;
    const int sp = x.inner && f0 == 0 ? clamp_id(x.spr, a.num_spatial) : 0;
    int e[FC];
#pragma unroll
    for (int u = 0; u < FC; ++u) e[u] = x.inner && f0 + u < a.F ? clamp_id(x.er[u], a.num_edges) : 0;
    const bool virt = x.valid && !x.inner && f0 == 0;
    const bool cold = sp > NHOT;
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = ldf(&x.raw[u]);
    if (NHOT > 0) {
#pragma unroll
        for (int r = 0; r < NHOT; ++r) {
            const bool hit = sp == r + 1;
#pragma unroll
            for (int u = 0; u < 8; ++u) hot[r][u] += hit ? v[u] : 0.f;
        }
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
        const int h = h0 + u;
        if (h < H && v[u] != 0.f) {              // masked (padded) positions carry exact zeros
            if (cold) atomicAdd(&acc_sp[sp * H + h], v[u]);
#pragma unroll
            for (int w = 0; w < FC; ++w)
                if (e[w] > 0) atomicAdd(&acc_e[e[w] * H + h], v[u]);
            if (virt) atomicAdd(&acc_v[h], v[u]);
        }
    }
}

// ONEPASS: H <= 8 and F <= FC, one fetch per position; the fetch of the next position is issued
// before the current one is consumed.
template <typename T, int NHOT, bool ONEPASS, int FC>
__global__ __launch_bounds__(256) void k_graph_bias_bwd(BiasArgs a, const T* __restrict__ dout, float* __restrict__ partial,
                                                        int copies) {
    extern __shared__ float acc_all[];
    const int n_acc = (a.num_spatial + a.num_edges + 1) * a.H;
    for (int k = threadIdx.x; k < n_acc * copies; k += 256) acc_all[k] = 0.f;
    __syncthreads();
    // neighbouring lanes add into different copies of the tables
    float* acc = acc_all + (threadIdx.x % copies) * n_acc;
    float* acc_sp = acc;
    float* acc_e = acc + a.num_spatial * a.H;
    float* acc_v = acc_e + a.num_edges * a.H;
    const int H = a.H, F = a.F;
    const int64_t total = (int64_t)a.b * (a.s + 1) * (a.s + 1);
    const int64_t stride = (int64_t)gridDim.x * 256;
    float hot[NHOT > 0 ? NHOT : 1][8];
#pragma unroll
    for (int r = 0; r < (NHOT > 0 ? NHOT : 1); ++r)
#pragma unroll
        for (int u = 0; u < 8; ++u) hot[r][u] = 0.f;
    if (ONEPASS) {
        BiasFetch<T, FC> cur, nxt;
        int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
        const BiasStep step = bias_step(stride, a.s + 1);
        BiasPos p = bias_pos(t, a.s + 1);
        if (t - threadIdx.x < total) bias_fetch(a, dout, p, t < total, 0, 0, cur);
        for (; t - threadIdx.x < total; t += stride) {
            bias_advance(p, step, a.s + 1);
            bias_fetch(a, dout, p, t + stride < total, 0, 0, nxt);
            bias_consume<T, NHOT, FC>(a, cur, 0, 0, acc_sp, acc_e, acc_v, hot);
            cur = nxt;
        }
    } else {
        for (int64_t t0 = (int64_t)blockIdx.x * 256; t0 < total; t0 += stride)
            for (int f0 = 0; f0 < F; f0 += FC)
                for (int h0 = 0; h0 < H; h0 += 8) {
                    BiasFetch<T, FC> x;
                    bias_fetch(a, dout, bias_pos(t0 + threadIdx.x, a.s + 1), t0 + threadIdx.x < total, f0, h0, x);
                    // the spatial id counts once per head pass, in the first feature pass
                    bias_consume<T, NHOT, FC>(a, x, f0, h0, acc_sp, acc_e, acc_v, hot);
                }
    }
    if (NHOT > 0) {
        // the wave's sums of the ids kept in registers (NHOT > 0 only with H <= 8: one pass over the heads)
#pragma unroll
        for (int r = 0; r < NHOT; ++r)
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                float x = hot[r][u];
#pragma unroll
                for (int off = 32; off >= 1; off >>= 1) x += __shfl_xor(x, off);
                if (threadIdx.x % 64 == 0 && u < H && r + 1 < a.num_spatial) atomicAdd(&acc_sp[(r + 1) * H + u], x);
            }
    }
    __syncthreads();
    const float inv_f = 1.f / (float)F;                       // mean over the edge features (:150)
    const int e_lo = a.num_spatial * H, e_hi = e_lo + a.num_edges * H;
    for (int k = threadIdx.x; k < n_acc; k += 256) {
        float t = 0.f;
        for (int c = 0; c < copies; ++c) t += acc_all[c * n_acc + k];       // copies in order
        partial[(int64_t)blockIdx.x * n_acc + k] = k >= e_lo && k < e_hi ? t * inv_f : t;
    }
}

// Sum of the workgroup partials in a fixed order: 64 slices of the workers per entry, then the slices.
template <typename T>
__global__ __launch_bounds__(256) void k_graph_bias_reduce(const float* __restrict__ partial, int workers, int n_sp, int n_e,
                                                           int n_v, T* __restrict__ d_sp, T* __restrict__ d_e,
                                                           T* __restrict__ d_v) {
    __shared__ float part[64][4];
    const int n = n_sp + n_e + n_v;
    const int kl = threadIdx.x % 4, slice = threadIdx.x / 4;
    const int k = blockIdx.x * 4 + kl;
    float t = 0.f;
    if (k < n)
        for (int w = slice; w < workers; w += 64) t += partial[(int64_t)w * n + k];
    part[slice][kl] = t;
    __syncthreads();
    if (slice != 0 || k >= n) return;
    t = 0.f;
#pragma unroll
    for (int c = 0; c < 64; ++c) t += part[c][kl];
    if (k < n_sp) stf(d_sp + k, t);
    else if (k < n_sp + n_e) stf(d_e + (k - n_sp), t);
    else stf(d_v + (k - n_sp - n_e), t);
}

constexpr int kBiasWorkers = 1024;
constexpr int kBiasCopies = 16;

int bias_check(int b, int s, int H, int F, int num_spatial, int num_edges, int dtype, const char* who) {
    if (b < 0 || s < 0 || H < 1 || F < 1 || num_spatial < 1 || num_edges < 1 ||
        (dtype != TGT_DTYPE_F32 && dtype != TGT_DTYPE_BF16)) {
        set_error("%s: bad size or dtype", who);
        return TGT_ERR_INVALID_ARG;
    }
    if (H > kMaxHeads) {
        set_error("%s: at most %d heads", who, kMaxHeads);
        return TGT_ERR_UNSUPPORTED;
    }
    return TGT_OK;
}

// One workgroup per graph.  Distances (uint16: at most 2 * 510) live in LDS; the intermediate nodes (int16) too
// for graphs of up to 128 nodes, beyond that they are kept in the output array itself (every (i, j) has one
// owner thread, so nobody else reads them).  Within one k the k-th row and column do not change
// (M[k][k] = 0), so all (i, j) of a step can be relaxed at once and give exactly the sequential result.
constexpr int kFwMax = 256;
constexpr int kFwLdsPath = 128;      // largest graph whose intermediate nodes fit in LDS beside the distances
constexpr int kFwInf = 510;          // data/algos.pyx:30

// 1024 threads: thread (r, j) = (tid / COLS, tid % COLS) owns column j of rows r, r + 1024 / COLS, ...: no
// division per element, row i's M[i][k] is one LDS word for all lanes of a row, M[k][j] runs along the lanes.
template <int COLS, bool PATH_IN_LDS>
__global__ __launch_bounds__(1024) void k_floyd_warshall(const uint8_t* __restrict__ adj, const int32_t* __restrict__ n_nodes,
                                                         int n_max, int32_t* __restrict__ dist, int32_t* __restrict__ path) {
    extern __shared__ uint16_t lds[];
    const int g = blockIdx.x;
    const int n = n_nodes ? min(max(n_nodes[g], 0), n_max) : n_max;      // a count outside [0, n_max] is clamped
    uint16_t* M = lds;                                   // [n][n]
    int16_t* P = reinterpret_cast<int16_t*>(lds + n * n);
    const uint8_t* A = adj + (int64_t)g * n_max * n_max;
    int32_t* D = dist + (int64_t)g * n_max * n_max;
    int32_t* Q = path + (int64_t)g * n_max * n_max;
    const int j = threadIdx.x % COLS, r = threadIdx.x / COLS;
    constexpr int kRows = 1024 / COLS;
    if (j < n)
        for (int i = r; i < n; i += kRows) {
            const uint16_t w = A[i * n_max + j];
            M[i * n + j] = i == j ? 0 : (w == 0 ? kFwInf : w);       // :27-32
            if (PATH_IN_LDS) P[i * n + j] = -1;
            else Q[i * n_max + j] = -1;
        }
    __syncthreads();
    for (int k = 0; k < n; ++k) {
        if (j < n && j != k) {
            const uint16_t kj = M[k * n + j];
            for (int i = r; i < n; i += kRows) {
                const uint16_t c = M[i * n + k] + kj;
                if (M[i * n + j] > c && i != k) {        // row k and column k never improve through k
                    M[i * n + j] = c;
                    if (PATH_IN_LDS) P[i * n + j] = (int16_t)k;
                    else Q[i * n_max + j] = k;
                }
            }
        }
        __syncthreads();
    }
    if (j < n)
        for (int i = r; i < n; i += kRows) {
            const bool far = M[i * n + j] >= kFwInf;     // :49-53
            D[i * n_max + j] = far ? kFwInf : M[i * n + j];
            if (PATH_IN_LDS) Q[i * n_max + j] = far ? kFwInf : P[i * n + j];
            else if (far) Q[i * n_max + j] = kFwInf;
        }
}

}  // namespace
}  // namespace tgt

extern "C" {

int tgt_graph_attn_bias_fwd(const void* d_attn_bias, const int64_t* d_spatial_pos, const int64_t* d_edge_type, int F,
                            const void* d_spatial_table, int num_spatial, const void* d_edge_table, int num_edges,
                            const void* d_virtual_dist, int b, int s, int H, int dtype, void* d_out, void* stream) {
    using namespace tgt;
    const int rc = bias_check(b, s, H, F, num_spatial, num_edges, dtype, "tgt_graph_attn_bias_fwd");
    if (rc != TGT_OK) return rc;
    if (b == 0) return TGT_OK;
    if (!d_attn_bias || !d_spatial_table || !d_edge_table || !d_virtual_dist || !d_out ||
        (s > 0 && (!d_spatial_pos || !d_edge_type))) {
        set_error("tgt_graph_attn_bias_fwd: null pointer");
        return TGT_ERR_INVALID_ARG;
    }
    BiasArgs a{d_attn_bias, d_spatial_pos, d_edge_type, d_spatial_table, d_edge_table, d_virtual_dist,
               b, s, H, F, num_spatial, num_edges};
    const int64_t total = (int64_t)b * (s + 1) * (s + 1);
    const dim3 grid((unsigned)((total + 255) / 256));
    hipStream_t st = (hipStream_t)stream;
    KernelTimer timer(KS_GRAPH_BIAS_FWD, st);
    const size_t tab_bytes = sizeof(float) * (size_t)(num_spatial + num_edges + 1) * H;
    if (H == 8 && tab_bytes <= 32 * 1024) {
        const dim3 g8((unsigned)std::min<int64_t>((total + 255) / 256, 4096));
        if (dtype == TGT_DTYPE_F32) hipLaunchKernelGGL((k_graph_bias_fwd8<float>), g8, dim3(256), tab_bytes, st, a, (float*)d_out);
        else hipLaunchKernelGGL((k_graph_bias_fwd8<gbf16>), g8, dim3(256), tab_bytes, st, a, (gbf16*)d_out);
    } else if (dtype == TGT_DTYPE_F32) {
        hipLaunchKernelGGL((k_graph_bias_fwd<float>), grid, dim3(256), 0, st, a, (float*)d_out);
    } else {
        hipLaunchKernelGGL((k_graph_bias_fwd<gbf16>), grid, dim3(256), 0, st, a, (gbf16*)d_out);
    }
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

int64_t tgt_graph_attn_bias_bwd_workspace_bytes(int num_spatial, int num_edges, int H) {
    if (num_spatial < 1 || num_edges < 1 || H < 1) return 0;
    return (int64_t)sizeof(float) * tgt::kBiasWorkers * (num_spatial + num_edges + 1) * H;
}

int tgt_graph_attn_bias_bwd(const void* d_dout, const int64_t* d_spatial_pos, const int64_t* d_edge_type, int F,
                            int num_spatial, int num_edges, int b, int s, int H, int dtype, void* d_dspatial_table,
                            void* d_dedge_table, void* d_dvirtual_dist, void* d_workspace, int64_t workspace_bytes,
                            void* stream) {
    using namespace tgt;
    const int rc = bias_check(b, s, H, F, num_spatial, num_edges, dtype, "tgt_graph_attn_bias_bwd");
    if (rc != TGT_OK) return rc;
    if (!d_dspatial_table || !d_dedge_table || !d_dvirtual_dist ||
        (b > 0 && (!d_dout || (s > 0 && (!d_spatial_pos || !d_edge_type))))) {
        set_error("tgt_graph_attn_bias_bwd: null pointer");
        return TGT_ERR_INVALID_ARG;
    }
    const int n_acc = (num_spatial + num_edges + 1) * H;
    if ((size_t)n_acc * sizeof(float) > 128 * 1024) {
        set_error("tgt_graph_attn_bias_bwd: (num_spatial + num_edges + 1) * H = %d table entries exceed the %d kept on chip",
                  n_acc, 128 * 1024 / 4);
        return TGT_ERR_UNSUPPORTED;
    }
    if (!d_workspace || workspace_bytes < tgt_graph_attn_bias_bwd_workspace_bytes(num_spatial, num_edges, H)) {
        set_error("tgt_graph_attn_bias_bwd: workspace of %lld bytes needed, got %lld",
                  (long long)tgt_graph_attn_bias_bwd_workspace_bytes(num_spatial, num_edges, H), (long long)workspace_bytes);
        return TGT_ERR_WORKSPACE;
    }
    BiasArgs a{nullptr, d_spatial_pos, d_edge_type, nullptr, nullptr, nullptr, b, s, H, F, num_spatial, num_edges};
    const int64_t total = (int64_t)b * (s + 1) * (s + 1);
    const int workers = (int)std::max<int64_t>(1, std::min<int64_t>((total + 255) / 256, kBiasWorkers));
    hipStream_t st = (hipStream_t)stream;
    KernelTimer timer(KS_GRAPH_BIAS_BWD, st);
    float* partial = (float*)d_workspace;
    int copies = kBiasCopies;
    while (copies > 1 && (size_t)n_acc * copies * sizeof(float) > 16 * 1024) copies /= 2;      // more workgroups per CU beat more copies
    const size_t lds = (size_t)n_acc * copies * sizeof(float);
    const unsigned rgrid = (unsigned)((n_acc + 3) / 4);
    auto launch = [&](auto kernel, auto reduce, auto* dout, auto* dsp, auto* de, auto* dv) -> int {
        if (lds > 48 * 1024)
            TGT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                              128 * 1024));
        hipLaunchKernelGGL(kernel, dim3(workers), dim3(256), lds, st, a, dout, partial, copies);
        hipLaunchKernelGGL(reduce, dim3(rgrid), dim3(256), 0, st, (const float*)partial, workers, num_spatial * H, num_edges * H, H,
                           dsp, de, dv);
        return TGT_OK;
    };
    // registers for the frequent ids need one pass over the heads; the prefetching loop one pass over the features too
    const int variant = H > 8 ? 0 : (F > kBiasFeat ? 1 : (F > 1 ? 2 : 3));
    int lrc;
    if (dtype == TGT_DTYPE_F32) {
        auto* red = &k_graph_bias_reduce<float>;
        const float* dout = (const float*)d_dout;
        float *dsp = (float*)d_dspatial_table, *de = (float*)d_dedge_table, *dv = (float*)d_dvirtual_dist;
        lrc = variant == 3   ? launch(&k_graph_bias_bwd<float, kBiasHot, true, 1>, red, dout, dsp, de, dv)
              : variant == 2 ? launch(&k_graph_bias_bwd<float, kBiasHot, true, kBiasFeat>, red, dout, dsp, de, dv)
              : variant == 1 ? launch(&k_graph_bias_bwd<float, kBiasHot, false, kBiasFeat>, red, dout, dsp, de, dv)
                             : launch(&k_graph_bias_bwd<float, 0, false, kBiasFeat>, red, dout, dsp, de, dv);
    } else {
        auto* red = &k_graph_bias_reduce<gbf16>;
        const gbf16* dout = (const gbf16*)d_dout;
        gbf16 *dsp = (gbf16*)d_dspatial_table, *de = (gbf16*)d_dedge_table, *dv = (gbf16*)d_dvirtual_dist;
        lrc = variant == 3   ? launch(&k_graph_bias_bwd<gbf16, kBiasHot, true, 1>, red, dout, dsp, de, dv)
              : variant == 2 ? launch(&k_graph_bias_bwd<gbf16, kBiasHot, true, kBiasFeat>, red, dout, dsp, de, dv)
              : variant == 1 ? launch(&k_graph_bias_bwd<gbf16, kBiasHot, false, kBiasFeat>, red, dout, dsp, de, dv)
                             : launch(&k_graph_bias_bwd<gbf16, 0, false, kBiasFeat>, red, dout, dsp, de, dv);
    }
    if (lrc != TGT_OK) return lrc;
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

int tgt_floyd_warshall(const uint8_t* d_adj, const int32_t* d_n_nodes, int num_graphs, int n_max, int32_t* d_dist,
                       int32_t* d_path, void* stream) {
    using namespace tgt;
    if (num_graphs < 0 || n_max < 1 || (num_graphs > 0 && (!d_adj || !d_dist || !d_path))) {
        set_error("tgt_floyd_warshall: null pointer or bad size");
        return TGT_ERR_INVALID_ARG;
    }
    if (n_max > kFwMax) {
        set_error("tgt_floyd_warshall: graphs of up to %d nodes (got n_max = %d)", kFwMax, n_max);
        return TGT_ERR_UNSUPPORTED;
    }
    if (num_graphs == 0) return TGT_OK;
    hipStream_t st = (hipStream_t)stream;
    if (n_max <= kFwLdsPath) {
        const size_t lds = (size_t)n_max * n_max * 4;
        static bool raised = false;
        if (!raised && lds > 48 * 1024) {
            TGT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&k_floyd_warshall<128, true>),
                                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)(kFwLdsPath * kFwLdsPath * 4)));
            raised = true;
        }
        hipLaunchKernelGGL((k_floyd_warshall<128, true>), dim3(num_graphs), dim3(1024), lds, st, d_adj, d_n_nodes, n_max, d_dist,
                           d_path);
    } else {
        const size_t lds = (size_t)n_max * n_max * 2;      // up to 128 KB of the CU's 160
        static bool raised = false;
        if (!raised) {
            TGT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&k_floyd_warshall<256, false>),
                                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)(kFwMax * kFwMax * 2)));
            raised = true;
        }
        hipLaunchKernelGGL((k_floyd_warshall<256, false>), dim3(num_graphs), dim3(1024), lds, st, d_adj, d_n_nodes, n_max, d_dist,
                           d_path);
    }
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

}  // extern "C"
