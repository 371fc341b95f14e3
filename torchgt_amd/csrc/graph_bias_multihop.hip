// The path-encoding ('multi_hop') branch of the graph-level attention bias and the routine that
// prepares its input.
//
//   tgt_graph_attn_bias_multi_hop_fwd / _bwd   GraphAttnBias.forward with edge_type == 'multi_hop'
//                                              (models/graphormer_graph_level.py:94-156, :119-147) and the
//                                              gradients of its four parameter tensors
//   tgt_gen_edge_input                         gen_edge_input of data/algos.pyx:64-92: the edge features
//                                              along the recorded shortest path of every node pair
//
// The reference gathers a [b, s, s, D, F, H] tensor of edge embeddings, averages it over the features,
// multiplies every hop by its own H x H matrix (a bmm over D batches of b s s rows), sums the hops and
// divides by the path length: five tensors of b s s D H elements.  Here one thread owns one (graph, i, j)
// position: it reads the D F ids once, forms the D averaged embeddings in registers, applies the hop
// matrices from LDS and writes the H bias values.  The backward recomputes the averaged embeddings,
// and forms the gradient of the hop matrices as the sum over positions of (embedding of hop dd) x
// (bias gradient / path length): the 64 positions of a wave are staged in LDS and every lane owns
// fixed (row, column) entries of the H x H matrices, which it sums in registers over the whole walk.
#include "common.h"
#include <algorithm>

namespace tgt {
namespace {

struct mbf16 { uint16_t x; };
__device__ __forceinline__ float ldf(const float* p) { return *p; }
__device__ __forceinline__ float ldf(const mbf16* p) { return __uint_as_float(((uint32_t)p->x) << 16); }
__device__ __forceinline__ void stf(float* p, float v) { *p = v; }
__device__ __forceinline__ void stf(mbf16* p, float v) {
    const __bf16 b = static_cast<__bf16>(v);
    p->x = __builtin_bit_cast(uint16_t, b);
}
__device__ __forceinline__ int clamp_id(int64_t v, int n) { return v < 0 ? 0 : (v >= n ? n - 1 : (int)v); }

struct HopArgs {
    const void* attn_bias;        // [b, S1, S1]
    const int64_t* spatial_pos;   // [b, s, s]
    const int64_t* edge_input;    // [b, s, s, D0, F]
    const void* spatial_table;    // [num_spatial, H]
    const void* edge_table;       // [num_edges, H]
    const void* hop_weight;       // [num_edge_dis, H, H]
    const void* virtual_dist;     // [H]
    int b, s, H, F, D0, D, num_spatial, num_edges, max_dist;
};

// Path length the summed hop terms are divided by (:121-126): padding (0) and self (1) count as one
// hop, id p > 1 is a distance of p - 1; clamped to the number of hops kept when a limit is set.
__device__ __forceinline__ int hop_count(int sp, int max_dist) {
    int n = sp <= 1 ? 1 : sp - 1;
    if (max_dist > 0) n = min(n, max_dist);
    return n;
}

// Hop matrices into LDS as float, row stride HT (zero beyond H).
template <typename T, int HT>
__device__ __forceinline__ void load_hop_weight(const HopArgs& a, float* w_lds) {
    const T* w = reinterpret_cast<const T*>(a.hop_weight);
    for (int k = threadIdx.x; k < a.D * HT * HT; k += 256) {
        const int h = k % HT, h0 = (k / HT) % HT, dd = k / (HT * HT);
        w_lds[k] = h < a.H && h0 < a.H ? ldf(w + (dd * a.H + h0) * a.H + h) : 0.f;
    }
}

// Averaged edge embedding of hop dd at position pos: mean over the F features (:129).
template <typename T, int HT>
__device__ __forceinline__ void hop_embedding(const HopArgs& a, int64_t pos, int dd, float (&m)[HT]) {
    const T* e_tab = reinterpret_cast<const T*>(a.edge_table);
    const int64_t* ids = a.edge_input + (pos * a.D0 + dd) * a.F;
#pragma unroll
    for (int h = 0; h < HT; ++h) m[h] = 0.f;
    for (int f = 0; f < a.F; ++f) {
        const int id = clamp_id(ids[f], a.num_edges);
#pragma unroll
        for (int h = 0; h < HT; ++h)
            if (h < a.H) m[h] += ldf(e_tab + id * a.H + h);
    }
    const float inv_f = 1.f / (float)a.F;
#pragma unroll
    for (int h = 0; h < HT; ++h) m[h] *= inv_f;
}

template <typename T, int HT>
__global__ __launch_bounds__(256) void k_multi_hop_fwd(HopArgs a, T* __restrict__ out) {
    extern __shared__ float w_lds[];          // [D][HT][HT]
    load_hop_weight<T, HT>(a, w_lds);
    __syncthreads();
    const int S1 = a.s + 1;
    const int64_t plane = (int64_t)S1 * S1;
    const int64_t total = (int64_t)a.b * plane;
    const T* sp_tab = reinterpret_cast<const T*>(a.spatial_table);
    const T* vd = reinterpret_cast<const T*>(a.virtual_dist);
    for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < total; t += (int64_t)gridDim.x * 256) {
        const int64_t g = t / plane;
        const int ij = (int)(t - g * plane), i = ij / S1, j = ij - i * S1;
        const bool inner = i >= 1 && j >= 1;
        const float base = 2.f * ldf(reinterpret_cast<const T*>(a.attn_bias) + t);     // the clone plus the re-add (:104, :153)
        float v[HT];
#pragma unroll
        for (int h = 0; h < HT; ++h) v[h] = base;
        if (inner) {
            const int64_t pos = (g * a.s + (i - 1)) * a.s + (j - 1);
            const int sp = clamp_id(a.spatial_pos[pos], a.num_spatial);
            float y[HT];
#pragma unroll
            for (int h = 0; h < HT; ++h) y[h] = 0.f;
            for (int dd = 0; dd < a.D; ++dd) {
                float m[HT];
                hop_embedding<T, HT>(a, pos, dd, m);
                const float* w = w_lds + dd * HT * HT;
#pragma unroll
                for (int h0 = 0; h0 < HT; ++h0)
#pragma unroll
                    for (int h = 0; h < HT; ++h) y[h] += m[h0] * w[h0 * HT + h];       // (:134-139)
            }
            const float hops = (float)hop_count(sp, a.max_dist);
#pragma unroll
            for (int h = 0; h < HT; ++h)
                if (h < a.H) v[h] += ldf(sp_tab + sp * a.H + h) + y[h] / hops;         // (:110-111, :145-152)
        } else {
#pragma unroll
            for (int h = 0; h < HT; ++h)
                if (h < a.H) v[h] += ldf(vd + h);                                      // (:115-117)
        }
        T* o = out + g * a.H * plane + ij;
#pragma unroll
        for (int h = 0; h < HT; ++h)
            if (h < a.H) stf(o + h * plane, v[h]);
    }
}

// Layout of one workgroup's sums (floats): spatial table, edge table, virtual distance, hop matrices.
struct HopAcc {
    int n_sp, n_e, n_v, n_w;
    __host__ __device__ int total() const { return n_sp + n_e + n_v + n_w; }
};
__host__ __device__ inline HopAcc hop_acc(int num_spatial, int num_edges, int H, int D) {
    return HopAcc{num_spatial * H, num_edges * H, H, D * H * H};
}

constexpr int kHopWorkers = 1024;

// DC: hops per pass over the staged positions (the per-lane sums of a pass live in registers).
template <typename T, int HT, int DC>
__global__ __launch_bounds__(256) void k_multi_hop_bwd(HopArgs a, const T* __restrict__ dout, float* __restrict__ partial) {
    constexpr int EPL = HT * HT / 64;                 // matrix entries of one hop owned by a lane
    extern __shared__ float lds[];
    const HopAcc L = hop_acc(a.num_spatial, a.num_edges, a.H, a.D);
    float* w_lds = lds;                               // [D][HT][HT]
    float* st_dy = w_lds + a.D * HT * HT;             // [256][HT]  bias gradient / path length of the staged positions
    float* st_m = st_dy + 256 * HT;                   // [256][HT]  averaged embedding of one hop
    float* acc = st_m + 256 * HT;                     // [L.total()]
    float* acc_sp = acc;
    float* acc_e = acc_sp + L.n_sp;
    float* acc_v = acc_e + L.n_e;
    float* acc_w = acc_v + L.n_v;
    load_hop_weight<T, HT>(a, w_lds);
    for (int k = threadIdx.x; k < L.total(); k += 256) acc[k] = 0.f;
    __syncthreads();
    const int S1 = a.s + 1, H = a.H;
    const int64_t plane = (int64_t)S1 * S1;
    const int64_t total = (int64_t)a.b * plane;
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    const float inv_f = 1.f / (float)a.F;
    for (int dc = 0; dc < a.D || dc == 0; dc += DC) {          // one walk per DC hops (one walk when D <= DC)
        float wsum[DC][EPL];
#pragma unroll
        for (int u = 0; u < DC; ++u)
#pragma unroll
            for (int e = 0; e < EPL; ++e) wsum[u][e] = 0.f;
        for (int64_t t0 = (int64_t)blockIdx.x * 256; t0 < total; t0 += (int64_t)gridDim.x * 256) {
            const int64_t t = t0 + threadIdx.x;
            const bool valid = t < total;
            const int64_t g = valid ? t / plane : 0;
            const int ij = valid ? (int)(t - g * plane) : 0, i = ij / S1, j = ij - i * S1;
            const bool inner = valid && i >= 1 && j >= 1;
            const int64_t pos = inner ? (g * a.s + (i - 1)) * a.s + (j - 1) : 0;
            float dy[HT];
#pragma unroll
            for (int h = 0; h < HT; ++h) dy[h] = 0.f;
            if (valid) {
                const T* dg = dout + g * H * plane + ij;
                const int sp = inner ? clamp_id(a.spatial_pos[pos], a.num_spatial) : 0;
                const float hops = (float)hop_count(sp, a.max_dist);
#pragma unroll
                for (int h = 0; h < HT; ++h) {
                    if (h < H) {
                        const float d = ldf(dg + h * plane);
                        if (dc == 0 && d != 0.f) {                          // table gradients: first walk only
                            if (inner) { if (sp > 0) atomicAdd(&acc_sp[sp * H + h], d); }     // row 0 = padding index
                            else atomicAdd(&acc_v[h], d);
                        }
                        dy[h] = inner ? d / hops : 0.f;
                    }
                }
            }
#pragma unroll
            for (int h = 0; h < HT; ++h) st_dy[threadIdx.x * HT + h] = dy[h];
#pragma unroll
            for (int u = 0; u < DC; ++u) {
                const int dd = dc + u;
                if (dd < a.D) {                                              // uniform over the workgroup
                float m[HT];
#pragma unroll
                for (int h = 0; h < HT; ++h) m[h] = 0.f;
                if (inner) {
                    hop_embedding<T, HT>(a, pos, dd, m);
                    // gradient of the averaged embedding, handed to the F edge-table rows it was averaged from
                    const float* w = w_lds + dd * HT * HT;
                    const int64_t* ids = a.edge_input + (pos * a.D0 + dd) * a.F;
#pragma unroll
                    for (int h0 = 0; h0 < HT; ++h0) {
                        if (h0 >= H) continue;
                        float dm = 0.f;
#pragma unroll
                        for (int h = 0; h < HT; ++h) dm += w[h0 * HT + h] * dy[h];
                        dm *= inv_f;
                        if (dm != 0.f)
                            for (int f = 0; f < a.F; ++f) {
                                const int id = clamp_id(ids[f], a.num_edges);
                                if (id > 0) atomicAdd(&acc_e[id * H + h0], dm);            // row 0 = padding index
                            }
                    }
                }
#pragma unroll
                for (int h = 0; h < HT; ++h) st_m[threadIdx.x * HT + h] = m[h];
                __syncthreads();
                // lane owns entries (h0, h) = divmod(lane + 64 e, HT) of the hop matrix; its wave's 64 positions
#pragma unroll 4
                for (int p = 0; p < 64; ++p) {
                    const int q = (wave * 64 + p) * HT;
#pragma unroll
                    for (int e = 0; e < EPL; ++e) {
                        const int idx = lane + 64 * e;
                        wsum[u][e] += st_m[q + idx / HT] * st_dy[q + idx % HT];
                    }
                }
                __syncthreads();
                }
            }
        }
#pragma unroll
        for (int u = 0; u < DC; ++u) {
            const int dd = dc + u;
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                const int idx = lane + 64 * e, h0 = idx / HT, h = idx % HT;
                if (dd < a.D && h0 < H && h < H) atomicAdd(&acc_w[(dd * H + h0) * H + h], wsum[u][e]);
            }
        }
    }
    __syncthreads();
    for (int k = threadIdx.x; k < L.total(); k += 256) partial[(int64_t)blockIdx.x * L.total() + k] = acc[k];
}

// Sum of the workgroup partials in a fixed order; one thread per entry.
template <typename T>
__global__ __launch_bounds__(256) void k_multi_hop_reduce(const float* __restrict__ partial, int workers, HopAcc L, int H,
                                                          T* __restrict__ d_sp, T* __restrict__ d_e, T* __restrict__ d_v,
                                                          T* __restrict__ d_w_used, int64_t n_w_all) {
    const int n = L.total();
    const int64_t k = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (k < n) {
        float t = 0.f;
        for (int w = 0; w < workers; ++w) t += partial[(int64_t)w * n + k];
        if (k < L.n_sp) stf(d_sp + k, t);
        else if (k < L.n_sp + L.n_e) stf(d_e + (k - L.n_sp), t);
        else if (k < L.n_sp + L.n_e + L.n_v) stf(d_v + (k - L.n_sp - L.n_e), t);
        else stf(d_w_used + (k - L.n_sp - L.n_e - L.n_v), t);
    } else if (k - n < n_w_all - L.n_w) {
        stf(d_w_used + L.n_w + (k - n), 0.f);             // hop matrices beyond the hops in use
    }
}

int hop_check(int b, int s, int H, int F, int D0, int num_spatial, int num_edges, int num_edge_dis, int max_dist, int dtype,
              const char* who, int* D) {
    if (b < 0 || s < 0 || H < 1 || F < 1 || D0 < 0 || num_spatial < 1 || num_edges < 1 || num_edge_dis < 0 || max_dist < 0 ||
        (dtype != TGT_DTYPE_F32 && dtype != TGT_DTYPE_BF16)) {
        set_error("%s: bad size or dtype", who);
        return TGT_ERR_INVALID_ARG;
    }
    *D = max_dist > 0 ? std::min(D0, max_dist) : D0;       // (:125-127)
    if (*D > num_edge_dis) {
        set_error("%s: %d hops but only %d hop matrices", who, *D, num_edge_dis);      // the reference's bmm would raise
        return TGT_ERR_INVALID_ARG;
    }
    if (H > 32) {
        set_error("%s: at most 32 heads", who);
        return TGT_ERR_UNSUPPORTED;
    }
    return TGT_OK;
}

inline int head_tile(int H) { return H <= 8 ? 8 : (H <= 16 ? 16 : 32); }

// gen_edge_input (data/algos.pyx:64-92).  One thread per ordered pair (i, j) of a graph.  The
// reference expands the recorded intermediate node k = path[i][j] recursively as
// nodes(i, k) + [k] + nodes(k, j) (:56-61); the same order comes out of a walk that keeps the pending
// right ends on a stack: with the current node a and the top b, a direct pair (path[a][b] == -1) is
// the next hop, anything else pushes path[a][b].  Every stack entry is a distinct node of one shortest
// path, so n entries suffice.
constexpr int kGeiMaxNodes = 128;
constexpr int kGeiFar = 510;

template <typename FeatT>
__global__ __launch_bounds__(128) void k_gen_edge_input(const int32_t* __restrict__ path, const FeatT* __restrict__ feat,
                                                        const int32_t* __restrict__ n_nodes, int n_max, int F, int max_dist,
                                                        int64_t total, int64_t* __restrict__ out) {
    __shared__ uint8_t stack[kGeiMaxNodes][128];          // [depth][thread]: a thread's entries sit in its own bank column
    const int64_t t = (int64_t)blockIdx.x * 128 + threadIdx.x;
    if (t >= total) return;
    const int64_t plane = (int64_t)n_max * n_max;
    const int64_t g = t / plane;
    const int ij = (int)(t - g * plane), i = ij / n_max, j = ij - i * n_max;
    const int n = n_nodes ? n_nodes[g] : n_max;
    const int32_t* P = path + g * plane;
    const FeatT* Fg = feat + g * plane * F;
    int64_t* o = out + t * max_dist * F;
    int hop = 0;
    if (i < n && j < n && i != j && P[ij] != kGeiFar) {   // (:82-85)
        int a = i, depth = 1;
        stack[0][threadIdx.x] = (uint8_t)j;
        while (depth > 0 && hop < max_dist) {
            const int b = stack[depth - 1][threadIdx.x];
            const int k = P[a * n_max + b];
            if (k < 0 || k >= n || depth >= kGeiMaxNodes) {        // a direct edge: the next hop (:89)
                for (int f = 0; f < F; ++f) o[hop * F + f] = (int64_t)Fg[((int64_t)a * n_max + b) * F + f];
                ++hop;
                a = b;
                --depth;
            } else {
                stack[depth][threadIdx.x] = (uint8_t)k;
                ++depth;
            }
        }
    }
    for (int r = hop * F; r < max_dist * F; ++r) o[r] = -1;       // (:77)
}

}  // namespace
}  // namespace tgt

extern "C" {

int tgt_graph_attn_bias_multi_hop_fwd(const void* d_attn_bias, const int64_t* d_spatial_pos, const int64_t* d_edge_input, int D0,
                                      int F, const void* d_spatial_table, int num_spatial, const void* d_edge_table,
                                      int num_edges, const void* d_edge_dis_weight, int num_edge_dis, const void* d_virtual_dist,
                                      int multi_hop_max_dist, int b, int s, int H, int dtype, void* d_out, void* stream) {
    using namespace tgt;
    int D = 0;
    const int rc = hop_check(b, s, H, F, D0, num_spatial, num_edges, num_edge_dis, multi_hop_max_dist, dtype,
                             "tgt_graph_attn_bias_multi_hop_fwd", &D);
    if (rc != TGT_OK) return rc;
    if (b == 0) return TGT_OK;
    if (!d_attn_bias || !d_spatial_table || !d_edge_table || !d_virtual_dist || !d_out || (D > 0 && !d_edge_dis_weight) ||
        (s > 0 && (!d_spatial_pos || (D > 0 && !d_edge_input)))) {
        set_error("tgt_graph_attn_bias_multi_hop_fwd: null pointer");
        return TGT_ERR_INVALID_ARG;
    }
    const int HT = head_tile(H);
    const size_t lds = sizeof(float) * (size_t)D * HT * HT;
    if (lds > 48 * 1024) {
        set_error("tgt_graph_attn_bias_multi_hop_fwd: %d hop matrices of %d heads exceed the 48 KB kept on chip", D, H);
        return TGT_ERR_UNSUPPORTED;
    }
    HopArgs a{d_attn_bias, d_spatial_pos, d_edge_input, d_spatial_table, d_edge_table, d_edge_dis_weight, d_virtual_dist,
              b, s, H, F, D0, D, num_spatial, num_edges, multi_hop_max_dist};
    const int64_t total = (int64_t)b * (s + 1) * (s + 1);
    const dim3 grid((unsigned)std::min<int64_t>((total + 255) / 256, 8192));
    hipStream_t st = (hipStream_t)stream;
    KernelTimer timer(KS_GRAPH_BIAS_FWD, st);
#define TGT_HOP_FWD(T, HTV) hipLaunchKernelGGL((k_multi_hop_fwd<T, HTV>), grid, dim3(256), lds, st, a, (T*)d_out)
    if (dtype == TGT_DTYPE_F32) {
        if (HT == 8) TGT_HOP_FWD(float, 8); else if (HT == 16) TGT_HOP_FWD(float, 16); else TGT_HOP_FWD(float, 32);
    } else {
        if (HT == 8) TGT_HOP_FWD(mbf16, 8); else if (HT == 16) TGT_HOP_FWD(mbf16, 16); else TGT_HOP_FWD(mbf16, 32);
    }
#undef TGT_HOP_FWD
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

int64_t tgt_graph_attn_bias_multi_hop_bwd_workspace_bytes(int num_spatial, int num_edges, int H, int D) {
    if (num_spatial < 1 || num_edges < 1 || H < 1 || D < 0) return 0;
    return (int64_t)sizeof(float) * tgt::kHopWorkers * tgt::hop_acc(num_spatial, num_edges, H, D).total();
}

int tgt_graph_attn_bias_multi_hop_bwd(const void* d_dout, const int64_t* d_spatial_pos, const int64_t* d_edge_input, int D0, int F,
                                      const void* d_edge_table, int num_spatial, int num_edges, const void* d_edge_dis_weight,
                                      int num_edge_dis, int multi_hop_max_dist, int b, int s, int H, int dtype,
                                      void* d_dspatial_table, void* d_dedge_table, void* d_dedge_dis_weight,
                                      void* d_dvirtual_dist, void* d_workspace, int64_t workspace_bytes, void* stream) {
    using namespace tgt;
    int D = 0;
    const int rc = hop_check(b, s, H, F, D0, num_spatial, num_edges, num_edge_dis, multi_hop_max_dist, dtype,
                             "tgt_graph_attn_bias_multi_hop_bwd", &D);
    if (rc != TGT_OK) return rc;
    if (!d_dspatial_table || !d_dedge_table || !d_dvirtual_dist || (num_edge_dis > 0 && !d_dedge_dis_weight) ||
        (b > 0 && (!d_dout || !d_edge_table || (D > 0 && !d_edge_dis_weight) ||
                   (s > 0 && (!d_spatial_pos || (D > 0 && !d_edge_input)))))) {
        set_error("tgt_graph_attn_bias_multi_hop_bwd: null pointer");
        return TGT_ERR_INVALID_ARG;
    }
    const HopAcc L = hop_acc(num_spatial, num_edges, H, D);
    const int64_t need = tgt_graph_attn_bias_multi_hop_bwd_workspace_bytes(num_spatial, num_edges, H, D);
    if (!d_workspace || workspace_bytes < need) {
        set_error("tgt_graph_attn_bias_multi_hop_bwd: workspace of %lld bytes needed, got %lld", (long long)need,
                  (long long)workspace_bytes);
        return TGT_ERR_WORKSPACE;
    }
    const int HT = head_tile(H);
    const size_t lds = sizeof(float) * ((size_t)D * HT * HT + 2 * 256 * HT + L.total());
    if (lds > 128 * 1024) {
        set_error("tgt_graph_attn_bias_multi_hop_bwd: tables of %d entries, %d hops and %d heads need %zu bytes on chip (limit 131072)",
                  L.n_sp + L.n_e + L.n_v, D, H, lds);
        return TGT_ERR_UNSUPPORTED;
    }
    HopArgs a{nullptr, d_spatial_pos, d_edge_input, nullptr, d_edge_table, d_edge_dis_weight, nullptr,
              b, s, H, F, D0, D, num_spatial, num_edges, multi_hop_max_dist};
    const int64_t total = (int64_t)b * (s + 1) * (s + 1);
    const int workers = (int)std::max<int64_t>(1, std::min<int64_t>((total + 255) / 256, kHopWorkers));
    hipStream_t st = (hipStream_t)stream;
    KernelTimer timer(KS_GRAPH_BIAS_BWD, st);
    float* partial = (float*)d_workspace;
    const int64_t n_w_all = (int64_t)num_edge_dis * H * H;
    const unsigned rgrid = (unsigned)((L.total() + (n_w_all - L.n_w) + 255) / 256);
    auto launch = [&](auto kernel, auto reduce, auto* dout, auto* dsp, auto* de, auto* dv, auto* dw) -> int {
        if (lds > 48 * 1024)
            TGT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                              128 * 1024));
        hipLaunchKernelGGL(kernel, dim3(workers), dim3(256), lds, st, a, dout, partial);
        hipLaunchKernelGGL(reduce, dim3(rgrid), dim3(256), 0, st, (const float*)partial, workers, L, H, dsp, de, dv, dw, n_w_all);
        return TGT_OK;
    };
    int lrc;
    // hops per walk: 8 for up to 16 heads (8 or 32 sums per lane), 2 for 32 heads (32 sums per lane)
    if (dtype == TGT_DTYPE_F32) {
        auto* red = &k_multi_hop_reduce<float>;
        const float* dout = (const float*)d_dout;
        float *dsp = (float*)d_dspatial_table, *de = (float*)d_dedge_table, *dv = (float*)d_dvirtual_dist,
              *dw = (float*)d_dedge_dis_weight;
        lrc = HT == 8    ? launch(&k_multi_hop_bwd<float, 8, 8>, red, dout, dsp, de, dv, dw)
              : HT == 16 ? launch(&k_multi_hop_bwd<float, 16, 8>, red, dout, dsp, de, dv, dw)
                         : launch(&k_multi_hop_bwd<float, 32, 2>, red, dout, dsp, de, dv, dw);
    } else {
        auto* red = &k_multi_hop_reduce<mbf16>;
        const mbf16* dout = (const mbf16*)d_dout;
        mbf16 *dsp = (mbf16*)d_dspatial_table, *de = (mbf16*)d_dedge_table, *dv = (mbf16*)d_dvirtual_dist,
              *dw = (mbf16*)d_dedge_dis_weight;
        lrc = HT == 8    ? launch(&k_multi_hop_bwd<mbf16, 8, 8>, red, dout, dsp, de, dv, dw)
              : HT == 16 ? launch(&k_multi_hop_bwd<mbf16, 16, 8>, red, dout, dsp, de, dv, dw)
                         : launch(&k_multi_hop_bwd<mbf16, 32, 2>, red, dout, dsp, de, dv, dw);
    }
    if (lrc != TGT_OK) return lrc;
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

int tgt_gen_edge_input(const int32_t* d_path, const void* d_edge_feat, int feat_is_int64, int F, const int32_t* d_n_nodes,
                       int num_graphs, int n_max, int max_dist, int64_t* d_out, void* stream) {
    using namespace tgt;
    if (num_graphs < 0 || n_max < 1 || F < 1 || max_dist < 0 ||
        (num_graphs > 0 && max_dist > 0 && (!d_path || !d_edge_feat || !d_out))) {
        set_error("tgt_gen_edge_input: null pointer or bad size");
        return TGT_ERR_INVALID_ARG;
    }
    if (n_max > kGeiMaxNodes) {
        set_error("tgt_gen_edge_input: graphs of up to %d nodes (got n_max = %d)", kGeiMaxNodes, n_max);
        return TGT_ERR_UNSUPPORTED;
    }
    if (num_graphs == 0 || max_dist == 0) return TGT_OK;
    const int64_t total = (int64_t)num_graphs * n_max * n_max;
    const dim3 grid((unsigned)((total + 127) / 128));
    hipStream_t st = (hipStream_t)stream;
    if (feat_is_int64)
        hipLaunchKernelGGL((k_gen_edge_input<int64_t>), grid, dim3(128), 0, st, d_path, (const int64_t*)d_edge_feat, d_n_nodes,
                           n_max, F, max_dist, total, d_out);
    else
        hipLaunchKernelGGL((k_gen_edge_input<int32_t>), grid, dim3(128), 0, st, d_path, (const int32_t*)d_edge_feat, d_n_nodes,
                           n_max, F, max_dist, total, d_out);
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

}  // extern "C"
