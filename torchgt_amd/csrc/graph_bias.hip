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

// Table gradients.  Each workgroup keeps the three tables in LDS ([num_spatial + num_edges + 1][H]
// floats), walks its share of the positions and writes one partial.  Row 0 of the two
// embedding tables is the padding index: it receives no gradient (nn.Embedding padding_idx=0).
template <typename T>
__global__ __launch_bounds__(256) void k_graph_bias_bwd(BiasArgs a, const T* __restrict__ dout, float* __restrict__ partial,
                                                        int copies) {
    extern __shared__ float acc_all[];
    const int n_acc = (a.num_spatial + a.num_edges + 1) * a.H;
    for (int k = threadIdx.x; k < n_acc * copies; k += 256) acc_all[k] = 0.f;
    __syncthreads();
    // few distinct ids meet many positions: neighbouring lanes add into different copies of the tables
    float* acc = acc_all + (threadIdx.x % copies) * n_acc;
    float* acc_sp = acc;
    float* acc_e = acc + a.num_spatial * a.H;
    float* acc_v = acc_e + a.num_edges * a.H;
    const int S1 = a.s + 1;
    const int64_t total = (int64_t)a.b * S1 * S1;
    const float inv_f = 1.f / (float)a.F;
    for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < total; t += (int64_t)gridDim.x * 256) {
        const int j = (int)(t % S1), i = (int)((t / S1) % S1);
        const int64_t g = t / ((int64_t)S1 * S1);
        const bool inner = i >= 1 && j >= 1;
        int sp = 0;
        const int64_t* et = nullptr;
        if (inner) {
            const int64_t pos = (g * a.s + (i - 1)) * a.s + (j - 1);
            sp = clamp_id(a.spatial_pos[pos], a.num_spatial);
            et = a.edge_type + pos * a.F;
        }
        for (int h = 0; h < a.H; ++h) {
            const float v = ldf(dout + ((g * a.H + h) * S1 + i) * S1 + j);
            if (v == 0.f) continue;              // masked (padded) positions carry exact zeros
            if (inner) {
                if (sp > 0) atomicAdd(&acc_sp[sp * a.H + h], v);
                for (int f = 0; f < a.F; ++f) {
                    const int e = clamp_id(et[f], a.num_edges);
                    if (e > 0) atomicAdd(&acc_e[e * a.H + h], v * inv_f);
                }
            } else {
                atomicAdd(&acc_v[h], v);
            }
        }
    }
    __syncthreads();
    for (int k = threadIdx.x; k < n_acc; k += 256) {
        float t = 0.f;
        for (int c = 0; c < copies; ++c) t += acc_all[c * n_acc + k];       // copies in order
        partial[(int64_t)blockIdx.x * n_acc + k] = t;
    }
}

template <typename T>
__global__ __launch_bounds__(256) void k_graph_bias_reduce(const float* __restrict__ partial, int workers, int n_sp, int n_e,
                                                           int n_v, T* __restrict__ d_sp, T* __restrict__ d_e,
                                                           T* __restrict__ d_v) {
    const int n = n_sp + n_e + n_v;
    const int k = blockIdx.x * 256 + threadIdx.x;
    if (k >= n) return;
    float t = 0.f;
    for (int w = 0; w < workers; ++w) t += partial[(int64_t)w * n + k];
    if (k < n_sp) stf(d_sp + k, t);
    else if (k < n_sp + n_e) stf(d_e + (k - n_sp), t);
    else stf(d_v + (k - n_sp - n_e), t);
}

constexpr int kBiasWorkers = 256;

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

// One workgroup per graph.  Distances (uint16: at most 2 * 510) and intermediate nodes (int16)
// live in LDS.  Within one k the k-th row and column do not change (M[k][k] = 0), so all
// (i, j) of a step can be relaxed at once and give exactly the sequential result.
constexpr int kFwMax = 128;
constexpr int kFwInf = 510;          // data/algos.pyx:30

__global__ __launch_bounds__(256) void k_floyd_warshall(const uint8_t* __restrict__ adj, const int32_t* __restrict__ n_nodes,
                                                        int n_max, int32_t* __restrict__ dist, int32_t* __restrict__ path) {
    extern __shared__ uint16_t lds[];
    const int g = blockIdx.x;
    const int n = n_nodes ? n_nodes[g] : n_max;
    uint16_t* M = lds;                                   // [n][n]
    int16_t* P = reinterpret_cast<int16_t*>(lds + n * n);
    const uint8_t* A = adj + (int64_t)g * n_max * n_max;
    for (int t = threadIdx.x; t < n * n; t += 256) {
        const int i = t / n, j = t % n;
        const uint16_t w = A[i * n_max + j];
        M[t] = i == j ? 0 : (w == 0 ? kFwInf : w);       // :27-32
        P[t] = -1;
    }
    __syncthreads();
    for (int k = 0; k < n; ++k) {
        for (int t = threadIdx.x; t < n * n; t += 256) {
            const int i = t / n, j = t % n;
            const uint16_t c = M[i * n + k] + M[k * n + j];
            if (M[t] > c && i != k && j != k) {          // row k and column k never improve through k
                M[t] = c;
                P[t] = (int16_t)k;
            }
        }
        __syncthreads();
    }
    int32_t* D = dist + (int64_t)g * n_max * n_max;
    int32_t* Q = path + (int64_t)g * n_max * n_max;
    for (int t = threadIdx.x; t < n * n; t += 256) {
        const int i = t / n, j = t % n;
        const bool far = M[t] >= kFwInf;                 // :49-53
        D[i * n_max + j] = far ? kFwInf : M[t];
        Q[i * n_max + j] = far ? kFwInf : P[t];
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
    if (dtype == TGT_DTYPE_F32) hipLaunchKernelGGL((k_graph_bias_fwd<float>), grid, dim3(256), 0, st, a, (float*)d_out);
    else hipLaunchKernelGGL((k_graph_bias_fwd<gbf16>), grid, dim3(256), 0, st, a, (gbf16*)d_out);
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
    if ((size_t)n_acc * sizeof(float) > 60 * 1024) {
        set_error("tgt_graph_attn_bias_bwd: (num_spatial + num_edges + 1) * H = %d table entries exceed the %d kept on chip",
                  n_acc, 60 * 1024 / 4);
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
    float* partial = (float*)d_workspace;
    int copies = 16;
    while (copies > 1 && (size_t)n_acc * copies * sizeof(float) > 60 * 1024) copies /= 2;
    const size_t lds = (size_t)n_acc * copies * sizeof(float);
    if (lds > 48 * 1024) {
        TGT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&k_graph_bias_bwd<float>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, 60 * 1024));
        TGT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&k_graph_bias_bwd<gbf16>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, 60 * 1024));
    }
    const unsigned rgrid = (unsigned)((n_acc + 255) / 256);
    if (dtype == TGT_DTYPE_F32) {
        hipLaunchKernelGGL((k_graph_bias_bwd<float>), dim3(workers), dim3(256), lds, st, a, (const float*)d_dout, partial, copies);
        hipLaunchKernelGGL((k_graph_bias_reduce<float>), dim3(rgrid), dim3(256), 0, st, partial, workers, num_spatial * H,
                           num_edges * H, H, (float*)d_dspatial_table, (float*)d_dedge_table, (float*)d_dvirtual_dist);
    } else {
        hipLaunchKernelGGL((k_graph_bias_bwd<gbf16>), dim3(workers), dim3(256), lds, st, a, (const gbf16*)d_dout, partial, copies);
        hipLaunchKernelGGL((k_graph_bias_reduce<gbf16>), dim3(rgrid), dim3(256), 0, st, partial, workers, num_spatial * H,
                           num_edges * H, H, (gbf16*)d_dspatial_table, (gbf16*)d_dedge_table, (gbf16*)d_dvirtual_dist);
    }
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
    const size_t lds = (size_t)n_max * n_max * 4;
    static bool raised = false;
    if (!raised && lds > 48 * 1024) {
        TGT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&k_floyd_warshall),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)(kFwMax * kFwMax * 4)));
        raised = true;
    }
    hipLaunchKernelGGL(k_floyd_warshall, dim3(num_graphs), dim3(256), lds, (hipStream_t)stream, d_adj, d_n_nodes, n_max,
                       d_dist, d_path);
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

}  // extern "C"
