// Input features of the graph-level model: GraphNodeFeature.forward
// (models/graphormer_graph_level.py:18-60) and the gradients of its four embedding tables.
//
//   out[g, 0, :]     = graph_token
//   out[g, 1 + i, :] = sum_f atom_table[x[g, i, f]] + in_degree_table[in_degree[g, i]]
//                      + out_degree_table[out_degree[g, i]]
//
// The reference runs three embedding lookups, a sum over the features, two adds, a repeat and a
// concatenation; here one kernel reads the ids and writes every output row once.  The backward adds
// the output gradient into float copies of the tables with vector-memory atomics (row 0 of the three
// lookup tables is the padding index and gets none) and a last kernel hands the sums over in the
// caller's type: results agree to rounding between runs, not bit for bit.  With a few dozen atom types every
// table row is shared by hundreds of node rows and atomics on one address serialise (55 us for the 33 K rows of
// 256 padded graphs; summing a workgroup's share in LDS first costs the same, the LDS float atomics of a CU
// serialise likewise), so neighbouring workgroups add into different copies of the sums (up to 64, at most 16 MB
// in all) that the last kernel adds up: 21 us.
#include "common.h"
#include <algorithm>

namespace tgt {
namespace {

struct nbf16 { uint16_t x; };
__device__ __forceinline__ float ldf(const float* p) { return *p; }
__device__ __forceinline__ float ldf(const nbf16* p) { return __uint_as_float(((uint32_t)p->x) << 16); }
__device__ __forceinline__ void stf(float* p, float v) { *p = v; }
__device__ __forceinline__ void stf(nbf16* p, float v) {
    const __bf16 b = static_cast<__bf16>(v);
    p->x = __builtin_bit_cast(uint16_t, b);
}
__device__ __forceinline__ int clamp_id(int64_t v, int n) { return v < 0 ? 0 : (v >= n ? n - 1 : (int)v); }

struct NodeFeatArgs {
    const int64_t* x;            // [b, s, Fx]
    const int64_t* in_degree;    // [b, s]
    const int64_t* out_degree;   // [b, s]
    int b, s, Fx, C, num_atoms, num_in, num_out;
    int pad_rows;                // 1: row 0 of the atom table is a padding index (no gradient); 0: an ordinary row
    int has_degree, has_token;   // without degrees: the atom sum alone; without token: s rows per graph, no row 0
};

// one thread per (graph, node, channel), channel fastest
template <typename T>
__global__ __launch_bounds__(256) void k_node_feature_fwd(NodeFeatArgs a, const T* __restrict__ atom, const T* __restrict__ tin,
                                                          const T* __restrict__ tout, const T* __restrict__ token,
                                                          T* __restrict__ out) {
    const int rows = a.s + a.has_token;
    const int64_t total = (int64_t)a.b * rows * a.C;
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= total) return;
    const int c = (int)(t % a.C);
    const int64_t row = t / a.C;
    const int node = (int)(row % rows) + 1 - a.has_token;             // 0 = the graph token's row
    const int64_t g = row / rows;
    float v;
    if (node == 0) {
        v = ldf(token + c);                                           // (:52-56)
    } else {
        const int64_t p = g * a.s + (node - 1);
        v = 0.f;
        for (int f = 0; f < a.Fx; ++f) v += ldf(atom + (int64_t)clamp_id(a.x[p * a.Fx + f], a.num_atoms) * a.C + c);   // (:45)
        if (a.has_degree) {
            v += ldf(tin + (int64_t)clamp_id(a.in_degree[p], a.num_in) * a.C + c);                                      // (:46-50)
            v += ldf(tout + (int64_t)clamp_id(a.out_degree[p], a.num_out) * a.C + c);
        }
    }
    stf(out + t, v);
}

__global__ __launch_bounds__(256) void k_fill_zero(float* __restrict__ p, int64_t n) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t < n) p[t] = 0.f;
}

// One wave per output row (lane = channel, channels beyond 64 in further passes): the ids of a row are read once
// by the whole wave, the row's position in the batch costs one division.  acc is the float copy of the tables in
// memory: float [num_atoms + num_in + num_out + 1][C].
template <typename T>
__device__ __forceinline__ void node_feature_bwd_row(const NodeFeatArgs& a, const T* __restrict__ dout, int64_t row, int lane,
                                                     float* acc) {
    const int rows = a.s + a.has_token;
    const int64_t g = row / rows;
    const int node = (int)(row - g * rows) + 1 - a.has_token;
    float* acc_in = acc + (int64_t)a.num_atoms * a.C;
    float* acc_out = acc_in + (int64_t)a.num_in * a.C;
    float* acc_tok = acc_out + (int64_t)a.num_out * a.C;
    const T* d_row = dout + row * a.C;
    if (node == 0) {
        for (int c = lane; c < a.C; c += 64) {
            const float d = ldf(d_row + c);
            if (d != 0.f) atomicAdd(acc_tok + c, d);
        }
        return;
    }
    const int64_t p = g * a.s + (node - 1);
    int ii = 0, io = 0;
    if (a.has_degree) {
        ii = clamp_id(a.in_degree[p], a.num_in);
        io = clamp_id(a.out_degree[p], a.num_out);
    }
    for (int c = lane; c < a.C; c += 64) {
        const float d = ldf(d_row + c);
        if (d == 0.f) continue;
        for (int f = 0; f < a.Fx; ++f) {
            const int id = clamp_id(a.x[p * a.Fx + f], a.num_atoms);
            if (id >= a.pad_rows) atomicAdd(acc + (int64_t)id * a.C + c, d);        // row 0 = padding index
        }
        if (ii > 0) atomicAdd(acc_in + (int64_t)ii * a.C + c, d);
        if (io > 0) atomicAdd(acc_out + (int64_t)io * a.C + c, d);
    }
}

template <typename T>
__global__ __launch_bounds__(256) void k_node_feature_bwd(NodeFeatArgs a, const T* __restrict__ dout, float* __restrict__ acc,
                                                          int copies, int64_t n_acc) {
    const int64_t n_rows = (int64_t)a.b * (a.s + a.has_token);
    const int64_t row = (int64_t)blockIdx.x * 4 + threadIdx.x / 64;
    // neighbouring workgroups add into different copies of the sums: rows that many positions share serialise less
    if (row < n_rows) node_feature_bwd_row(a, dout, row, threadIdx.x % 64, acc + (blockIdx.x % copies) * n_acc);
}

// Sum of the copies, handed over in the caller's type.  64 entries per workgroup along the lanes; the four waves take
// every fourth copy each (four loads in flight per lane) and their partial sums are added in wave order.
template <typename T>
__global__ __launch_bounds__(256) void k_node_feature_finish(const float* __restrict__ acc, int64_t n_atom, int64_t n_in,
                                                             int64_t n_out, int64_t n_tok, int copies, T* __restrict__ d_atom,
                                                             T* __restrict__ d_in, T* __restrict__ d_out, T* __restrict__ d_tok) {
    __shared__ float part[4][64];
    const int64_t n_acc = n_atom + n_in + n_out + n_tok;
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    const int64_t t = (int64_t)blockIdx.x * 64 + lane;
    float v = 0.f;
    if (t < n_acc) {
        for (int c0 = wave; c0 < copies; c0 += 16) {
            float x[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) x[u] = c0 + 4 * u < copies ? acc[(int64_t)(c0 + 4 * u) * n_acc + t] : 0.f;
            v += (x[0] + x[1]) + (x[2] + x[3]);
        }
    }
    part[wave][lane] = v;
    __syncthreads();
    if (wave != 0 || t >= n_acc) return;
    v = (part[0][lane] + part[1][lane]) + (part[2][lane] + part[3][lane]);
    if (t < n_atom) stf(d_atom + t, v);
    else if (t < n_atom + n_in) stf(d_in + (t - n_atom), v);
    else if (t < n_atom + n_in + n_out) stf(d_out + (t - n_atom - n_in), v);
    else stf(d_tok + (t - n_atom - n_in - n_out), v);
}

// Copies of the float sums the backward spreads its atomics over: as many as stay under 16 MB in all, at most 64.
inline int node_feat_copies(int64_t n_acc) {
    int copies = 64;
    while (copies > 1 && n_acc * copies * (int64_t)sizeof(float) > (16 << 20)) copies /= 2;
    return copies;
}

int node_feat_check(int b, int s, int Fx, int C, int num_atoms, int num_in, int num_out, int dtype, const char* who) {
    if (b < 0 || s < 0 || Fx < 1 || C < 1 || num_atoms < 1 || num_in < 1 || num_out < 1 ||
        (dtype != TGT_DTYPE_F32 && dtype != TGT_DTYPE_BF16)) {
        set_error("%s: bad size or dtype", who);
        return TGT_ERR_INVALID_ARG;
    }
    return TGT_OK;
}

}  // namespace
}  // namespace tgt

namespace tgt {
namespace {

int node_feature_fwd_impl(NodeFeatArgs a, const void* d_atom_table, const void* d_in_table, const void* d_out_table,
                          const void* d_graph_token, int dtype, void* d_out, void* stream) {
    const int64_t total = (int64_t)a.b * (a.s + a.has_token) * a.C;
    if (total == 0) return TGT_OK;
    const dim3 grid((unsigned)((total + 255) / 256));
    hipStream_t st = (hipStream_t)stream;
    if (dtype == TGT_DTYPE_F32)
        hipLaunchKernelGGL((k_node_feature_fwd<float>), grid, dim3(256), 0, st, a, (const float*)d_atom_table, (const float*)d_in_table,
                           (const float*)d_out_table, (const float*)d_graph_token, (float*)d_out);
    else
        hipLaunchKernelGGL((k_node_feature_fwd<nbf16>), grid, dim3(256), 0, st, a, (const nbf16*)d_atom_table, (const nbf16*)d_in_table,
                           (const nbf16*)d_out_table, (const nbf16*)d_graph_token, (nbf16*)d_out);
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

// acc layout: [num_atoms][C], [num_in][C], [num_out][C], [1][C]; tables that are not in use have num = 0 rows here
int node_feature_bwd_impl(NodeFeatArgs a, const void* d_dout, int dtype, void* d_datom, void* d_din, void* d_dout_table,
                          void* d_dtoken, float* acc, void* stream) {
    hipStream_t st = (hipStream_t)stream;
    const int64_t n_atom = (int64_t)a.num_atoms * a.C, n_in = a.has_degree ? (int64_t)a.num_in * a.C : 0,
                  n_out = a.has_degree ? (int64_t)a.num_out * a.C : 0, n_tok = a.has_token ? a.C : 0;
    const int64_t n_acc = n_atom + n_in + n_out + n_tok;
    if (!a.has_degree) a.num_in = a.num_out = 0;          // the kernel's offsets of the sums that follow the atom table
    const int64_t n_rows = (int64_t)a.b * (a.s + a.has_token);
    const int64_t total = n_rows * a.C;
    const dim3 fgrid((unsigned)((n_acc + 63) / 64));
    const int copies = node_feat_copies(n_acc);
    hipLaunchKernelGGL(k_fill_zero, dim3((unsigned)((n_acc * copies + 255) / 256)), dim3(256), 0, st, acc, n_acc * copies);
    if (dtype == TGT_DTYPE_F32) {
        if (total > 0)
            hipLaunchKernelGGL((k_node_feature_bwd<float>), dim3((unsigned)((n_rows + 3) / 4)), dim3(256), 0, st, a,
                               (const float*)d_dout, acc, copies, n_acc);
        hipLaunchKernelGGL((k_node_feature_finish<float>), fgrid, dim3(256), 0, st, (const float*)acc, n_atom, n_in, n_out, n_tok, copies,
                           (float*)d_datom, (float*)d_din, (float*)d_dout_table, (float*)d_dtoken);
    } else {
        if (total > 0)
            hipLaunchKernelGGL((k_node_feature_bwd<nbf16>), dim3((unsigned)((n_rows + 3) / 4)), dim3(256), 0, st, a,
                               (const nbf16*)d_dout, acc, copies, n_acc);
        hipLaunchKernelGGL((k_node_feature_finish<nbf16>), fgrid, dim3(256), 0, st, (const float*)acc, n_atom, n_in, n_out, n_tok, copies,
                           (nbf16*)d_datom, (nbf16*)d_din, (nbf16*)d_dout_table, (nbf16*)d_dtoken);
    }
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

}  // namespace
}  // namespace tgt

extern "C" {

int tgt_graph_node_feature_fwd(const int64_t* d_x, const int64_t* d_in_degree, const int64_t* d_out_degree, int Fx,
                               const void* d_atom_table, int num_atoms, const void* d_in_table, int num_in,
                               const void* d_out_table, int num_out, const void* d_graph_token, int b, int s, int C, int dtype,
                               void* d_out, void* stream) {
    using namespace tgt;
    const int rc = node_feat_check(b, s, Fx, C, num_atoms, num_in, num_out, dtype, "tgt_graph_node_feature_fwd");
    if (rc != TGT_OK) return rc;
    if (b == 0) return TGT_OK;
    if (!d_atom_table || !d_in_table || !d_out_table || !d_graph_token || !d_out || (s > 0 && (!d_x || !d_in_degree || !d_out_degree))) {
        set_error("tgt_graph_node_feature_fwd: null pointer");
        return TGT_ERR_INVALID_ARG;
    }
    NodeFeatArgs a{d_x, d_in_degree, d_out_degree, b, s, Fx, C, num_atoms, num_in, num_out, 1, 1, 1};
    return node_feature_fwd_impl(a, d_atom_table, d_in_table, d_out_table, d_graph_token, dtype, d_out, stream);
}

int64_t tgt_graph_node_feature_bwd_workspace_bytes(int num_atoms, int num_in, int num_out, int C) {
    if (num_atoms < 1 || num_in < 1 || num_out < 1 || C < 1) return 0;
    const int64_t n_acc = ((int64_t)num_atoms + num_in + num_out + 1) * C;
    return (int64_t)sizeof(float) * n_acc * tgt::node_feat_copies(n_acc);
}

int tgt_graph_node_feature_bwd(const void* d_dout, const int64_t* d_x, const int64_t* d_in_degree, const int64_t* d_out_degree,
                               int Fx, int num_atoms, int num_in, int num_out, int b, int s, int C, int dtype, void* d_datom_table,
                               void* d_din_table, void* d_dout_table, void* d_dgraph_token, void* d_workspace,
                               int64_t workspace_bytes, void* stream) {
    using namespace tgt;
    const int rc = node_feat_check(b, s, Fx, C, num_atoms, num_in, num_out, dtype, "tgt_graph_node_feature_bwd");
    if (rc != TGT_OK) return rc;
    if (!d_datom_table || !d_din_table || !d_dout_table || !d_dgraph_token ||
        (b > 0 && (!d_dout || (s > 0 && (!d_x || !d_in_degree || !d_out_degree))))) {
        set_error("tgt_graph_node_feature_bwd: null pointer");
        return TGT_ERR_INVALID_ARG;
    }
    const int64_t need = tgt_graph_node_feature_bwd_workspace_bytes(num_atoms, num_in, num_out, C);
    if (!d_workspace || workspace_bytes < need) {
        set_error("tgt_graph_node_feature_bwd: workspace of %lld bytes needed, got %lld", (long long)need, (long long)workspace_bytes);
        return TGT_ERR_WORKSPACE;
    }
    NodeFeatArgs a{d_x, d_in_degree, d_out_degree, b, s, Fx, C, num_atoms, num_in, num_out, 1, 1, 1};
    return node_feature_bwd_impl(a, d_dout, dtype, d_datom_table, d_din_table, d_dout_table, d_dgraph_token, (float*)d_workspace, stream);
}

int tgt_embedding_sum_fwd(const int64_t* d_x, int Fx, const void* d_table, int num_rows, int b, int s, int C, int dtype, void* d_out,
                          void* stream) {
    using namespace tgt;
    const int rc = node_feat_check(b, s, Fx, C, num_rows, 1, 1, dtype, "tgt_embedding_sum_fwd");
    if (rc != TGT_OK) return rc;
    if (b == 0 || s == 0) return TGT_OK;
    if (!d_table || !d_out || !d_x) {
        set_error("tgt_embedding_sum_fwd: null pointer");
        return TGT_ERR_INVALID_ARG;
    }
    NodeFeatArgs a{d_x, nullptr, nullptr, b, s, Fx, C, num_rows, 1, 1, 0, 0, 0};
    return node_feature_fwd_impl(a, d_table, nullptr, nullptr, nullptr, dtype, d_out, stream);
}

int64_t tgt_embedding_sum_bwd_workspace_bytes(int num_rows, int C) {
    if (num_rows < 1 || C < 1) return 0;
    const int64_t n_acc = (int64_t)num_rows * C;
    return (int64_t)sizeof(float) * n_acc * tgt::node_feat_copies(n_acc);
}

int tgt_embedding_sum_bwd(const void* d_dout, const int64_t* d_x, int Fx, int num_rows, int b, int s, int C, int dtype, void* d_dtable,
                          void* d_workspace, int64_t workspace_bytes, void* stream) {
    using namespace tgt;
    const int rc = node_feat_check(b, s, Fx, C, num_rows, 1, 1, dtype, "tgt_embedding_sum_bwd");
    if (rc != TGT_OK) return rc;
    if (!d_dtable || (b > 0 && s > 0 && (!d_dout || !d_x))) {
        set_error("tgt_embedding_sum_bwd: null pointer");
        return TGT_ERR_INVALID_ARG;
    }
    const int64_t need = tgt_embedding_sum_bwd_workspace_bytes(num_rows, C);
    if (!d_workspace || workspace_bytes < need) {
        set_error("tgt_embedding_sum_bwd: workspace of %lld bytes needed, got %lld", (long long)need, (long long)workspace_bytes);
        return TGT_ERR_WORKSPACE;
    }
    NodeFeatArgs a{d_x, nullptr, nullptr, b, s, Fx, C, num_rows, 1, 1, 0, 0, 0};
    return node_feature_bwd_impl(a, d_dout, dtype, d_dtable, nullptr, nullptr, nullptr, (float*)d_workspace, stream);
}

}  // extern "C"
