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

// Position (graph, row, column) of a thread in the [b, S1, S1] index space and its step from one
// iteration of a grid-stride loop to the next, without a 64-bit division per iteration.
struct HopPos {
    int64_t g;
    int i, j;
};
__device__ __forceinline__ HopPos hop_pos(int64_t t, int S1) {
    const int64_t plane = (int64_t)S1 * S1;
    HopPos p;
    p.g = t / plane;
    const int ij = (int)(t - p.g * plane);
    p.i = ij / S1;
    p.j = ij - p.i * S1;
    return p;
}
__device__ __forceinline__ void hop_advance(HopPos& p, const HopPos& d, int S1) {
    p.j += d.j;
    if (p.j >= S1) { p.j -= S1; ++p.i; }
    p.i += d.i;
    if (p.i >= S1) { p.i -= S1; ++p.g; }
    p.g += d.g;
}

// Entry idx of the hop matrices read straight from the caller's tensor.  With a uniform index and a
// pointer the kernel never writes through, the compiler turns these into scalar loads: a hop's 64 values
// sit in scalar registers and cost the LDS nothing (eight heads only: the layout is then [D][8][8]).
__device__ __forceinline__ float w_at(const float* __restrict__ w, int idx) { return w[idx]; }
__device__ __forceinline__ float w_at(const mbf16* __restrict__ w, int idx) {
    const uint32_t pr = reinterpret_cast<const uint32_t*>(w)[idx >> 1];
    return __uint_as_float((idx & 1) ? (pr & 0xffff0000u) : (pr << 16));
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
// A table [rows, H] into LDS as float, row stride HT (zero beyond H).
template <typename T, int HT>
__device__ __forceinline__ void load_table(const void* table, int rows, int H, float* t_lds) {
    const T* t = reinterpret_cast<const T*>(table);
    for (int k = threadIdx.x; k < rows * HT; k += 256) {
        const int h = k % HT, r = k / HT;
        t_lds[k] = h < H ? ldf(t + r * H + h) : 0.f;
    }
}

// TAB_LDS: the spatial and edge tables fit LDS next to the hop matrices.
// WS: eight heads, the hop matrices come through scalar loads from wq instead of LDS.
template <typename T, int HT, bool TAB_LDS, bool WS>
__global__ __launch_bounds__(256) void k_multi_hop_fwd(HopArgs a, const T* __restrict__ wq, T* __restrict__ out) {
    extern __shared__ float w_lds[];          // [D][HT][HT], then [num_edges][HT], [num_spatial][HT] with TAB_LDS
    float* e_lds = w_lds + a.D * HT * HT;
    float* sp_lds = e_lds + a.num_edges * HT;
    if (!WS) load_hop_weight<T, HT>(a, w_lds);
    if (TAB_LDS) {
        load_table<T, HT>(a.edge_table, a.num_edges, a.H, e_lds);
        load_table<T, HT>(a.spatial_table, a.num_spatial, a.H, sp_lds);
    }
    __syncthreads();
    const int S1 = a.s + 1;
    const int64_t plane = (int64_t)S1 * S1;
    const int64_t total = (int64_t)a.b * plane;
    const T* sp_tab = reinterpret_cast<const T*>(a.spatial_table);
    const T* e_tab = reinterpret_cast<const T*>(a.edge_table);
    const T* vd = reinterpret_cast<const T*>(a.virtual_dist);
    const float inv_f = 1.f / (float)a.F;
    const int64_t stride = (int64_t)gridDim.x * 256;
    const HopPos step = hop_pos(stride, S1);
    HopPos ps = hop_pos((int64_t)blockIdx.x * 256 + threadIdx.x, S1);
    for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < total; t += stride, hop_advance(ps, step, S1)) {
        const int64_t g = ps.g;
        const int i = ps.i, j = ps.j, ij = i * S1 + j;
        const bool inner = i >= 1 && j >= 1;
        const float base = 2.f * ldf(reinterpret_cast<const T*>(a.attn_bias) + t);     // the clone plus the re-add (:104, :153)
        float v[HT];
#pragma unroll
        for (int h = 0; h < HT; ++h) v[h] = base;
        // a masked position (-inf from the collator: padded key columns) stays -inf whatever the finite table
        // entries add: its lanes sit the hop loop out, and a wave of such lanes skips it altogether
        if (inner && base != -INFINITY) {
            const int64_t pos = (g * a.s + (i - 1)) * a.s + (j - 1);
            const int sp = clamp_id(a.spatial_pos[pos], a.num_spatial);
            float y[HT];
#pragma unroll
            for (int h = 0; h < HT; ++h) y[h] = 0.f;
            // the D F ids of the position, eight at a time so that their loads are in flight together; the hop
            // (dd) and feature (f) counters are uniform, the embedding sum m of a hop is closed after its last feature
            const int64_t* ids = a.edge_input + pos * a.D0 * a.F;
            const int n_ids = a.D * a.F;
            float m[HT];
#pragma unroll
            for (int h = 0; h < HT; ++h) m[h] = 0.f;
            int dd = 0, f = 0;
            for (int k0 = 0; k0 < n_ids; k0 += 8) {
                int64_t idr[8];
#pragma unroll
                for (int k = 0; k < 8; ++k) idr[k] = ids[min(k0 + k, n_ids - 1)];
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    if (k0 + k < n_ids) {
                        const int id = clamp_id(idr[k], a.num_edges);
#pragma unroll
                        for (int h = 0; h < HT; ++h) {
                            if (TAB_LDS) m[h] += e_lds[id * HT + h];
                            else if (h < a.H) m[h] += ldf(e_tab + id * a.H + h);
                        }
                        if (++f == a.F) {
                            const float* w = w_lds + dd * HT * HT;
#pragma unroll
                            for (int h0 = 0; h0 < HT; ++h0) {
                                const float mh = m[h0] * inv_f;                            // mean over the features (:129)
#pragma unroll
                                for (int h = 0; h < HT; ++h)                               // (:134-139)
                                    y[h] += mh * (WS ? w_at(wq, dd * 64 + h0 * 8 + h) : w[h0 * HT + h]);
                                m[h0] = 0.f;
                            }
                            f = 0;
                            ++dd;
                        }
                    }
                }
            }
            const float hops = (float)hop_count(sp, a.max_dist);
#pragma unroll
            for (int h = 0; h < HT; ++h)
                if (h < a.H) v[h] += (TAB_LDS ? sp_lds[sp * HT + h] : ldf(sp_tab + sp * a.H + h)) + y[h] / hops;   // (:110-111, :145-152)
        } else if (!inner) {
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

// Orders the LDS writes of a wave's lanes before the LDS reads of the same wave that follow (and the other way
// round): the hardware runs a wave's LDS instructions in order, this keeps the compiler from moving them.
__device__ __forceinline__ void wave_sync_lds() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Layout of one workgroup's sums (floats): spatial table, edge table, virtual distance, hop matrices.
struct HopAcc {
    int n_sp, n_e, n_v, n_w;
    __host__ __device__ int total() const { return n_sp + n_e + n_v + n_w; }
};
__host__ __device__ inline HopAcc hop_acc(int num_spatial, int num_edges, int H, int D) {
    return HopAcc{num_spatial * H, num_edges * H, H, D * H * H};
}

constexpr int kHopWorkers = 768;        // three workgroups of the gradient kernel fit a CU: one round
constexpr int kStage = 260;            // row stride of the staged positions: rows of consecutive heads start 4 banks apart
constexpr int kHopHotSp = 5;      // spatial ids 1..5 (self, one to four hops) and
constexpr int kHopHotE = 4;       // edge ids 1..4 are summed in registers when there are at most eight heads

// Gradients.  An LDS float atomic costs a few cycles per active lane whatever the address, and nearly
// every position would issue one per head for its spatial id and one per head, hop and feature for its
// edge ids: with up to eight heads the frequent small ids are summed in registers instead (a compare,
// a select and an add per id and head), added over the wave at the end and put into LDS by one lane.
// The hop-matrix gradient is a sum over positions of outer products: the workgroup's 256 positions are
// staged head-major in LDS and lane (h0, h) of every wave sums m[h0] dy[h] over its wave's 64 positions
// with 16-byte LDS reads.
// DC: hops per pass over the positions (the per-lane sums of a pass live in registers).
template <typename T, int HT, int DC, bool TAB_LDS, bool WS>
__global__ __launch_bounds__(256) void k_multi_hop_bwd(HopArgs a, const T* __restrict__ wq, const T* __restrict__ dout,
                                                       float* __restrict__ partial) {
    constexpr int EPL = HT * HT / 64;                 // matrix entries of one hop owned by a lane
    constexpr bool HOT = HT == 8;
    constexpr int NHS = HOT ? kHopHotSp : 1, NHE = HOT ? kHopHotE : 1;
    extern __shared__ float lds[];
    const HopAcc L = hop_acc(a.num_spatial, a.num_edges, a.H, a.D);
    float* w_lds = lds;                               // [D][HT][HT]
    float* st_dy = w_lds + a.D * HT * HT;             // [HT][kStage]  bias gradient / path length of the staged positions
    float* st_m = st_dy + kStage * HT;                // [min(D, DC)][HT][kStage]  averaged embeddings of the hops of a pass
    float* acc = st_m + kStage * HT * min(a.D, DC);   // [L.total()]
    float* acc_sp = acc;
    float* acc_e = acc_sp + L.n_sp;
    float* acc_v = acc_e + L.n_e;
    float* acc_w = acc_v + L.n_v;
    float* e_lds = acc + ((L.total() + 3) & ~3);      // [num_edges][HT] with TAB_LDS
    if (!WS) load_hop_weight<T, HT>(a, w_lds);
    if (TAB_LDS) load_table<T, HT>(a.edge_table, a.num_edges, a.H, e_lds);
    for (int k = threadIdx.x; k < L.total(); k += 256) acc[k] = 0.f;
    __syncthreads();
    const int S1 = a.s + 1, H = a.H;
    const int64_t plane = (int64_t)S1 * S1;
    const int64_t total = (int64_t)a.b * plane;
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    const float inv_f = 1.f / (float)a.F;
    const T* e_tab = reinterpret_cast<const T*>(a.edge_table);
    float hot_sp[NHS][HT], hot_e[NHE][HT];
#pragma unroll
    for (int h = 0; h < HT; ++h) {
#pragma unroll
        for (int r = 0; r < NHS; ++r) hot_sp[r][h] = 0.f;
#pragma unroll
        for (int r = 0; r < NHE; ++r) hot_e[r][h] = 0.f;
    }
    for (int dc = 0; dc < a.D || dc == 0; dc += DC) {          // one walk per DC hops (one walk when D <= DC)
        float wsum[DC][EPL];
#pragma unroll
        for (int u = 0; u < DC; ++u)
#pragma unroll
            for (int e = 0; e < EPL; ++e) wsum[u][e] = 0.f;
        const int64_t stride = (int64_t)gridDim.x * 256;
        const HopPos step = hop_pos(stride, S1);
        HopPos ps = hop_pos((int64_t)blockIdx.x * 256 + threadIdx.x, S1);
        for (int64_t t0 = (int64_t)blockIdx.x * 256; t0 < total; t0 += stride, hop_advance(ps, step, S1)) {
            const int64_t t = t0 + threadIdx.x;
            const bool valid = t < total;
            const int64_t g = valid ? ps.g : 0;
            const int i = valid ? ps.i : 0, j = valid ? ps.j : 0, ij = i * S1 + j;
            const bool inner = valid && i >= 1 && j >= 1;
            const int64_t pos = inner ? (g * a.s + (i - 1)) * a.s + (j - 1) : 0;
            float dy[HT];
#pragma unroll
            for (int h = 0; h < HT; ++h) dy[h] = 0.f;
            if (valid) {
                const T* dg = dout + g * H * plane + ij;
                const int sp = inner ? clamp_id(a.spatial_pos[pos], a.num_spatial) : 0;
                const float inv_hops = 1.f / (float)hop_count(sp, a.max_dist);
                float d[HT];
#pragma unroll
                for (int h = 0; h < HT; ++h) d[h] = h < H ? ldf(dg + h * plane) : 0.f;
                if (dc == 0) {                                              // table gradients: first walk only
                    if (HOT && inner) {
#pragma unroll
                        for (int r = 0; r < NHS; ++r) {
                            const float hit = sp == r + 1 ? 1.f : 0.f;
#pragma unroll
                            for (int h = 0; h < HT; ++h) hot_sp[r][h] += hit * d[h];
                        }
                    }
                    const bool cold = inner && (HOT ? sp > NHS : sp > 0);   // row 0 = padding index
#pragma unroll
                    for (int h = 0; h < HT; ++h) {
                        if (h < H && d[h] != 0.f) {
                            if (cold) atomicAdd(&acc_sp[sp * H + h], d[h]);
                            if (!inner) atomicAdd(&acc_v[h], d[h]);
                        }
                    }
                }
#pragma unroll
                for (int h = 0; h < HT; ++h) dy[h] = inner ? d[h] * inv_hops : 0.f;
            }
            // positions without gradient (masked entries, the rows and columns of padding nodes: exact zeros from the
            // attention's backward) add nothing to any sum: their lanes sit the hop work out, a wave of them skips it
            bool nz = false;
#pragma unroll
            for (int h = 0; h < HT; ++h) nz = nz || dy[h] != 0.f;
            const bool wave_nz = __any(nz);
#pragma unroll
            for (int h = 0; h < HT; ++h) st_dy[h * kStage + threadIdx.x] = dy[h];
            // the first feature's id of every hop of this pass, fetched whether or not the position carries a gradient:
            // behind the branch these loads would wait for the gradient's own loads to return
            int64_t id0[DC];
#pragma unroll
            for (int u = 0; u < DC; ++u) id0[u] = dc + u < a.D && a.s > 0 ? a.edge_input[(pos * a.D0 + dc + u) * a.F] : 0;   // s = 0: no ids at all
#pragma unroll
            for (int u = 0; u < DC; ++u) {
                const int dd = dc + u;
                if (dd < a.D) {                                              // uniform over the workgroup
                    float m[HT];
#pragma unroll
                    for (int h = 0; h < HT; ++h) m[h] = 0.f;
                    if (nz) {
                        // gradient of the averaged embedding, handed to the F edge-table rows it was averaged from
                        const float* w = w_lds + dd * HT * HT;
                        float dm[HT];
#pragma unroll
                        for (int h0 = 0; h0 < HT; ++h0) {
                            float x = 0.f;
#pragma unroll
                            for (int h = 0; h < HT; ++h) x += (WS ? w_at(wq, dd * 64 + h0 * 8 + h) : w[h0 * HT + h]) * dy[h];
                            dm[h0] = x * inv_f;
                        }
                        const int64_t* ids = a.edge_input + (pos * a.D0 + dd) * a.F;
                        for (int f = 0; f < a.F; ++f) {
                            const int id = clamp_id(f == 0 ? id0[u] : ids[f], a.num_edges);
#pragma unroll
                            for (int h = 0; h < HT; ++h) {                   // the averaged embedding itself (:129)
                                if (TAB_LDS) m[h] += e_lds[id * HT + h];
                                else if (h < H) m[h] += ldf(e_tab + id * H + h);
                            }
                            if (HOT) {
#pragma unroll
                                for (int r = 0; r < NHE; ++r) {
                                    const float hit = id == r + 1 ? 1.f : 0.f;
#pragma unroll
                                    for (int h0 = 0; h0 < HT; ++h0) hot_e[r][h0] += hit * dm[h0];
                                }
                            }
                            if (HOT ? id > NHE : id > 0) {                   // row 0 = padding index
#pragma unroll
                                for (int h0 = 0; h0 < HT; ++h0)
                                    if (h0 < H && dm[h0] != 0.f) atomicAdd(&acc_e[id * H + h0], dm[h0]);
                            }
                        }
#pragma unroll
                        for (int h = 0; h < HT; ++h) m[h] *= inv_f;
                    }
#pragma unroll
                    for (int h = 0; h < HT; ++h) st_m[(u * HT + h) * kStage + threadIdx.x] = m[h];
                }
            }
            wave_sync_lds();                 // a wave reads back only what its own lanes staged: no workgroup barrier
            // lane owns entries (h0, h) = divmod(lane + 64 e, HT) of the hop matrices; its wave's 64 positions
            const int nu = min(DC, a.D - dc);
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                if (!wave_nz) break;                                         // uniform over the wave: its 64 positions add nothing
                const int idx = lane + 64 * e;
                const float4* pm = reinterpret_cast<const float4*>(st_m + (idx / HT) * kStage + wave * 64);
                const float4* pd = reinterpret_cast<const float4*>(st_dy + (idx % HT) * kStage + wave * 64);
#pragma unroll 2
                for (int p = 0; p < 16; ++p) {
                    const float4 dd4 = pd[p];
#pragma unroll
                    for (int u = 0; u < DC; ++u) {
                        if (u < nu) {                                        // uniform over the workgroup
                            const float4 mm = pm[u * (HT * kStage / 4) + p];
                            float x = wsum[u][e];
                            x += mm.x * dd4.x;
                            x += mm.y * dd4.y;
                            x += mm.z * dd4.z;
                            x += mm.w * dd4.w;
                            wsum[u][e] = x;
                        }
                    }
                }
            }
            wave_sync_lds();                 // the reads are done before the next pass stages over them
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
    if (HOT) {
        // the wave's sums of the ids kept in registers
#pragma unroll
        for (int h = 0; h < HT; ++h) {
#pragma unroll
            for (int r = 0; r < NHS; ++r) {
                float x = hot_sp[r][h];
#pragma unroll
                for (int off = 32; off >= 1; off >>= 1) x += __shfl_xor(x, off);
                if (lane == 0 && h < H && r + 1 < a.num_spatial) atomicAdd(&acc_sp[(r + 1) * H + h], x);
            }
#pragma unroll
            for (int r = 0; r < NHE; ++r) {
                float x = hot_e[r][h];
#pragma unroll
                for (int off = 32; off >= 1; off >>= 1) x += __shfl_xor(x, off);
                if (lane == 0 && h < H && r + 1 < a.num_edges) atomicAdd(&acc_e[(r + 1) * H + h], x);
            }
        }
    }
    __syncthreads();
    for (int k = threadIdx.x; k < L.total(); k += 256) partial[(int64_t)blockIdx.x * L.total() + k] = acc[k];
}

// Sum of the workgroup partials in a fixed order: 64 slices of the workers per entry, then the slices.
// Four entries per workgroup; the workgroups past the last entry clear the hop matrices that are not in use.
template <typename T>
__global__ __launch_bounds__(256) void k_multi_hop_reduce(const float* __restrict__ partial, int workers, HopAcc L, int H,
                                                          T* __restrict__ d_sp, T* __restrict__ d_e, T* __restrict__ d_v,
                                                          T* __restrict__ d_w_used, int64_t n_w_all) {
    __shared__ float part[64][4];
    const int n = L.total();
    const int n_groups = (n + 3) / 4;
    if ((int)blockIdx.x >= n_groups) {
        const int64_t k = (int64_t)(blockIdx.x - n_groups) * 256 + threadIdx.x;
        if (k < n_w_all - L.n_w) stf(d_w_used + L.n_w + k, 0.f);
        return;
    }
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
    if (k < L.n_sp) stf(d_sp + k, t);
    else if (k < L.n_sp + L.n_e) stf(d_e + (k - L.n_sp), t);
    else if (k < L.n_sp + L.n_e + L.n_v) stf(d_v + (k - L.n_sp - L.n_e), t);
    else stf(d_w_used + (k - L.n_sp - L.n_e - L.n_v), t);
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
constexpr int kGeiMaxNodes = 256;
constexpr int kGeiFar = 510;

template <typename FeatT, int MAXN>
__global__ __launch_bounds__(128) void k_gen_edge_input(const int32_t* __restrict__ path, const FeatT* __restrict__ feat,
                                                        const int32_t* __restrict__ n_nodes, int n_max, int F, int max_dist,
                                                        int64_t total, int64_t* __restrict__ out) {
    __shared__ uint8_t stack[MAXN][128];                  // [depth][thread]: a thread's entries sit in its own bank column
    const int64_t t = (int64_t)blockIdx.x * 128 + threadIdx.x;
    if (t >= total) return;
    const int64_t plane = (int64_t)n_max * n_max;
    const int64_t g = t / plane;
    const int ij = (int)(t - g * plane), i = ij / n_max, j = ij - i * n_max;
    const int n = n_nodes ? min(max(n_nodes[g], 0), n_max) : n_max;      // a count outside [0, n_max] is clamped
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
            if (k < 0 || k >= n || depth >= MAXN) {        // a direct edge: the next hop (:89)
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
    const size_t w_bytes = sizeof(float) * (size_t)D * HT * HT;
    if (w_bytes > 32 * 1024) {
        set_error("tgt_graph_attn_bias_multi_hop_fwd: %d hop matrices of %d heads exceed the 32 KB kept on chip", D, H);
        return TGT_ERR_UNSUPPORTED;
    }
    const size_t tab_bytes = sizeof(float) * (size_t)(num_spatial + num_edges) * HT;
    const bool tab_lds = w_bytes + tab_bytes <= 48 * 1024;
    const size_t lds = w_bytes + (tab_lds ? tab_bytes : 0);
    HopArgs a{d_attn_bias, d_spatial_pos, d_edge_input, d_spatial_table, d_edge_table, d_edge_dis_weight, d_virtual_dist,
              b, s, H, F, D0, D, num_spatial, num_edges, multi_hop_max_dist};
    const int64_t total = (int64_t)b * (s + 1) * (s + 1);
    const dim3 grid((unsigned)std::min<int64_t>((total + 255) / 256, 8192));
    hipStream_t st = (hipStream_t)stream;
    KernelTimer timer(KS_GRAPH_BIAS_FWD, st);
    const bool ws = H == 8 && ((uintptr_t)d_edge_dis_weight & 3) == 0;
#define TGT_HOP_FWD2(T, HTV, TL, WSV) \
    hipLaunchKernelGGL((k_multi_hop_fwd<T, HTV, TL, WSV>), grid, dim3(256), lds, st, a, (const T*)d_edge_dis_weight, (T*)d_out)
#define TGT_HOP_FWD(T, HTV)                                                       \
    do {                                                                          \
        if (tab_lds) TGT_HOP_FWD2(T, HTV, true, false);                           \
        else TGT_HOP_FWD2(T, HTV, false, false);                                  \
    } while (0)
    if (ws) {
        if (dtype == TGT_DTYPE_F32) { if (tab_lds) TGT_HOP_FWD2(float, 8, true, true); else TGT_HOP_FWD2(float, 8, false, true); }
        else { if (tab_lds) TGT_HOP_FWD2(mbf16, 8, true, true); else TGT_HOP_FWD2(mbf16, 8, false, true); }
    } else if (dtype == TGT_DTYPE_F32) {
        if (HT == 8) TGT_HOP_FWD(float, 8); else if (HT == 16) TGT_HOP_FWD(float, 16); else TGT_HOP_FWD(float, 32);
    } else {
        if (HT == 8) TGT_HOP_FWD(mbf16, 8); else if (HT == 16) TGT_HOP_FWD(mbf16, 16); else TGT_HOP_FWD(mbf16, 32);
    }
#undef TGT_HOP_FWD2
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
    const int DC = HT == 8 ? 8 : (HT == 16 ? 2 : 1);             // hops per walk, as instantiated below
    const size_t base_lds = sizeof(float) * ((size_t)D * HT * HT + (size_t)(1 + std::min(D, DC)) * kStage * HT + ((L.total() + 3) & ~3));
    const size_t tab_bytes = sizeof(float) * (size_t)num_edges * HT;
    const bool tab_lds = base_lds + tab_bytes <= 64 * 1024;
    const size_t lds = base_lds + (tab_lds ? tab_bytes : 0);
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
    const unsigned rgrid = (unsigned)((L.total() + 3) / 4 + (n_w_all - L.n_w + 255) / 256);
    auto launch = [&](auto kernel, auto reduce, auto* dout, auto* dsp, auto* de, auto* dv, auto* dw) -> int {
        if (lds > 48 * 1024)
            TGT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                              128 * 1024));
        hipLaunchKernelGGL(kernel, dim3(workers), dim3(256), lds, st, a, (decltype(dout))d_edge_dis_weight, dout, partial);
        hipLaunchKernelGGL(reduce, dim3(rgrid), dim3(256), 0, st, (const float*)partial, workers, L, H, dsp, de, dv, dw, n_w_all);
        return TGT_OK;
    };
    int lrc;
    // hops per walk: as many as are staged in LDS at once
    const bool ws = H == 8 && ((uintptr_t)d_edge_dis_weight & 3) == 0;
#define TGT_HOP_BWD(T, HTV, DCV)                                                                          \
    (ws && HTV == 8 ? (tab_lds ? launch(&k_multi_hop_bwd<T, 8, 8, true, true>, red, dout, dsp, de, dv, dw)        \
                               : launch(&k_multi_hop_bwd<T, 8, 8, false, true>, red, dout, dsp, de, dv, dw))      \
     : tab_lds      ? launch(&k_multi_hop_bwd<T, HTV, DCV, true, false>, red, dout, dsp, de, dv, dw)      \
                    : launch(&k_multi_hop_bwd<T, HTV, DCV, false, false>, red, dout, dsp, de, dv, dw))
    if (dtype == TGT_DTYPE_F32) {
        auto* red = &k_multi_hop_reduce<float>;
        const float* dout = (const float*)d_dout;
        float *dsp = (float*)d_dspatial_table, *de = (float*)d_dedge_table, *dv = (float*)d_dvirtual_dist,
              *dw = (float*)d_dedge_dis_weight;
        lrc = HT == 8 ? TGT_HOP_BWD(float, 8, 8) : HT == 16 ? TGT_HOP_BWD(float, 16, 2) : TGT_HOP_BWD(float, 32, 1);
    } else {
        auto* red = &k_multi_hop_reduce<mbf16>;
        const mbf16* dout = (const mbf16*)d_dout;
        mbf16 *dsp = (mbf16*)d_dspatial_table, *de = (mbf16*)d_dedge_table, *dv = (mbf16*)d_dvirtual_dist,
              *dw = (mbf16*)d_dedge_dis_weight;
        lrc = HT == 8 ? TGT_HOP_BWD(mbf16, 8, 8) : HT == 16 ? TGT_HOP_BWD(mbf16, 16, 2) : TGT_HOP_BWD(mbf16, 32, 1);
    }
#undef TGT_HOP_BWD
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
#define TGT_GEI(FEAT_, MAXN_)                                                                                              \
    hipLaunchKernelGGL((k_gen_edge_input<FEAT_, MAXN_>), grid, dim3(128), 0, st, d_path, (const FEAT_*)d_edge_feat, d_n_nodes, \
                       n_max, F, max_dist, total, d_out)
    if (n_max <= 128) {          // the stack of a walk is as deep as the graph is large
        if (feat_is_int64) TGT_GEI(int64_t, 128);
        else TGT_GEI(int32_t, 128);
    } else {
        if (feat_is_int64) TGT_GEI(int64_t, kGeiMaxNodes);
        else TGT_GEI(int32_t, kGeiMaxNodes);
    }
#undef TGT_GEI
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

}  // extern "C"
