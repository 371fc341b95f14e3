// The projections on either side of the attention: y_j = x W_j^T + b_j for up to
// three weights in one pass over x, and the backward of that.
//
// Replaces linear_q / linear_k / linear_v and output_layer of MultiHeadAttention
// (models/graphormer_dist_node_level.py:233-241 construct them, :255-257 and :271
// apply them; same module in models/gt_dist_node_level.py and
// models/graphormer_dist_graph_level.py).  In the reference these are three
// separate GEMMs that each read x, plus one for the output; their backward is two
// GEMMs and a column sum per weight.
//
// N (nodes) is large and the feature widths are small (64 in the node-level
// configurations), so every kernel walks panels of node rows and keeps the
// weights / weight gradients on chip:
//   k_linear<DX=false>   y_j = x W_j^T + b_j         panel of 128 rows, x staged once
//   k_linear<DX=true>    dx  = sum_j dy_j W_j         same walk, W staged transposed
//   k_linear_gradw       dW_j = dy_j^T x, db_j = colsum(dy_j): each workgroup keeps a
//                        64 x 64 tile of every dW_j in registers over its share of the
//                        panels and writes one partial; the fixed-order sum of reduce.hip adds the
//                        partials in a fixed order (no atomics: results are reproducible)
// Matrix instructions: v_mfma_f32_32x32x2_f32 for float32 (exact fp32 products,
// fp32 accumulation; the 64-wide forward instead splits every float into three
// bf16 and uses the bf16 instructions, see k_linear64_split),
// v_mfma_f32_32x32x8_bf16_1k for bf16 (fp32 accumulation).
//   A 32xk : lane l holds A[l%32][k-slice of half l/32]
//   B kx32 : lane l holds B[k-slice of half l/32][l%32]
//   C 32x32: lane l, register r holds C[8*(r/4) + 4*(l/32) + r%4][l%32]
// Both operands are kept in LDS with the contraction index contiguous, and half
// l/32 of the wave takes the contraction indices [half*KC/2, (half+1)*KC/2): a
// lane then fetches the operands of four (fp32) or two (bf16) instructions with one
// 16-byte LDS read.  (Any assignment of contraction indices to instructions gives
// the same product as long as A and B use the same one.)
#include "common.h"
#include <algorithm>

namespace tgt {
namespace {

typedef short short4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
struct pbf16 { uint16_t x; };

constexpr int kThreads = 256;
constexpr int kPanel = 128;     // node rows per workgroup of the forward / input-gradient kernel
constexpr int kChunk = 64;      // contraction indices per LDS stage
constexpr int kCols = 64;       // output columns per accumulation pass
constexpr int kGradRows = 64;   // node rows per step of the weight-gradient kernel
constexpr int kGradWorkers = 512;   // workgroups (partials) of the weight-gradient kernel per output tile set

template <typename T> constexpr int lds_stride(int inner) { return inner + 16 / (int)sizeof(T); }

__device__ __forceinline__ float ld1(const float* p) { return *p; }
__device__ __forceinline__ float ld1(const pbf16* p) { return __uint_as_float(((uint32_t)p->x) << 16); }
__device__ __forceinline__ void st1(float* p, float v) { *p = v; }
__device__ __forceinline__ void st1(pbf16* p, float v) {
    const __bf16 b = static_cast<__bf16>(v);
    p->x = __builtin_bit_cast(uint16_t, b);
}

__device__ __forceinline__ float16_t zero16() {
    float16_t z;
#pragma unroll
    for (int i = 0; i < 16; ++i) z[i] = 0.f;
    return z;
}

// The 16 accumulator values of a lane (rows 8*(r/4) + r%4 below its first row, one
// column) plus a bias.  All values are formed before the first store and a wave
// whose rows all exist stores without per-row branches: with a branch per store
// the compiler reuses one data register and waits for each store to finish.
template <typename T>
__device__ __forceinline__ void store_rows(T* __restrict__ out, int64_t ld, const float16_t& acc, float bias,
                                           int64_t rows_left) {
    float v[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) v[r] = acc[r] + bias;
    // a lane writes rows 0..27 below its first row and the lanes of a wave differ by 4 in rows_left:
    // 32 rows left for the first lane means every row of every lane exists
    if (__builtin_amdgcn_readfirstlane(rows_left >= 32 ? 1 : 0)) {
#pragma unroll
        for (int r = 0; r < 16; ++r) st1(out + (8 * (r >> 2) + (r & 3)) * ld, v[r]);
    } else {
#pragma unroll
        for (int r = 0; r < 16; ++r)
            if (8 * (r >> 2) + (r & 3) < rows_left) st1(out + (8 * (r >> 2) + (r & 3)) * ld, v[r]);
    }
}

// The same with an activation on top: u = acc + bias goes to out_u and act(u) to out_h.  The activation is taken of
// the value as it is stored (rounded to bf16 for bf16 outputs), so a separate activation kernel that reads out_u
// gives the same bits.
__device__ __forceinline__ float as_stored(float v, const float*) { return v; }
__device__ __forceinline__ float as_stored(float v, const pbf16*) { return static_cast<float>(static_cast<__bf16>(v)); }
template <typename T, bool RELU>
__device__ __forceinline__ void store_rows_act(T* __restrict__ out_u, T* __restrict__ out_h, int64_t ld, const float16_t& acc,
                                               float bias, int64_t rows_left) {
    float v[16], w[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        v[r] = acc[r] + bias;
        w[r] = act_value<RELU>(as_stored(v[r], out_u));
    }
    if (__builtin_amdgcn_readfirstlane(rows_left >= 32 ? 1 : 0)) {
#pragma unroll
        for (int r = 0; r < 16; ++r) st1(out_u + (8 * (r >> 2) + (r & 3)) * ld, v[r]);
#pragma unroll
        for (int r = 0; r < 16; ++r) st1(out_h + (8 * (r >> 2) + (r & 3)) * ld, w[r]);
    } else {
#pragma unroll
        for (int r = 0; r < 16; ++r)
            if (8 * (r >> 2) + (r & 3) < rows_left) {
                st1(out_u + (8 * (r >> 2) + (r & 3)) * ld, v[r]);
                st1(out_h + (8 * (r >> 2) + (r & 3)) * ld, w[r]);
            }
    }
}

// 16 bytes of src[row * ld + col ..], zero if (row, col) lies outside [0,nrows) x [0,ncols).
// The address is clamped into the array and the result selected, so the load is
// unconditional: a branch around it would make the compiler wait for every load
// before issuing the next.  nrows >= 1; ncols is a multiple of the vector width.
template <typename T>
__device__ __forceinline__ uint4 load16_clamped(const T* __restrict__ src, int64_t ld, int64_t row, int64_t nrows,
                                                int col, int ncols) {
    constexpr int VE = 16 / (int)sizeof(T);
    const int64_t rr = row < nrows ? row : nrows - 1;
    const int cc = col < ncols ? col : ncols - VE;
    return *reinterpret_cast<const uint4*>(src + rr * ld + cc);
}
__device__ __forceinline__ uint4 zero_unless(bool ok, uint4 u) {
    u.x = ok ? u.x : 0u; u.y = ok ? u.y : 0u; u.z = ok ? u.z : 0u; u.w = ok ? u.w : 0u;
    return u;
}
template <typename T>
__device__ __forceinline__ uint4 load16_or_zero(const T* __restrict__ src, int64_t ld, int64_t row, int64_t nrows,
                                                int col, int ncols) {
    return zero_unless(row < nrows && col < ncols, load16_clamped(src, ld, row, nrows, col, ncols));
}

// tile[r][c] = src[(row0 + r) * ld + col0 + c], r < R, c < 64; zero outside [0,nrows) x [0,ncols)
template <typename T, int R, int STRIDE>
__device__ __forceinline__ void stage_natural(T* __restrict__ tile, const T* __restrict__ src, int64_t ld,
                                              int64_t row0, int64_t nrows, int col0, int ncols) {
    constexpr int VE = 16 / (int)sizeof(T);
    constexpr int VPR = kChunk / VE;
    constexpr int NV = R * VPR / kThreads;
    static_assert(R * VPR % kThreads == 0, "tile shape");
    uint4 val[NV];            // all loads are issued before the first LDS write
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int v = threadIdx.x + i * kThreads, r = v / VPR, c = (v % VPR) * VE;
        val[i] = load16_or_zero(src, ld, row0 + r, nrows, col0 + c, ncols);
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int v = threadIdx.x + i * kThreads, r = v / VPR, c = (v % VPR) * VE;
        *reinterpret_cast<uint4*>(tile + r * STRIDE + c) = val[i];
    }
}

// tile[c][r] = src[(row0 + r) * ld + col0 + c], r < R, c < 64; zero outside.  Four
// lanes read 64 consecutive bytes of one source row and sixteen rows go per
// instruction, which keeps the scattered LDS writes to two per bank.
template <typename T, int R, int STRIDE>
__device__ __forceinline__ void stage_transposed(T* __restrict__ tile, const T* __restrict__ src, int64_t ld,
                                                 int64_t row0, int64_t nrows, int col0, int ncols) {
    constexpr int VE = 16 / (int)sizeof(T);
    constexpr int VPR = kChunk / VE;
    constexpr int NV = R * VPR / kThreads;
    static_assert(R % 16 == 0 && VPR % 4 == 0 && R * VPR % kThreads == 0, "tile shape");
    uint4 val[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int v = threadIdx.x + i * kThreads;
        const int cq = v & 3, r_lo = (v >> 2) & 15, rest = v >> 6;
        const int r = (rest % (R / 16)) * 16 + r_lo;
        const int c = ((rest / (R / 16)) * 4 + cq) * VE;
        val[i] = load16_or_zero(src, ld, row0 + r, nrows, col0 + c, ncols);
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int v = threadIdx.x + i * kThreads;
        const int cq = v & 3, r_lo = (v >> 2) & 15, rest = v >> 6;
        const int r = (rest % (R / 16)) * 16 + r_lo;
        const int c = ((rest / (R / 16)) * 4 + cq) * VE;
        const T* e = reinterpret_cast<const T*>(&val[i]);
#pragma unroll
        for (int t = 0; t < VE; ++t) tile[(c + t) * STRIDE + r] = e[t];
    }
}

// The same transposed tile in two steps, so that the loads of the next tile can be
// in flight during the products of the current one: fetch_t reads the thread's
// 16-byte pieces into registers, put_t scatters them into the LDS tile.
template <typename T> struct PieceRegs { uint4 v[(64 * 64 * sizeof(T)) / (16 * kThreads)]; };

template <typename T, int R>
__device__ __forceinline__ void piece_pos(int i, int& r, int& c) {
    constexpr int VE = 16 / (int)sizeof(T);
    const int v = threadIdx.x + i * kThreads;
    const int cq = v & 3, r_lo = (v >> 2) & 15, rest = v >> 6;
    r = (rest % (R / 16)) * 16 + r_lo;
    c = ((rest / (R / 16)) * 4 + cq) * VE;
}
template <typename T>
__device__ __forceinline__ void fetch_t(PieceRegs<T>& t, const T* __restrict__ src, int64_t ld, int64_t row0,
                                        int64_t nrows, int col0, int ncols) {
    constexpr int NV = (int)(sizeof(PieceRegs<T>) / 16);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        int r, c;
        piece_pos<T, 64>(i, r, c);
        t.v[i] = load16_clamped(src, ld, row0 + r, nrows, col0 + c, ncols);
    }
}
// (the pieces outside the array are zeroed here, not in fetch_t: touching the loaded
// values there would make the wave wait for the loads at once)
template <typename T, int STRIDE>
__device__ __forceinline__ void put_t(const PieceRegs<T>& t, T* __restrict__ tile, int64_t row0, int64_t nrows,
                                      int col0, int ncols) {
    constexpr int VE = 16 / (int)sizeof(T), NV = (int)(sizeof(PieceRegs<T>) / 16);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        int r, c;
        piece_pos<T, 64>(i, r, c);
        const uint4 u = zero_unless(row0 + r < nrows && col0 + c < ncols, t.v[i]);
        const T* e = reinterpret_cast<const T*>(&u);
#pragma unroll
        for (int k = 0; k < VE; ++k) tile[(c + k) * STRIDE + r] = e[k];
    }
}

// acc += A B over KC contraction indices; a, b: the lane's operand rows in LDS,
// already offset by its half's first contraction index.
template <typename T, int KC> struct Mma;
template <int KC> struct Mma<float, KC> {
    static __device__ __forceinline__ void run(const float* a, const float* b, float16_t& acc) {
#pragma unroll
        for (int i = 0; i < KC / 2; i += 4) {
            const float4 av = *reinterpret_cast<const float4*>(a + i);
            const float4 bv = *reinterpret_cast<const float4*>(b + i);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av.x, bv.x, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av.y, bv.y, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av.z, bv.z, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av.w, bv.w, acc, 0, 0, 0);
        }
    }
};
template <int KC> struct Mma<pbf16, KC> {
    static __device__ __forceinline__ void run(const pbf16* a, const pbf16* b, float16_t& acc) {
#pragma unroll
        for (int i = 0; i < KC / 2; i += 8) {
            const uint4 av = *reinterpret_cast<const uint4*>(a + i);
            const uint4 bv = *reinterpret_cast<const uint4*>(b + i);
            acc = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(__builtin_bit_cast(short4_t, make_uint2(av.x, av.y)),
                                                           __builtin_bit_cast(short4_t, make_uint2(bv.x, bv.y)),
                                                           acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(__builtin_bit_cast(short4_t, make_uint2(av.z, av.w)),
                                                           __builtin_bit_cast(short4_t, make_uint2(bv.z, bv.w)),
                                                           acc, 0, 0, 0);
        }
    }
};

struct LinArgs {
    const void* A[3];      // forward: A[0] = x [N, K]; input gradient: A[j] = dy_j [N, M]
    const void* W[3];      // [M, K] row-major (nn.Linear.weight)
    const void* bias[3];   // forward only; entries may be null
    void* out[3];          // forward: y_j [N, M]; input gradient: out[0] = dx [N, K]
    int nw;
    int64_t N;
    int K, M;
};

// One workgroup per panel of 128 node rows; wave w owns rows [32w, 32w+32) and two
// 32-column blocks of the current 64 output columns.
template <typename T, bool DX>
__global__ __launch_bounds__(kThreads) void k_linear(LinArgs a) {
    constexpr int S = lds_stride<T>(kChunk);
    __shared__ __align__(16) T tA[kPanel * S];
    __shared__ __align__(16) T tB[kCols * S];
    const int L = DX ? a.M : a.K;          // contraction length
    const int C = DX ? a.K : a.M;          // output columns
    const int n_out = DX ? 1 : a.nw, n_src = DX ? a.nw : 1;
    const int64_t row0 = (int64_t)blockIdx.x * kPanel;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, l32 = lane & 31, h = lane >> 5;
    const bool a_resident = (n_src == 1 && L <= kChunk);   // the source panel is staged once for all outputs
    bool a_loaded = false;
    for (int o = 0; o < n_out; ++o) {
        for (int c0 = 0; c0 < C; c0 += kCols) {
            float16_t acc0 = zero16(), acc1 = zero16();
            for (int s = 0; s < n_src; ++s) {
                const T* W = reinterpret_cast<const T*>(a.W[DX ? s : o]);
                for (int l0 = 0; l0 < L; l0 += kChunk) {
                    __syncthreads();
                    if (!(a_resident && a_loaded)) {
                        stage_natural<T, kPanel, S>(tA, reinterpret_cast<const T*>(a.A[s]), L, row0, a.N, l0, L);
                        a_loaded = true;
                    }
                    if (!DX) stage_natural<T, kCols, S>(tB, W, a.K, c0, a.M, l0, a.K);       // rows = output columns
                    else stage_transposed<T, kChunk, S>(tB, W, a.K, l0, a.M, c0, a.K);       // rows of W = contraction
                    __syncthreads();
                    const T* ap = tA + (wave * 32 + l32) * S + h * (kChunk / 2);
                    Mma<T, kChunk>::run(ap, tB + l32 * S + h * (kChunk / 2), acc0);
                    Mma<T, kChunk>::run(ap, tB + (32 + l32) * S + h * (kChunk / 2), acc1);
                }
            }
            T* out = reinterpret_cast<T*>(a.out[o]);
            const T* bias = DX ? nullptr : reinterpret_cast<const T*>(a.bias[o]);
#pragma unroll
            for (int cb = 0; cb < 2; ++cb) {
                const int col = c0 + 32 * cb + l32;
                if (col >= C) continue;
                const float bv = bias ? ld1(bias + col) : 0.f;
                const float16_t& acc = cb ? acc1 : acc0;
                const int64_t first = row0 + wave * 32 + 4 * h;
                store_rows<T>(out + first * C + col, C, acc, bv, a.N - first);
            }
        }
    }
}

// A 64-row x 64-column tile on its way from global memory to LDS: each thread
// holds 16-byte pieces in registers, so the loads of the next panel can be in
// flight while the current one is multiplied.
template <typename T> struct TileRegs { uint4 v[(64 * 64 * sizeof(T)) / (16 * kThreads)]; };

template <typename T>
__device__ __forceinline__ void tile_fetch(TileRegs<T>& t, const T* __restrict__ src, int64_t row0, int64_t nrows) {
    constexpr int VE = 16 / (int)sizeof(T), VPR = 64 / VE, NV = (int)(sizeof(TileRegs<T>) / 16);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int v = threadIdx.x + i * kThreads, r = v / VPR, c = (v % VPR) * VE;
        t.v[i] = load16_clamped(src, 64, row0 + r, nrows, c, 64);     // rows past the end repeat the last row: their
                                                                      // products land in output rows that are not stored
    }
}
template <typename T, int STRIDE>
__device__ __forceinline__ void tile_put(const TileRegs<T>& t, T* __restrict__ tile) {
    constexpr int VE = 16 / (int)sizeof(T), VPR = 64 / VE, NV = (int)(sizeof(TileRegs<T>) / 16);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int v = threadIdx.x + i * kThreads, r = v / VPR, c = (v % VPR) * VE;
        *reinterpret_cast<uint4*>(tile + r * STRIDE + c) = t.v[i];
    }
}

// in_features = out_features = 64 (the node-level models).  The weights stay in LDS
// for the life of the workgroup, which walks panels of 64 node rows; the next
// panel's rows are fetched into registers while the current panel is multiplied.
// Wave w owns the 32 x 32 block (w/2, w%2) of every 64 x 64 output tile.
// ACT (forward with one weight only): 1 = GELU, 2 = RELU: out[0] gets u = x W^T + b and out[1] the activation of u.
template <typename T, bool DX, int NW, int ACT = 0>
__global__ __launch_bounds__(kThreads) void k_linear64(LinArgs a) {
    static_assert(ACT == 0 || (!DX && NW == 1), "the activation rides on a forward with one weight");
    constexpr int S = lds_stride<T>(64);
    constexpr int NA = DX ? NW : 1;      // source tiles per panel
    constexpr int NO = DX ? 1 : NW;      // output tiles per panel
    extern __shared__ __align__(16) unsigned char smem[];
    T* tW = reinterpret_cast<T*>(smem);          // [NW][64][S]
    T* tA = tW + NW * 64 * S;                    // [NA][64][S]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, l32 = lane & 31, h = lane >> 5;
    const int rb = wave >> 1, cb = wave & 1;
    const int64_t n_panels = (a.N + 63) / 64;
    TileRegs<T> next[NA];
    int64_t p = blockIdx.x;
    if (p < n_panels) {
#pragma unroll
        for (int s = 0; s < NA; ++s) tile_fetch(next[s], reinterpret_cast<const T*>(a.A[s]), p * 64, a.N);
    }
#pragma unroll
    for (int j = 0; j < NW; ++j) {
        const T* W = reinterpret_cast<const T*>(a.W[j]);
        if (!DX) stage_natural<T, 64, S>(tW + j * 64 * S, W, 64, 0, 64, 0, 64);        // rows = output columns
        else stage_transposed<T, 64, S>(tW + j * 64 * S, W, 64, 0, 64, 0, 64);         // rows = columns of W
    }
    float bv[NO];
#pragma unroll
    for (int o = 0; o < NO; ++o) {
        const T* bias = DX ? nullptr : reinterpret_cast<const T*>(a.bias[o]);
        bv[o] = bias ? ld1(bias + 32 * cb + l32) : 0.f;
    }
    // use the bias values once here, so that the wait for their loads stands before the loop and
    // not inside it, where it would also wait for the prefetched panel
#pragma unroll
    for (int o = 0; o < NO; ++o) asm volatile("" ::"v"(bv[o]));
    for (; p < n_panels; p += gridDim.x) {
        __syncthreads();                 // the previous panel has been read
#pragma unroll
        for (int s = 0; s < NA; ++s) tile_put<T, S>(next[s], tA + s * 64 * S);
        __syncthreads();
        if (p + gridDim.x < n_panels) {
#pragma unroll
            for (int s = 0; s < NA; ++s)
                tile_fetch(next[s], reinterpret_cast<const T*>(a.A[s]), (p + gridDim.x) * 64, a.N);
        }
#pragma unroll
        for (int o = 0; o < NO; ++o) {
            float16_t acc = zero16();
#pragma unroll
            for (int s = 0; s < NA; ++s)
                Mma<T, 64>::run(tA + (s * 64 + 32 * rb + l32) * S + h * 32,
                                tW + ((DX ? s : o) * 64 + 32 * cb + l32) * S + h * 32, acc);
            const int64_t at = (p * 64 + 32 * rb + 4 * h) * 64 + 32 * cb + l32;
            T* out = reinterpret_cast<T*>(a.out[o]) + at;
            if constexpr (ACT != 0) store_rows_act<T, ACT == 2>(out, reinterpret_cast<T*>(a.out[1]) + at, 64, acc, bv[o], a.N - (p * 64 + 32 * rb + 4 * h));
            else store_rows<T>(out, 64, acc, bv[o], a.N - (p * 64 + 32 * rb + 4 * h));
        }
    }
}

// ---------------------------------------------------------------------------
// float32 at the bf16 matrix rate.  A float is the exact sum of three bf16 numbers: hi = its upper 16 bits (sign,
// exponent, the first 8 bits of the significand), mid = the upper 16 bits of x - hi, lo = x - hi - mid (what is left
// has at most 8 significant bits; every subtraction is exact).  So x * w = hi*hi + hi*mid + mid*hi + mid*mid + hi*lo +
// lo*hi + terms below 2^-24: six v_mfma_f32_32x32x16_bf16 (fp32 accumulation) give the float32 product to a few 2^-23,
// and take 0.4 of the time of the eight v_mfma_f32_32x32x2_f32 they replace (measured on this part: 16.8 ns against
// 30.4 ns per instruction).  Cutting the words costs four full-rate vector instructions per value and one byte
// permute per pair and plane; the rounding conversions (v_cvt_pk_bf16_f32) it was first written with run at a quarter
// of that rate and made the split the longest part of the backward.  The weights are split once per workgroup into
// three bf16 planes in LDS; the node rows stay float32 in LDS and are split in registers when a wave loads them.
// ---------------------------------------------------------------------------
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));

// the three parts as float32 words: each is a bf16 in its upper half (the lower half is zero)
__device__ __forceinline__ void split3(float x, uint32_t& hi, uint32_t& mid, uint32_t& lo) {
    hi = __float_as_uint(x) & 0xffff0000u;
    const float r1 = x - __uint_as_float(hi);
    mid = __float_as_uint(r1) & 0xffff0000u;
    lo = __float_as_uint(r1 - __uint_as_float(mid));
}
__device__ __forceinline__ __bf16 upper_bf16(uint32_t w) { return __builtin_bit_cast(__bf16, (uint16_t)(w >> 16)); }
// the upper halves of eight such words as one matrix operand
__device__ __forceinline__ bf16x8_t pack8(const uint32_t (&w)[8]) {
    uint4 u;
    u.x = __builtin_amdgcn_perm(w[1], w[0], 0x07060302u);
    u.y = __builtin_amdgcn_perm(w[3], w[2], 0x07060302u);
    u.z = __builtin_amdgcn_perm(w[5], w[4], 0x07060302u);
    u.w = __builtin_amdgcn_perm(w[7], w[6], 0x07060302u);
    return __builtin_bit_cast(bf16x8_t, u);
}

constexpr int kPlaneStride = 72;                       // bf16 per row of a weight plane (64 + 8 of padding)
constexpr int kPlaneElems = 64 * kPlaneStride;

struct Split32 { bf16x8_t hi[4], mid[4], lo[4]; };    // the 32 contraction indices of a lane's half row

// row: 32 consecutive floats in LDS
__device__ __forceinline__ void load_split(Split32& f, const float* row) {
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const float4 u0 = *reinterpret_cast<const float4*>(row + 8 * t);
        const float4 u1 = *reinterpret_cast<const float4*>(row + 8 * t + 4);
        const float v[8] = {u0.x, u0.y, u0.z, u0.w, u1.x, u1.y, u1.z, u1.w};
        uint32_t a[8], b[8], c[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) split3(v[i], a[i], b[i], c[i]);
        f.hi[t] = pack8(a); f.mid[t] = pack8(b); f.lo[t] = pack8(c);
    }
}

// acc += x_rows W_rows^T over the lane's 32 contraction indices; w: the lane's row in plane 0
__device__ __forceinline__ void mma_split(const Split32& x, const __bf16* w, float16_t& acc) {
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const bf16x8_t wh = *reinterpret_cast<const bf16x8_t*>(w + 8 * t);
        const bf16x8_t wm = *reinterpret_cast<const bf16x8_t*>(w + kPlaneElems + 8 * t);
        const bf16x8_t wl = *reinterpret_cast<const bf16x8_t*>(w + 2 * kPlaneElems + 8 * t);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x.lo[t], wh, acc, 0, 0, 0);     // small terms first
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x.hi[t], wl, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x.mid[t], wm, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x.mid[t], wh, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x.hi[t], wm, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x.hi[t], wh, acc, 0, 0, 0);
    }
}

// Same walk as k_linear64 (64 -> 64 features, weights resident, 64-row panels, register prefetch) for float32
// through the split.  Weight planes in LDS: [NW][3][64][kPlaneStride] bf16; node rows: [NA][64][68] float.
template <bool DX, int NW, int ACT = 0>
__global__ __launch_bounds__(kThreads) void k_linear64_split(LinArgs a) {
    static_assert(ACT == 0 || (!DX && NW == 1), "the activation rides on a forward with one weight");
    constexpr int S = lds_stride<float>(64);
    constexpr int NA = DX ? NW : 1;
    constexpr int NO = DX ? 1 : NW;
    extern __shared__ __align__(16) unsigned char smem[];
    __bf16* tW = reinterpret_cast<__bf16*>(smem);
    float* tA = reinterpret_cast<float*>(smem + (size_t)NW * 3 * kPlaneElems * sizeof(__bf16));
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, l32 = lane & 31, h = lane >> 5;
    const int rb = wave >> 1, cb = wave & 1;
    const int64_t n_panels = (a.N + 63) / 64;
    TileRegs<float> next[NA];
    int64_t p = blockIdx.x;
    if (p < n_panels) {
#pragma unroll
        for (int s = 0; s < NA; ++s) tile_fetch(next[s], reinterpret_cast<const float*>(a.A[s]), p * 64, a.N);
    }
    {   // weights: 16 elements per thread and weight, split into the three planes
        uint4 raw[NW][4];
#pragma unroll
        for (int j = 0; j < NW; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int v = threadIdx.x + i * kThreads;                       // 16-byte piece: row v / 16, columns 4 (v % 16) ..
                raw[j][i] = *reinterpret_cast<const uint4*>(reinterpret_cast<const float*>(a.W[j]) + v * 4);
            }
#pragma unroll
        for (int j = 0; j < NW; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int v = threadIdx.x + i * kThreads, r = v >> 4, c = (v & 15) * 4;
                const float* e = reinterpret_cast<const float*>(&raw[j][i]);
                __bf16* plane = tW + (size_t)j * 3 * kPlaneElems;
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    uint32_t w0, w1, w2;
                    split3(e[t], w0, w1, w2);
                    const __bf16 x0 = upper_bf16(w0), x1 = upper_bf16(w1), x2 = upper_bf16(w2);
                    // forward: plane row = output column r, contraction index c + t; input gradient: row = c + t, index r
                    const int at = DX ? (c + t) * kPlaneStride + r : r * kPlaneStride + c + t;
                    plane[at] = x0;
                    plane[kPlaneElems + at] = x1;
                    plane[2 * kPlaneElems + at] = x2;
                }
            }
    }
    float bv[NO];
#pragma unroll
    for (int o = 0; o < NO; ++o) {
        const float* bias = DX ? nullptr : reinterpret_cast<const float*>(a.bias[o]);
        bv[o] = bias ? bias[32 * cb + l32] : 0.f;
    }
#pragma unroll
    for (int o = 0; o < NO; ++o) asm volatile("" ::"v"(bv[o]));      // wait for the bias loads here, not in the loop
    for (; p < n_panels; p += gridDim.x) {
        __syncthreads();
#pragma unroll
        for (int s = 0; s < NA; ++s) tile_put<float, S>(next[s], tA + s * 64 * S);
        __syncthreads();
        if (p + gridDim.x < n_panels) {
#pragma unroll
            for (int s = 0; s < NA; ++s)
                tile_fetch(next[s], reinterpret_cast<const float*>(a.A[s]), (p + gridDim.x) * 64, a.N);
        }
        if (!DX) {
            Split32 x;
            load_split(x, tA + (32 * rb + l32) * S + h * 32);
#pragma unroll
            for (int o = 0; o < NW; ++o) {
                float16_t acc = zero16();
                mma_split(x, tW + (size_t)o * 3 * kPlaneElems + (32 * cb + l32) * kPlaneStride + h * 32, acc);
                const int64_t at = (p * 64 + 32 * rb + 4 * h) * 64 + 32 * cb + l32;
                float* out = reinterpret_cast<float*>(a.out[o]) + at;
                if constexpr (ACT != 0) store_rows_act<float, ACT == 2>(out, reinterpret_cast<float*>(a.out[1]) + at, 64, acc, bv[o], a.N - (p * 64 + 32 * rb + 4 * h));
                else store_rows<float>(out, 64, acc, bv[o], a.N - (p * 64 + 32 * rb + 4 * h));
            }
        } else {
            float16_t acc = zero16();
#pragma unroll
            for (int s = 0; s < NW; ++s) {
                Split32 x;
                load_split(x, tA + (s * 64 + 32 * rb + l32) * S + h * 32);
                mma_split(x, tW + (size_t)s * 3 * kPlaneElems + (32 * cb + l32) * kPlaneStride + h * 32, acc);
            }
            float* out = reinterpret_cast<float*>(a.out[0]) + (p * 64 + 32 * rb + 4 * h) * 64 + 32 * cb + l32;
            store_rows<float>(out, 64, acc, 0.f, a.N - (p * 64 + 32 * rb + 4 * h));
        }
    }
}

int num_cus() {
    static int cus = 0;
    if (cus == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
            cus = n;
        else
            cus = 256;
    }
    return cus;
}

template <typename T, bool DX, int NW, int ACT = 0>
int launch_linear64(const LinArgs& a, hipStream_t st) {
    constexpr int NA = DX ? NW : 1;
    // float32 forward goes through the three-way bf16 split.  The input gradient keeps the float32 matrix
    // instructions: it would split three source tiles per panel and stage transposed weight planes, and measured
    // slower at 64 K rows (28 against 26 us) though faster at 870 K (280 against 297 us).
    constexpr bool kSplit = sizeof(T) == 4 && !DX;
    const size_t lds = kSplit ? (size_t)NW * 3 * kPlaneElems * 2 + sizeof(float) * (size_t)NA * 64 * lds_stride<float>(64)
                              : sizeof(T) * (size_t)(NW + NA) * 64 * lds_stride<T>(64);
    const void* fn = kSplit ? reinterpret_cast<const void*>(&k_linear64_split<DX, NW, ACT>)
                            : reinterpret_cast<const void*>(&k_linear64<T, DX, NW, ACT>);
    static bool raised = false;
    if (!raised && lds > 48 * 1024) {
        TGT_HIP_CHECK(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        raised = true;
    }
    const int64_t n_panels = (a.N + 63) / 64;
    const int per_cu = (int)std::max<size_t>(1, std::min<size_t>(4, (size_t)(160 * 1024) / lds));
    const unsigned grid = (unsigned)std::min<int64_t>(n_panels, (int64_t)num_cus() * per_cu);
    if (kSplit) hipLaunchKernelGGL((k_linear64_split<DX, NW, ACT>), dim3(grid), dim3(kThreads), lds, st, a);
    else hipLaunchKernelGGL((k_linear64<T, DX, NW, ACT>), dim3(grid), dim3(kThreads), lds, st, a);
    return TGT_OK;
}

template <typename T, bool DX>
int launch_linear(const LinArgs& a, hipStream_t st) {
    if (a.K == 64 && a.M == 64) {
        if (a.nw == 1) return launch_linear64<T, DX, 1>(a, st);
        if (a.nw == 2) return launch_linear64<T, DX, 2>(a, st);
        return launch_linear64<T, DX, 3>(a, st);
    }
    hipLaunchKernelGGL((k_linear<T, DX>), dim3((unsigned)((a.N + kPanel - 1) / kPanel)), dim3(kThreads), 0, st, a);
    return TGT_OK;
}

struct GradWArgs {
    const void* x;         // [N, K]
    const void* dy[3];     // [N, M]
    float* partial;        // [workers][nw][M*K + M]
    int64_t N;
    int K, M;
};

// blockIdx.y picks a 64 x 64 tile (mt, kt) of the weight gradients, blockIdx.x a
// worker; wave w owns the 32 x 32 block (w/2, w%2) of the tile for every weight.
template <typename T, int NW>
__global__ __launch_bounds__(kThreads) void k_linear_gradw(GradWArgs a) {
    constexpr int S = lds_stride<T>(kGradRows);
    extern __shared__ __align__(16) unsigned char smem[];
    T* tX = reinterpret_cast<T*>(smem);          // [64 k][64 nodes]
    T* tD = tX + kCols * S;                      // NW x [64 m][64 nodes]
    const int kt_n = (a.K + kCols - 1) / kCols;
    const int mt = blockIdx.y / kt_n, kt = blockIdx.y % kt_n;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, l32 = lane & 31, h = lane >> 5;
    const int mi = wave >> 1, ki = wave & 1;
    float16_t acc[NW];
#pragma unroll
    for (int j = 0; j < NW; ++j) acc[j] = zero16();
    float colsum = 0.f;
    static_assert(kGradRows == 64, "piece layout");
    const int64_t n_panels = (a.N + kGradRows - 1) / kGradRows;
    PieceRegs<T> nx, nd[NW];
    int64_t p = blockIdx.x;
    if (p < n_panels) {
        fetch_t(nx, reinterpret_cast<const T*>(a.x), a.K, p * kGradRows, a.N, kt * kCols, a.K);
#pragma unroll
        for (int j = 0; j < NW; ++j)
            fetch_t(nd[j], reinterpret_cast<const T*>(a.dy[j]), a.M, p * kGradRows, a.N, mt * kCols, a.M);
    }
    for (; p < n_panels; p += gridDim.x) {
        __syncthreads();
        put_t<T, S>(nx, tX, p * kGradRows, a.N, kt * kCols, a.K);
#pragma unroll
        for (int j = 0; j < NW; ++j) put_t<T, S>(nd[j], tD + j * kCols * S, p * kGradRows, a.N, mt * kCols, a.M);
        __syncthreads();
        if (p + gridDim.x < n_panels) {
            const int64_t q = p + gridDim.x;
            fetch_t(nx, reinterpret_cast<const T*>(a.x), a.K, q * kGradRows, a.N, kt * kCols, a.K);
#pragma unroll
            for (int j = 0; j < NW; ++j)
                fetch_t(nd[j], reinterpret_cast<const T*>(a.dy[j]), a.M, q * kGradRows, a.N, mt * kCols, a.M);
        }
        const T* bp = tX + (32 * ki + l32) * S + h * (kGradRows / 2);
#pragma unroll
        for (int j = 0; j < NW; ++j)
            Mma<T, kGradRows>::run(tD + j * kCols * S + (32 * mi + l32) * S + h * (kGradRows / 2), bp, acc[j]);
        if (kt == 0 && wave < NW) {      // wave j adds up the columns of dy_j: lane = column
            const T* row = tD + wave * kCols * S + lane * S;
            float s = 0.f;
#pragma unroll 16
            for (int i = 0; i < kGradRows; ++i) s += ld1(row + i);
            colsum += s;
        }
    }
    const int64_t per = (int64_t)a.M * a.K + a.M;
    float* mine = a.partial + (int64_t)blockIdx.x * NW * per;
#pragma unroll
    for (int j = 0; j < NW; ++j) {
        const int k = kt * kCols + 32 * ki + l32;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int m = mt * kCols + 32 * mi + 8 * (r >> 2) + 4 * h + (r & 3);
            if (m < a.M && k < a.K) mine[j * per + (int64_t)m * a.K + k] = acc[j][r];
        }
    }
    if (kt == 0 && wave < NW) {
        const int m = mt * kCols + lane;
        if (m < a.M) mine[wave * per + (int64_t)a.M * a.K + m] = colsum;
    }
}

// ---------------------------------------------------------------------------
// in_features = out_features = 64: the whole backward in one pass over dy.  A workgroup walks panels of 64 node
// rows; for each it forms the panel of dx = sum_j dy_j W_j (weights resident in LDS, transposed) and adds
// dy_j^T x and the column sums of dy_j to the 64 x 64 weight-gradient tiles it keeps in registers; at its end it
// writes one partial like k_linear_gradw (the fixed-order sum of reduce.hip adds them).  dy is read once instead of twice and
// one launch replaces two.
//   bf16 (k_linear64_bwd, four waves): wave w owns the 32 x 32 block (w/2, w%2) of the dx panel and of every dW_j;
//            the products over nodes need the node index contiguous: dy and x are also scattered into transposed
//            tiles, as in k_linear_gradw.
//   float32 (k_linear64_bwd_split, eight waves): see there.
// ---------------------------------------------------------------------------
struct Bwd64Args {
    const void* x;         // [N, 64]
    const void* dy[3];     // [N, 64]
    const void* W[3];      // [64, 64]
    void* dx;              // [N, 64]
    float* partial;        // [workers][nw][64*64 + 64]
    int64_t N;
    const void* u;         // [N, 64], ACT only: x = act(u), and dx leaves as dx * act'(u)
};

template <typename T, int NW> constexpr size_t bwd64_lds_bytes() {
    // W^T, natural dy and transposed dy per weight, transposed x
    return sizeof(T) * (size_t)64 * lds_stride<T>(64) * (3 * NW + 1);
}

// ACT (one weight only; 1 = GELU, 2 = RELU): the layer's input was x = act(u); what leaves in dx is the gradient of u,
// dx * act'(u), with dx rounded as it would have been stored.
template <typename T, int NW, int ACT = 0>
__global__ __launch_bounds__(kThreads) void k_linear64_bwd(Bwd64Args a) {
    static_assert(ACT == 0 || NW == 1, "the activation rides on a backward with one weight");
    static_assert(sizeof(T) == 2, "float32 takes k_linear64_bwd_split");
    constexpr int S = lds_stride<T>(64);
    extern __shared__ __align__(16) unsigned char smem[];
    T* tW = reinterpret_cast<T*>(smem);            // [NW][64 k][S]: W_j transposed, contraction index m contiguous
    T* tD = tW + NW * 64 * S;                      // [NW][64 nodes][S]: dy_j as in memory
    T* tX = tD + NW * 64 * S;                      // [64 k][S]: x transposed
    T* tDt = tX + 64 * S;                          // [NW][64 m][S]: dy_j transposed
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, l32 = lane & 31, h = lane >> 5;
    const int rb = wave >> 1, cb = wave & 1;
    const int64_t n_panels = (a.N + 63) / 64;
    const T* X = reinterpret_cast<const T*>(a.x);
    // a panel on its way from memory, in the transposing piece order (a piece is written to the natural tile as it
    // is and scattered into the transposed one)
    PieceRegs<T> nx_p, nd_p[NW];
    auto fetch = [&](int64_t p) {
        fetch_t(nx_p, X, 64, p * 64, a.N, 0, 64);
#pragma unroll
        for (int j = 0; j < NW; ++j) fetch_t(nd_p[j], reinterpret_cast<const T*>(a.dy[j]), 64, p * 64, a.N, 0, 64);
    };
    int64_t p = blockIdx.x;
    if (p < n_panels) fetch(p);
#pragma unroll
    for (int j = 0; j < NW; ++j) stage_transposed<T, 64, S>(tW + j * 64 * S, reinterpret_cast<const T*>(a.W[j]), 64, 0, 64, 0, 64);
    float16_t accw[NW];
#pragma unroll
    for (int j = 0; j < NW; ++j) accw[j] = zero16();
    float colsum = 0.f;
    for (; p < n_panels; p += gridDim.x) {
        __syncthreads();                 // the previous panel has been read
        {
            // rows past the end of the batch must read as zero here: they enter the sums over nodes
            constexpr int NV = (int)(sizeof(PieceRegs<T>) / 16);
            put_t<T, S>(nx_p, tX, p * 64, a.N, 0, 64);
#pragma unroll
            for (int j = 0; j < NW; ++j) {
                put_t<T, S>(nd_p[j], tDt + j * 64 * S, p * 64, a.N, 0, 64);
#pragma unroll
                for (int i = 0; i < NV; ++i) {
                    int r, c;
                    piece_pos<T, 64>(i, r, c);
                    *reinterpret_cast<uint4*>(tD + j * 64 * S + r * S + c) = zero_unless(p * 64 + r < a.N, nd_p[j].v[i]);
                }
            }
        }
        __syncthreads();
        if (p + gridDim.x < n_panels) fetch(p + gridDim.x);
        // dx panel: rows = nodes, contraction over m
        {
            float16_t acc = zero16();
            float uu[ACT != 0 ? 16 : 1];
            if constexpr (ACT != 0) {      // u where this lane writes; rows past the end repeat the last row and are not stored
                const T* U = reinterpret_cast<const T*>(a.u) + 32 * cb + l32;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int64_t row = p * 64 + 32 * rb + 4 * h + 8 * (r >> 2) + (r & 3);
                    uu[r] = ld1(U + (row < a.N ? row : a.N - 1) * 64);
                }
            }
#pragma unroll
            for (int j = 0; j < NW; ++j)
                Mma<T, 64>::run(tD + j * 64 * S + (32 * rb + l32) * S + h * 32, tW + j * 64 * S + (32 * cb + l32) * S + h * 32, acc);
            T* out = reinterpret_cast<T*>(a.dx) + (p * 64 + 32 * rb + 4 * h) * 64 + 32 * cb + l32;
            if constexpr (ACT != 0) {
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[r] = act_grad<ACT == 2>(uu[r], as_stored(acc[r], out));
            }
            store_rows<T>(out, 64, acc, 0.f, a.N - (p * 64 + 32 * rb + 4 * h));
        }
        // dW_j block (m = 32 rb + ., k = 32 cb + .): contraction over the 64 nodes of the panel
        {
            const T* bp = tX + (32 * cb + l32) * S + h * 32;
#pragma unroll
            for (int j = 0; j < NW; ++j) Mma<T, 64>::run(tDt + j * 64 * S + (32 * rb + l32) * S + h * 32, bp, accw[j]);
        }
        if (wave < NW) {      // wave j adds up the columns of dy_j: lane = column
            float sacc = 0.f;
            const T* row = tDt + wave * 64 * S + lane * S;
#pragma unroll 16
            for (int i = 0; i < 64; ++i) sacc += ld1(row + i);
            colsum += sacc;
        }
    }
    constexpr int64_t per = 64 * 64 + 64;
    float* mine = a.partial + (int64_t)blockIdx.x * NW * per;
#pragma unroll
    for (int j = 0; j < NW; ++j) {
        const int k = 32 * cb + l32;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int m = 32 * rb + 8 * (r >> 2) + 4 * h + (r & 3);
            mine[j * per + (int64_t)m * 64 + k] = accw[j][r];
        }
    }
    if (wave < NW) mine[wave * per + 64 * 64 + lane] = colsum;
}

// float32: the same pass with eight waves and the three-way bf16 split of k_linear64_split.  With the float32 matrix
// instructions this backward is bound by their rate (the two products of the q/k/v backward are 3.1 GFLOP: 20 us at
// the peak), and splitting the operands in the wave that multiplies them only trades matrix time for vector time.
// Here waves 0-3 form the dx panel (and the column sums) and waves 4-7 the weight-gradient blocks, both from the same
// staged tiles, so every SIMD holds one wave of each kind: while one splits its operands on the vector ALU the other
// runs its products.  W_j^T sits in LDS as three bf16 planes (split once per workgroup); dy and x stay float32 in
// their natural [node][feature] layout: the dx waves read their rows of dy (contraction over features, contiguous),
// the dW waves gather eight nodes of one column per product (contraction over nodes) and split them in registers.
// Six v_mfma_f32_32x32x16_bf16 per 16 contraction indices as in the forward: the float32 product to a few 2^-23.
constexpr int kThreads8 = 512;

template <int NW> constexpr size_t bwd64_split_lds_bytes() {
    return (size_t)NW * 3 * kPlaneElems * sizeof(__bf16) + sizeof(float) * (size_t)(NW + 1) * 64 * lds_stride<float>(64);
}

struct Split8 { bf16x8_t hi, mid, lo; };
// eight floats at p[0], p[stride], ...: one column of eight consecutive node rows
__device__ __forceinline__ void gather_split(Split8& f, const float* p, int stride) {
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = p[i * stride];
    uint32_t a[8], b[8], c[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) split3(v[i], a[i], b[i], c[i]);
    f.hi = pack8(a); f.mid = pack8(b); f.lo = pack8(c);
}

template <int NW, int ACT = 0>
__global__ __launch_bounds__(kThreads8, NW == 1 && ACT == 0 ? 4 : 2) void k_linear64_bwd_split(Bwd64Args a) {
    // one weight: two workgroups per CU (128 registers); with the activation's erf and exp that would spill: one
    static_assert(ACT == 0 || NW == 1, "the activation rides on a backward with one weight");
    constexpr int S = lds_stride<float>(64);
    extern __shared__ __align__(16) unsigned char smem[];
    __bf16* tW = reinterpret_cast<__bf16*>(smem);                                            // [NW][3][64 k][kPlaneStride]: W_j^T planes
    float* tD = reinterpret_cast<float*>(smem + (size_t)NW * 3 * kPlaneElems * sizeof(__bf16));   // [NW][64 nodes][S]: dy_j as in memory
    float* tX = tD + NW * 64 * S;                                                            // [64 nodes][S]: x as in memory
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, l32 = lane & 31, h = lane >> 5;
    const int role = wave >> 2, w4 = wave & 3, rb = w4 >> 1, cb = w4 & 1;
    const int64_t n_panels = (a.N + 63) / 64;
    const float* X = reinterpret_cast<const float*>(a.x);
    constexpr int NV = 64 * 64 * 4 / (16 * kThreads8);      // 16-byte pieces of a tile per thread: 2
    uint4 nx[NV], nd[NW][NV];
    auto fetch = [&](int64_t p) {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int v = threadIdx.x + i * kThreads8, r = v >> 4, c = (v & 15) * 4;
            nx[i] = load16_clamped(X, 64, p * 64 + r, a.N, c, 64);
#pragma unroll
            for (int j = 0; j < NW; ++j) nd[j][i] = load16_clamped(reinterpret_cast<const float*>(a.dy[j]), 64, p * 64 + r, a.N, c, 64);
        }
    };
    int64_t p = blockIdx.x;
    if (p < n_panels) fetch(p);
    {   // weights: W_j[m][k] goes to plane row k, contraction index m, split into the three planes
        uint4 raw[NW][NV];
#pragma unroll
        for (int j = 0; j < NW; ++j)
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const int v = threadIdx.x + i * kThreads8;
                raw[j][i] = *reinterpret_cast<const uint4*>(reinterpret_cast<const float*>(a.W[j]) + v * 4);
            }
#pragma unroll
        for (int j = 0; j < NW; ++j)
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const int v = threadIdx.x + i * kThreads8, m = v >> 4, k = (v & 15) * 4;
                const float* e = reinterpret_cast<const float*>(&raw[j][i]);
                __bf16* plane = tW + (size_t)j * 3 * kPlaneElems;
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    uint32_t w0, w1, w2;
                    split3(e[t], w0, w1, w2);
                    const __bf16 x0 = upper_bf16(w0), x1 = upper_bf16(w1), x2 = upper_bf16(w2);
                    const int at = (k + t) * kPlaneStride + m;
                    plane[at] = x0;
                    plane[kPlaneElems + at] = x1;
                    plane[2 * kPlaneElems + at] = x2;
                }
            }
    }
    float16_t accw[NW];
#pragma unroll
    for (int j = 0; j < NW; ++j) accw[j] = zero16();
    float colsum = 0.f;
    for (; p < n_panels; p += gridDim.x) {
        __syncthreads();                 // the previous panel has been read
#pragma unroll
        for (int i = 0; i < NV; ++i) {   // rows past the end of the batch must read as zero: they enter the sums over nodes
            const int v = threadIdx.x + i * kThreads8, r = v >> 4, c = (v & 15) * 4;
            const bool in = p * 64 + r < a.N;
            *reinterpret_cast<uint4*>(tX + r * S + c) = zero_unless(in, nx[i]);
#pragma unroll
            for (int j = 0; j < NW; ++j) *reinterpret_cast<uint4*>(tD + j * 64 * S + r * S + c) = zero_unless(in, nd[j][i]);
        }
        __syncthreads();
        if (p + gridDim.x < n_panels) fetch(p + gridDim.x);
        if (role == 0) {
            // dx panel: rows = nodes, contraction over m
            float16_t acc = zero16();
            float uu[ACT != 0 ? 16 : 1];
            if constexpr (ACT != 0) {      // u where this lane writes; rows past the end repeat the last row and are not stored
                const float* U = reinterpret_cast<const float*>(a.u) + 32 * cb + l32;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int64_t row = p * 64 + 32 * rb + 4 * h + 8 * (r >> 2) + (r & 3);
                    uu[r] = U[(row < a.N ? row : a.N - 1) * 64];
                }
            }
#pragma unroll
            for (int j = 0; j < NW; ++j) {
                Split32 d;
                load_split(d, tD + j * 64 * S + (32 * rb + l32) * S + h * 32);
                mma_split(d, tW + (size_t)j * 3 * kPlaneElems + (32 * cb + l32) * kPlaneStride + h * 32, acc);
            }
            float* out = reinterpret_cast<float*>(a.dx) + (p * 64 + 32 * rb + 4 * h) * 64 + 32 * cb + l32;
            if constexpr (ACT != 0) {
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[r] = act_grad<ACT == 2>(uu[r], acc[r]);
            }
            store_rows<float>(out, 64, acc, 0.f, a.N - (p * 64 + 32 * rb + 4 * h));
            if (w4 < NW) {      // wave j adds up the columns of dy_j: lane = column
                float sacc = 0.f;
                const float* col = tD + w4 * 64 * S + lane;
#pragma unroll 16
                for (int i = 0; i < 64; ++i) sacc += col[i * S];
                colsum += sacc;
            }
        } else {
            // dW_j block (m = 32 rb + ., k = 32 cb + .): contraction over the 64 nodes of the panel, sixteen per step,
            // of which this half of the wave takes eight
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int n0 = 16 * g + 8 * h;
                Split8 xs;
                gather_split(xs, tX + n0 * S + 32 * cb + l32, S);
#pragma unroll
                for (int j = 0; j < NW; ++j) {
                    Split8 ds;
                    gather_split(ds, tD + j * 64 * S + n0 * S + 32 * rb + l32, S);
                    accw[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ds.lo, xs.hi, accw[j], 0, 0, 0);     // small terms first
                    accw[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ds.hi, xs.lo, accw[j], 0, 0, 0);
                    accw[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ds.mid, xs.mid, accw[j], 0, 0, 0);
                    accw[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ds.mid, xs.hi, accw[j], 0, 0, 0);
                    accw[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ds.hi, xs.mid, accw[j], 0, 0, 0);
                    accw[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ds.hi, xs.hi, accw[j], 0, 0, 0);
                }
            }
        }
    }
    constexpr int64_t per = 64 * 64 + 64;
    float* mine = a.partial + (int64_t)blockIdx.x * NW * per;
    if (role == 1) {
#pragma unroll
        for (int j = 0; j < NW; ++j) {
            const int k = 32 * cb + l32;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = 32 * rb + 8 * (r >> 2) + 4 * h + (r & 3);
                mine[j * per + (int64_t)m * 64 + k] = accw[j][r];
            }
        }
    } else if (w4 < NW) {
        mine[w4 * per + 64 * 64 + lane] = colsum;
    }
}

template <int NW, int ACT = 0>
int launch_bwd64_split(const Bwd64Args& a, int workers, hipStream_t st) {
    constexpr size_t lds = bwd64_split_lds_bytes<NW>();
    static bool raised = false;
    if (!raised && lds > 48 * 1024) {
        TGT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&k_linear64_bwd_split<NW, ACT>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        raised = true;
    }
    hipLaunchKernelGGL((k_linear64_bwd_split<NW, ACT>), dim3(workers), dim3(kThreads8), lds, st, a);
    return TGT_OK;
}

template <typename T, int NW, int ACT = 0>
int launch_bwd64(const Bwd64Args& a, int workers, hipStream_t st) {
    constexpr size_t lds = bwd64_lds_bytes<T, NW>();
    static bool raised = false;
    if (!raised && lds > 48 * 1024) {
        TGT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&k_linear64_bwd<T, NW, ACT>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        raised = true;
    }
    hipLaunchKernelGGL((k_linear64_bwd<T, NW, ACT>), dim3(workers), dim3(kThreads), lds, st, a);
    return TGT_OK;
}

// What remains of a weight-gradient pass: the sum of the workers' partials ([workers][nw][M*K + M]) into dW_j and db_j.
tgt_reduce_desc gradw_sum(const float* partial, int workers, int nw, int K, int M, void* const* d_dW, void* const* d_db) {
    tgt_reduce_desc r{};
    const int per = M * K + M;
    r.partial = partial; r.workers = workers; r.n = per * nw; r.n_out = 2 * nw;
    for (int j = 0; j < nw; ++j) {
        r.out[2 * j] = d_dW[j];                      r.begin[2 * j] = j * per;
        r.out[2 * j + 1] = d_db ? d_db[j] : nullptr; r.begin[2 * j + 1] = j * per + M * K;
    }
    return r;
}

int check_shape(int n_out, int64_t N, int in_features, int out_features, int dtype) {
    if (n_out < 1 || n_out > 3 || N < 0 || in_features <= 0 || out_features <= 0) {
        set_error("linear: n_out must be 1..3 and sizes positive (n_out=%d N=%lld in=%d out=%d)", n_out, (long long)N,
                  in_features, out_features);
        return TGT_ERR_INVALID_ARG;
    }
    if (dtype != TGT_DTYPE_F32 && dtype != TGT_DTYPE_BF16) {
        set_error("linear: unknown dtype %d", dtype);
        return TGT_ERR_INVALID_ARG;
    }
    const int ve = dtype == TGT_DTYPE_F32 ? 4 : 8;      // rows are read in 16-byte pieces
    if (in_features % ve || out_features % ve) {
        set_error("linear: in_features and out_features must be multiples of %d for this dtype (got %d, %d)", ve,
                  in_features, out_features);
        return TGT_ERR_UNSUPPORTED;
    }
    if (N > (int64_t)INT32_MAX * kGradRows) {
        set_error("linear: N too large");
        return TGT_ERR_UNSUPPORTED;
    }
    return TGT_OK;
}

int grad_workers(int in_features, int out_features) {
    const int tiles = ((in_features + kCols - 1) / kCols) * ((out_features + kCols - 1) / kCols);
    return std::max(1, kGradWorkers / tiles);
}

template <typename T, int NW>
int launch_gradw(const GradWArgs& g, int workers, int tiles, hipStream_t st) {
    const size_t lds = sizeof(T) * (size_t)(1 + NW) * kCols * lds_stride<T>(kGradRows);
    static bool raised = false;   // per instantiation; the attribute is per function and sticks
    if (!raised && lds > 48 * 1024) {
        TGT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&k_linear_gradw<T, NW>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        raised = true;
    }
    hipLaunchKernelGGL((k_linear_gradw<T, NW>), dim3(workers, tiles), dim3(kThreads), lds, st, g);
    return TGT_OK;
}

template <typename T>
int linear_bwd_t(const void* d_x, const void* const* d_W, const void* const* d_dy, int n_out, int64_t N, int K, int M,
                 void* d_dx, void* const* d_dW, void* const* d_db, float* partial, hipStream_t st, tgt_reduce_desc* defer,
                 int act = 0, const void* d_u = nullptr) {
    if (act != 0 && !(d_dx && d_dW && N > 0 && K == 64 && M == 64 && n_out == 1)) {
        // no kernel of this shape applies the activation itself: the plain backward, then dx * act'(u) in place
        const int rc = linear_bwd_t<T>(d_x, d_W, d_dy, n_out, N, K, M, d_dx, d_dW, d_db, partial, st, defer);
        if (rc != TGT_OK || !d_dx || N == 0) return rc;
        const int code = sizeof(T) == 4 ? TGT_DTYPE_F32 : TGT_DTYPE_BF16;
        return act == TGT_ACT_RELU ? tgt_relu_bwd(d_u, d_dx, N * K, code, d_dx, st) : tgt_gelu_bwd(d_u, d_dx, N * K, code, d_dx, st);
    }
    if (d_dx && d_dW && N > 0 && K == 64 && M == 64) {
        // one pass for dx and the weight gradients
        constexpr bool split = sizeof(T) == 4;       // float32: eight waves and the bf16 split; bf16: four waves
        constexpr size_t lds1 = split ? bwd64_split_lds_bytes<1>() : bwd64_lds_bytes<T, 1>();
        constexpr size_t lds2 = split ? bwd64_split_lds_bytes<2>() : bwd64_lds_bytes<T, 2>();
        const size_t lds = lds1 + (n_out - 1) * (lds2 - lds1);
        const int64_t n_panels = (N + 63) / 64;
        const int per_cu = split && act != 0 ? 1 : (int)std::max<size_t>(1, std::min<size_t>(2, (size_t)(160 * 1024) / lds));
        const int workers = (int)std::max<int64_t>(1, std::min<int64_t>(std::min<int64_t>(n_panels, grad_workers(K, M)),
                                                                        (int64_t)num_cus() * per_cu));
        Bwd64Args b{};
        b.x = d_x; b.dx = d_dx; b.partial = partial; b.N = N; b.u = d_u;
        for (int j = 0; j < n_out; ++j) { b.dy[j] = d_dy[j]; b.W[j] = d_W[j]; }
        int rc = TGT_OK;
        {
            KernelTimer t(KS_LINEAR_DX, st);
            if constexpr (split) {
                if (act == TGT_ACT_GELU) rc = launch_bwd64_split<1, 1>(b, workers, st);
                else if (act == TGT_ACT_RELU) rc = launch_bwd64_split<1, 2>(b, workers, st);
                else if (n_out == 1) rc = launch_bwd64_split<1>(b, workers, st);
                else if (n_out == 2) rc = launch_bwd64_split<2>(b, workers, st);
                else rc = launch_bwd64_split<3>(b, workers, st);
            } else {
                if (act == TGT_ACT_GELU) rc = launch_bwd64<T, 1, 1>(b, workers, st);
                else if (act == TGT_ACT_RELU) rc = launch_bwd64<T, 1, 2>(b, workers, st);
                else if (n_out == 1) rc = launch_bwd64<T, 1>(b, workers, st);
                else if (n_out == 2) rc = launch_bwd64<T, 2>(b, workers, st);
                else rc = launch_bwd64<T, 3>(b, workers, st);
            }
        }
        if (rc != TGT_OK) return rc;
        TGT_HIP_CHECK(hipGetLastError());
        const tgt_reduce_desc r = gradw_sum(partial, workers, n_out, K, M, d_dW, d_db);
        if (defer) { *defer = r; return TGT_OK; }
        return reduce_partials(&r, 1, sizeof(T) == 4 ? TGT_DTYPE_F32 : TGT_DTYPE_BF16, st);
    }
    if (d_dx && N > 0) {
        LinArgs a{};
        for (int j = 0; j < n_out; ++j) { a.A[j] = d_dy[j]; a.W[j] = d_W[j]; }
        a.out[0] = d_dx;
        a.nw = n_out; a.N = N; a.K = K; a.M = M;
        KernelTimer t(KS_LINEAR_DX, st);
        const int rc = launch_linear<T, true>(a, st);
        if (rc != TGT_OK) return rc;
    }
    if (d_dW) {
        const int tiles = ((K + kCols - 1) / kCols) * ((M + kCols - 1) / kCols);
        const int64_t n_panels = (N + kGradRows - 1) / kGradRows;
        const int workers = (int)std::max<int64_t>(1, std::min<int64_t>(n_panels, grad_workers(K, M)));
        GradWArgs g{};
        g.x = d_x;
        for (int j = 0; j < n_out; ++j) g.dy[j] = d_dy[j];
        g.partial = partial; g.N = N; g.K = K; g.M = M;
        int rc = TGT_OK;
        {
            KernelTimer t(KS_LINEAR_DW, st);
            if (n_out == 1) rc = launch_gradw<T, 1>(g, workers, tiles, st);
            else if (n_out == 2) rc = launch_gradw<T, 2>(g, workers, tiles, st);
            else rc = launch_gradw<T, 3>(g, workers, tiles, st);
        }
        if (rc != TGT_OK) return rc;
        TGT_HIP_CHECK(hipGetLastError());
        const tgt_reduce_desc r = gradw_sum(partial, workers, n_out, K, M, d_dW, d_db);
        if (defer) { *defer = r; return TGT_OK; }
        return reduce_partials(&r, 1, sizeof(T) == 4 ? TGT_DTYPE_F32 : TGT_DTYPE_BF16, st);
    }
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

}  // namespace
}  // namespace tgt

extern "C" {

int tgt_linear_fwd(const void* d_x, const void* const* d_W, const void* const* d_b, void* const* d_y, int n_out,
                   int64_t N, int in_features, int out_features, int dtype, void* stream) {
    using namespace tgt;
    const int rc = check_shape(n_out, N, in_features, out_features, dtype);
    if (rc != TGT_OK) return rc;
    if (!d_W || !d_y || (N > 0 && !d_x)) { set_error("linear_fwd: null pointer"); return TGT_ERR_INVALID_ARG; }
    LinArgs a{};
    a.A[0] = d_x;
    for (int j = 0; j < n_out; ++j) {
        if (!d_W[j] || (N > 0 && !d_y[j])) { set_error("linear_fwd: null weight or output %d", j); return TGT_ERR_INVALID_ARG; }
        a.W[j] = d_W[j];
        a.bias[j] = d_b ? d_b[j] : nullptr;
        a.out[j] = d_y[j];
    }
    a.nw = n_out; a.N = N; a.K = in_features; a.M = out_features;
    if (N == 0) return TGT_OK;
    hipStream_t st = (hipStream_t)stream;
    KernelTimer t(KS_LINEAR_FWD, st);
    const int lrc = dtype == TGT_DTYPE_F32 ? launch_linear<float, false>(a, st) : launch_linear<pbf16, false>(a, st);
    if (lrc != TGT_OK) return lrc;
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

int64_t tgt_linear_bwd_workspace_bytes(int n_out, int in_features, int out_features) {
    using namespace tgt;
    if (n_out < 1 || n_out > 3 || in_features <= 0 || out_features <= 0) return 0;
    return (int64_t)sizeof(float) * grad_workers(in_features, out_features) * n_out *
           ((int64_t)in_features * out_features + out_features);
}

static int linear_bwd_entry(const void* d_x, const void* const* d_W, const void* const* d_dy, int n_out, int64_t N,
                            int in_features, int out_features, int dtype, void* d_dx, void* const* d_dW, void* const* d_db,
                            void* d_workspace, int64_t workspace_bytes, void* stream, tgt_reduce_desc* defer, int act = 0,
                            const void* d_u = nullptr) {
    using namespace tgt;
    const int rc = check_shape(n_out, N, in_features, out_features, dtype);
    if (rc != TGT_OK) return rc;
    if (!d_W || !d_dy || (N > 0 && !d_x)) { set_error("linear_bwd: null pointer"); return TGT_ERR_INVALID_ARG; }
    for (int j = 0; j < n_out; ++j) {
        if (!d_W[j] || (N > 0 && !d_dy[j]) || (d_dW && !d_dW[j])) {
            set_error("linear_bwd: null weight, gradient or output %d", j);
            return TGT_ERR_INVALID_ARG;
        }
    }
    if (d_db && !d_dW) { set_error("linear_bwd: bias gradients are produced with the weight gradients"); return TGT_ERR_INVALID_ARG; }
    if (d_dW && (!d_workspace || workspace_bytes < tgt_linear_bwd_workspace_bytes(n_out, in_features, out_features) ||
                 ((uintptr_t)d_workspace & 15))) {
        set_error("linear_bwd: workspace of %lld bytes (16-byte aligned) needed, got %lld",
                  (long long)tgt_linear_bwd_workspace_bytes(n_out, in_features, out_features), (long long)workspace_bytes);
        return TGT_ERR_WORKSPACE;
    }
    hipStream_t st = (hipStream_t)stream;
    if (dtype == TGT_DTYPE_F32)
        return linear_bwd_t<float>(d_x, d_W, d_dy, n_out, N, in_features, out_features, d_dx, d_dW, d_db,
                                   (float*)d_workspace, st, defer, act, d_u);
    return linear_bwd_t<pbf16>(d_x, d_W, d_dy, n_out, N, in_features, out_features, d_dx, d_dW, d_db,
                               (float*)d_workspace, st, defer, act, d_u);
}

int tgt_linear_act_fwd(const void* d_x, const void* d_W, const void* d_b, int64_t N, int in_features, int out_features, int dtype,
                       int act, void* d_u, void* d_h, void* stream) {
    using namespace tgt;
    const int rc = check_shape(1, N, in_features, out_features, dtype);
    if (rc != TGT_OK) return rc;
    if (act != TGT_ACT_GELU && act != TGT_ACT_RELU) { set_error("linear_act_fwd: unknown activation %d", act); return TGT_ERR_INVALID_ARG; }
    if (!d_W || (N > 0 && (!d_x || !d_u || !d_h))) { set_error("linear_act_fwd: null pointer"); return TGT_ERR_INVALID_ARG; }
    if (N == 0) return TGT_OK;
    hipStream_t st = (hipStream_t)stream;
    if (in_features != 64 || out_features != 64) {
        // no kernel of this shape applies the activation itself: the plain forward, then the activation kernel
        const void* W[1] = {d_W};
        const void* b[1] = {d_b};
        void* y[1] = {d_u};
        const int lrc = tgt_linear_fwd(d_x, W, b, y, 1, N, in_features, out_features, dtype, stream);
        if (lrc != TGT_OK) return lrc;
        return act == TGT_ACT_RELU ? tgt_relu_fwd(d_u, N * out_features, dtype, d_h, stream) : tgt_gelu_fwd(d_u, N * out_features, dtype, d_h, stream);
    }
    LinArgs a{};
    a.A[0] = d_x; a.W[0] = d_W; a.bias[0] = d_b; a.out[0] = d_u; a.out[1] = d_h;
    a.nw = 1; a.N = N; a.K = 64; a.M = 64;
    KernelTimer t(KS_LINEAR_FWD, st);
    int lrc;
    if (dtype == TGT_DTYPE_F32) lrc = act == TGT_ACT_GELU ? launch_linear64<float, false, 1, 1>(a, st) : launch_linear64<float, false, 1, 2>(a, st);
    else lrc = act == TGT_ACT_GELU ? launch_linear64<pbf16, false, 1, 1>(a, st) : launch_linear64<pbf16, false, 1, 2>(a, st);
    if (lrc != TGT_OK) return lrc;
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

int tgt_linear_act_bwd(const void* d_h, const void* d_W, const void* d_dy, const void* d_u, int64_t N, int in_features,
                       int out_features, int dtype, int act, void* d_du, void* d_dW, void* d_db, void* d_workspace,
                       int64_t workspace_bytes, void* stream, tgt_reduce_desc* desc) {
    if (act != TGT_ACT_GELU && act != TGT_ACT_RELU) { tgt::set_error("linear_act_bwd: unknown activation %d", act); return TGT_ERR_INVALID_ARG; }
    if (!d_du || !d_dW || (N > 0 && !d_u)) { tgt::set_error("linear_act_bwd: null pointer"); return TGT_ERR_INVALID_ARG; }
    const void* W[1] = {d_W};
    const void* dy[1] = {d_dy};
    void* dW[1] = {d_dW};
    void* db[1] = {d_db};
    if (desc) *desc = tgt_reduce_desc{};
    return linear_bwd_entry(d_h, W, dy, 1, N, in_features, out_features, dtype, d_du, dW, d_db ? db : nullptr, d_workspace,
                            workspace_bytes, stream, desc, act, d_u);
}

int tgt_linear_bwd(const void* d_x, const void* const* d_W, const void* const* d_dy, int n_out, int64_t N,
                   int in_features, int out_features, int dtype, void* d_dx, void* const* d_dW, void* const* d_db,
                   void* d_workspace, int64_t workspace_bytes, void* stream) {
    return linear_bwd_entry(d_x, d_W, d_dy, n_out, N, in_features, out_features, dtype, d_dx, d_dW, d_db, d_workspace,
                            workspace_bytes, stream, nullptr);
}

int tgt_linear_bwd_deferred(const void* d_x, const void* const* d_W, const void* const* d_dy, int n_out, int64_t N,
                            int in_features, int out_features, int dtype, void* d_dx, void* const* d_dW, void* const* d_db,
                            void* d_workspace, int64_t workspace_bytes, void* stream, tgt_reduce_desc* desc) {
    if (!desc || !d_dW) { tgt::set_error("linear_bwd_deferred: a descriptor and weight-gradient outputs are needed"); return TGT_ERR_INVALID_ARG; }
    *desc = tgt_reduce_desc{};
    return linear_bwd_entry(d_x, d_W, d_dy, n_out, N, in_features, out_features, dtype, d_dx, d_dW, d_db, d_workspace,
                            workspace_bytes, stream, desc);
}

}  // extern "C"
