// Dense biased attention for batches of small graphs (graph-level models), bf16
// MFMA with fp32 softmax.
//
// Replaces CoreAttention.forward of models/graphormer_graph_level.py:186-214
// (same body: attn_module.py:99-127, graphormer_dist_graph_level.py:211-235):
//   x = (q * sqrt(d)) k^T + attn_bias ; softmax over keys ; x v
// q, k, v: [b, S, H, d]; attn_bias: [b, H, S, S]; out: [b, S, H*d].
//
// One workgroup per (graph, head); wave w owns query tile w (32 queries) in the
// forward and, in the backward, also key tile w.  The matrix instruction is
// v_mfma_f32_32x32x8_bf16_1k (contraction depth 8 = head dim 8, no padding of K):
//   A 32x8  : lane l holds A[l%32][4*(l/32) .. +3]
//   B 8x32  : lane l holds B[4*(l/32) .. +3][l%32]
//   C 32x32 : lane l, register r holds C[8*(r/4) + 4*(l/32) + r%4][l%32]
// Scores are formed TRANSPOSED (A = K tile, B = Q^T), so a lane owns one query
// and its registers run over keys: the softmax reductions are register-local plus
// one cross-half shuffle, and the probabilities sit exactly in the B-operand
// layout of the next product (O^T = V^T P^T), no shuffle or LDS round trip.
// The bias is read straight from global memory in the layout each walk needs (see
// key_of_row and the backward kernel); only q/k/v/dout heads are staged in LDS.
#include "common.h"
#include "dense_dropout.h"
#include <algorithm>
#include <stdlib.h>

namespace tgt {

typedef short short4_t __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

struct dbf16 { uint16_t x; };

__device__ __forceinline__ short f2bf(float f) {
    const __bf16 b = static_cast<__bf16>(f);
    return __builtin_bit_cast(short, b);
}
__device__ __forceinline__ float bf2f(short s) { return __uint_as_float(((uint32_t)(uint16_t)s) << 16); }
// two / four floats -> bf16 (round to nearest even), two values per conversion instruction
__device__ __forceinline__ uint32_t cvt_pk(float lo, float hi) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    f32x2 x;
    x.x = lo; x.y = hi;
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(x, bf16x2));
}
typedef short short4_pk __attribute__((ext_vector_type(4)));
__device__ __forceinline__ short4_pk pack4(float a, float b, float c, float d) {
    typedef uint32_t u2 __attribute__((ext_vector_type(2)));
    u2 r;
    r.x = cvt_pk(a, b);
    r.y = cvt_pk(c, d);
    return __builtin_bit_cast(short4_pk, r);
}

// four consecutive elements as bf16 bits
__device__ __forceinline__ short4_t ld4(const dbf16* p) {
    return *reinterpret_cast<const short4_t*>(p);
}
__device__ __forceinline__ short4_t ld4(const float* p) {
    const float4_t f = *reinterpret_cast<const float4_t*>(p);
    return pack4(f.x, f.y, f.z, f.w);
}
__device__ __forceinline__ void st4(dbf16* p, float a, float b, float c, float d) {
    *reinterpret_cast<short4_t*>(p) = pack4(a, b, c, d);
}
__device__ __forceinline__ void st4(float* p, float a, float b, float c, float d) {
    float4_t r;
    r.x = a; r.y = b; r.z = c; r.w = d;
    *reinterpret_cast<float4_t*>(p) = r;
}
__device__ __forceinline__ float ld1(const float* p) { return *p; }
__device__ __forceinline__ float ld1(const dbf16* p) { return __uint_as_float(((uint32_t)p->x) << 16); }
__device__ __forceinline__ void st1(float* p, float v) { *p = v; }
__device__ __forceinline__ void st1(dbf16* p, float v) { p->x = (uint16_t)f2bf(v); }

__device__ __forceinline__ float16_t mfma(short4_t a, short4_t b, float16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ float16_t zero16() {
    float16_t z;
#pragma unroll
    for (int i = 0; i < 16; ++i) z[i] = 0.f;
    return z;
}
__device__ __forceinline__ short4_t zero4() { short4_t z; z.x = 0; z.y = 0; z.z = 0; z.w = 0; return z; }

// LDS images of X[g, :, h, :]: row-major [SP][D] and transposed [D][SP+4] (bf16 bits).
template <int D, int SP> constexpr int rm_elems() { return SP * D; }
template <int D, int SP> constexpr int tr_elems() { return D * (SP + 4); }

// Cooperative load of X[g, :, h, :] into either layout (rows >= S are zero).
template <typename T, int D, int SP>
__device__ __forceinline__ void load_head(const T* __restrict__ X, int g, int h, int S, int H,
                                          short* __restrict__ rm, short* __restrict__ tr) {
    for (int c = threadIdx.x; c < SP * (D / 4); c += blockDim.x) {
        const int row = c / (D / 4), part = c % (D / 4);
        short4_t x = zero4();
        if (row < S) x = ld4(X + (((int64_t)g * S + row) * H + h) * D + part * 4);
        if (rm) *reinterpret_cast<short4_t*>(&rm[row * D + part * 4]) = x;
        if (tr) {
            tr[(part * 4 + 0) * (SP + 4) + row] = x.x;
            tr[(part * 4 + 1) * (SP + 4) + row] = x.y;
            tr[(part * 4 + 2) * (SP + 4) + row] = x.z;
            tr[(part * 4 + 3) * (SP + 4) + row] = x.w;
        }
    }
}

// Sixteen consecutive elements of one bias row, as they come from memory.  A bias row of
// [b, H, S, S] starts at an arbitrary 2- or 4-byte boundary (S is odd for a batch with a virtual
// node); gfx950 global loads take any alignment, so a full group is fetched with 16-byte loads
// and the values are converted when they are used, not when they arrive.
template <typename T> struct Bias16;
template <> struct Bias16<dbf16> {
    uint32_t w[8];
    __device__ __forceinline__ float get(int r) const {
        return (r & 1) ? __uint_as_float(w[r >> 1] & 0xffff0000u) : __uint_as_float(w[r >> 1] << 16);
    }
};
template <> struct Bias16<float> {
    float w[16];
    __device__ __forceinline__ float get(int r) const { return w[r]; }
};
// elements p[0 .. n_valid) (n_valid <= 16); the others read as 0
__device__ __forceinline__ void load_bias16(const dbf16* __restrict__ p, int n_valid, Bias16<dbf16>& b) {
    if (n_valid >= 16) {
        // A row of an odd-length bias starts on a 2-byte boundary half of the time, and a vector load
        // from such an address is split into many cache accesses.  So the nine aligned dwords that
        // hold the group are loaded and funnel-shifted into place.  (With the shift the ninth dword
        // holds element 15; its upper half may lie 2 bytes past a tensor that ends there, inside the
        // allocation's granule.)
        const uintptr_t a = reinterpret_cast<uintptr_t>(p);
        const uint32_t* __restrict__ q = reinterpret_cast<const uint32_t*>(a & ~(uintptr_t)3);
        const uint32_t sh = (uint32_t)(a & 2) * 8;      // 0 or 16 bits
        uint32_t w9[9];
        __builtin_memcpy(w9, q, 32);
        w9[8] = sh ? q[8] : 0u;
#pragma unroll
        for (int i = 0; i < 8; ++i) b.w[i] = __builtin_amdgcn_alignbit(w9[i + 1], w9[i], sh);
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) b.w[i] = 0;
#pragma unroll
        for (int r = 0; r < 16; ++r)
            if (r < n_valid) b.w[r >> 1] |= ((uint32_t)p[r].x) << (16 * (r & 1));
    }
}
__device__ __forceinline__ void load_bias16(const float* __restrict__ p, int n_valid, Bias16<float>& b) {
    if (n_valid >= 16) {
        __builtin_memcpy(b.w, p, 64);
    } else {
#pragma unroll
        for (int r = 0; r < 16; ++r) b.w[r] = r < n_valid ? p[r] : 0.f;
    }
}
template <typename T>
__device__ __forceinline__ void zero_bias16(Bias16<T>& b) {
#pragma unroll
    for (int i = 0; i < (int)(sizeof(b.w) / sizeof(b.w[0])); ++i) b.w[i] = 0;
}
// raw single elements (the key-major walk of the backward reads one element per query)
__device__ __forceinline__ uint32_t raw1(const dbf16* p) { return p->x; }
__device__ __forceinline__ float raw1(const float* p) { return *p; }
__device__ __forceinline__ float cvt1(uint32_t x) { return __uint_as_float(x << 16); }
__device__ __forceinline__ float cvt1(float x) { return x; }

// ---------------------------------------------------------------------------
// The bias of the graph-level Graphormer formed inside the attention kernels (BSRC = 1) instead of
// read from a [b, H, S, S] tensor (GraphAttnBias.forward, models/graphormer_graph_level.py:94-156,
// simple edge-type branch, feeding CoreAttention.forward :186-214):
//   bias[g,h,i,j] = 2 attn_bias[g,i,j] + spatial_table[sp[g,i,j]][h] + mean_f edge_table[et[g,i,j,f]][h]
// with the ids packed beforehand to 16 bits over the padded [S, S] index space: on the virtual
// node's row and column sp holds the extra id num_spatial (its table slot is the virtual
// distance of head h) and et the extra id num_edges (slot 0.0).  A workgroup keeps the tables of
// its head in LDS as float, builds the [S, S] bias of its (graph, head) pair in LDS as bf16 once,
// and both walks read it from there.  In the backward the bias gradient dS never leaves the
// chip either: the query-major walk adds every dS into LDS accumulators indexed by the ids (ids
// below kHotIds into one of kHotCopies copies chosen by the lane, which keeps lanes that meet the
// same few shortest-path lengths off each other's address).  The accumulators are 32-bit
// integers: LDS integer atomics run about nine times faster than the floating-point ones on this
// part (measured: 16 against 54 ns per wave-wide add under this id distribution), and integer
// sums do not depend on the order of the adds, so the table gradients are reproducible bit for
// bit.  Every (graph, head) pair gets its own power-of-two scale from a bound on its dS: the rows
// of the softmax sum to one, so sum_k |dS[q,k]| <= 2 max_q |dout_q|_1 max|v| / (1 - p) =: B and no
// accumulator of one pair can exceed S B; with scale = 2^22 / B' (B' = B rounded up to a power of
// two) that stays below 2^30 for S <= 256, and one unit is 2^-22 B'.  A position adds its dS to the edge table once
// per edge feature, so an edge accumulator is bounded by F S B: its scale is 2^ceil(log2 F) times smaller.  After each pair the
// workgroup converts its integer sums to float and adds them to its partial in global memory.
// ---------------------------------------------------------------------------
struct IdsArgs {
    const void* ab;            // [b, S, S] of T, or null
    const uint16_t* sp;        // [b, S, S]
    const uint16_t* et;        // [b, S, S, F]
    const void* sp_tab;        // [ns, H] of T
    const void* e_tab;         // [ne, H] of T
    const void* vd;            // [H] of T
    float* partial;            // backward: [gridDim.x][ns + ne + 1], or null when no table gradient is wanted
    int F, ns, ne;
};
constexpr int kHotIds = 32, kHotCopies = 16, kHotStride = kHotIds + 1;

struct IdsLds {
    short* tile;               // [S][bst] bf16 bits
    float *tabS, *tabE;        // [ns + 1], [ne + 1]: the head's table columns (edge entries already divided by F)
    int *hot, *accS, *accE;    // backward only: fixed-point sums of the current pair ([kHotCopies][kHotStride], [ns + 1], [ne + 1])
    int* bound;                // backward only: max_q |dout_q|_1 and max |v| of the current pair, as float bits
    int bst;
};
__host__ __device__ __forceinline__ int ids_tile_stride(int S) { return (S + 7) & ~7; }
__host__ __device__ __forceinline__ size_t ids_tile_bytes(int S) { return (((size_t)S * ids_tile_stride(S) * 2) + 15) & ~(size_t)15; }
inline size_t ids_lds_bytes(int S, int ns, int ne, bool bwd) {
    // (+ 32: a lane's sixteen-key group of the last row may end up to 30 bytes behind the tile)
    return ids_tile_bytes(S) + 32 + sizeof(float) * ((size_t)(ns + ne + 2) * (bwd ? 2 : 1) + (bwd ? kHotCopies * kHotStride + 4 : 0));
}
__device__ __forceinline__ IdsLds ids_lds(char* base, int S, int ns, int ne) {
    IdsLds l;
    l.bst = ids_tile_stride(S);
    l.tile = reinterpret_cast<short*>(base);
    l.tabS = reinterpret_cast<float*>(base + ids_tile_bytes(S));
    l.tabE = l.tabS + ns + 1;
    l.hot = reinterpret_cast<int*>(l.tabE + ne + 1);
    l.accS = l.hot + kHotCopies * kHotStride;
    l.accE = l.accS + ns + 1;
    l.bound = l.accE + ne + 1;
    return l;
}
__device__ __forceinline__ float ldT(const float* p) { return *p; }
__device__ __forceinline__ float ldT(const dbf16* p) { return __uint_as_float(((uint32_t)p->x) << 16); }

template <typename T>
__device__ __forceinline__ void ids_load_tables(const IdsArgs& a, int h, int H, const IdsLds& l) {
    const T* st = reinterpret_cast<const T*>(a.sp_tab);
    const T* et = reinterpret_cast<const T*>(a.e_tab);
    for (int i = threadIdx.x; i < a.ns; i += blockDim.x) l.tabS[i] = ldT(st + (int64_t)i * H + h);
    const float inv_f = 1.f / (float)a.F;
    for (int i = threadIdx.x; i < a.ne; i += blockDim.x) l.tabE[i] = ldT(et + (int64_t)i * H + h) * inv_f;
    if (threadIdx.x == 0) {
        l.tabS[a.ns] = ldT(reinterpret_cast<const T*>(a.vd) + h);
        l.tabE[a.ne] = 0.f;
    }
}

// tile[i][j] = bias of (query i, key j) of graph g for the head whose tables are in LDS; columns S .. bst-1 are zero.
// A thread takes sixteen consecutive keys of a row at a time: three 32-byte requests (attn_bias, spatial ids, first
// edge feature) in flight together, sixteen pairs of table look-ups, one 32-byte LDS write; GB such groups per thread
// are requested before the first is used (a thread has only a handful of groups per pair: one after the other they
// would cost a memory round trip each).  The columns behind the last whole group of a row are done one per thread.
__device__ __forceinline__ float ids_bias_value(const IdsArgs& a, const IdsLds& l, float ab2, uint32_t sp, int64_t at) {
    float v = ab2 + l.tabS[min((int)sp, a.ns)];
    for (int f = 0; f < a.F; ++f) v += l.tabE[min((int)a.et[at * a.F + f], a.ne)];
    return v;
}
// x / d for 0 <= x < 65536 and 1 <= d <= 65536 through a multiplication: with m = ceil(2^32 / d), (x m) >> 32 is exact
// in that range (d = 1 has no 32-bit m: it is coded as 0)
__device__ __forceinline__ uint32_t div_magic(int d) { return d == 1 ? 0u : (uint32_t)((0x100000000ull + (uint32_t)d - 1) / (uint32_t)d); }
__device__ __forceinline__ int div_by(int x, uint32_t m) { return m == 0u ? x : (int)__umulhi((uint32_t)x, m); }

template <typename T, int GB>
__device__ __forceinline__ void ids_build_tile(const IdsArgs& a, int g, int S, const IdsLds& l) {
    const T* ab = reinterpret_cast<const T*>(a.ab);
    const int64_t base = (int64_t)g * S * S;
    const int bst = l.bst;
    const int gpr = S >> 4;                          // whole groups per row
    const int n_groups = S * gpr;
    const uint32_t m_gpr = div_magic(max(gpr, 1));
    for (int grp0 = threadIdx.x; grp0 < n_groups; grp0 += GB * blockDim.x) {
        Bias16<T> abr[GB];
        Bias16<dbf16> spr[GB], etr[GB];
#pragma unroll
        for (int u = 0; u < GB; ++u) {
            const int grp = min(grp0 + u * (int)blockDim.x, n_groups - 1);      // past the end: the last group again, not stored
            const int i = div_by(grp, m_gpr), j0 = (grp - i * gpr) * 16;
            const int64_t at = base + (int64_t)i * S + j0;
            zero_bias16(abr[u]);
            zero_bias16(etr[u]);
            if (ab) load_bias16(ab + at, 16, abr[u]);
            load_bias16(reinterpret_cast<const dbf16*>(a.sp) + at, 16, spr[u]);
            if (a.F == 1) load_bias16(reinterpret_cast<const dbf16*>(a.et) + at, 16, etr[u]);
        }
#pragma unroll
        for (int u = 0; u < GB; ++u) {
            const int grp = grp0 + u * (int)blockDim.x;
            const int gc = min(grp, n_groups - 1);
            const int i = div_by(gc, m_gpr), j0 = (gc - i * gpr) * 16;
            const int64_t at = base + (int64_t)i * S + j0;
            short v16[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float ab2 = 2.f * abr[u].get(r);                   // the clone plus the final re-add (:104, :153)
                const uint32_t sp = (spr[u].w[r >> 1] >> (16 * (r & 1))) & 0xffffu;
                float v;
                if (a.F == 1) v = ab2 + l.tabS[min((int)sp, a.ns)] + l.tabE[min((int)((etr[u].w[r >> 1] >> (16 * (r & 1))) & 0xffffu), a.ne)];
                else v = ids_bias_value(a, l, ab2, sp, at + r);
                v16[r] = f2bf(v);
            }
            if (grp < n_groups) __builtin_memcpy(l.tile + i * bst + j0, v16, 32);
        }
    }
    const int j_rest = gpr * 16, w_rest = bst - j_rest;        // columns j_rest .. bst-1 of every row, one per thread
    const uint32_t m_rest = div_magic(max(w_rest, 1));
    for (int e = threadIdx.x; e < S * w_rest; e += blockDim.x) {
        const int i = div_by(e, m_rest), j = j_rest + (e - i * w_rest);
        float v = 0.f;
        if (j < S) {
            const int64_t at = base + (int64_t)i * S + j;
            v = ids_bias_value(a, l, ab ? 2.f * ldT(ab + at) : 0.f, a.sp[at], at);
        }
        l.tile[i * bst + j] = f2bf(v);
    }
}

// sixteen consecutive bf16 of a tile row, from a 32-byte aligned position
__device__ __forceinline__ void load_tile16(const short* __restrict__ p, Bias16<dbf16>& b) {
    const uint4 u0 = *reinterpret_cast<const uint4*>(p), u1 = *reinterpret_cast<const uint4*>(p + 8);
    b.w[0] = u0.x; b.w[1] = u0.y; b.w[2] = u0.z; b.w[3] = u0.w;
    b.w[4] = u1.x; b.w[5] = u1.y; b.w[6] = u1.z; b.w[7] = u1.w;
}

// Where the backward adds one dS.  id 0 of either table is the padding index and gets no gradient
// (nn.Embedding(padding_idx=0), :82, :86); masked positions carry exact zeros.
struct IdsAcc {
    const uint16_t *sp, *et;   // of this graph: [S, S], [S, S, F]
    int *hot_copy, *accS, *accE;
    int F, ns, ne, hot_n;
    float scale;               // of the current pair: dS * scale is what the accumulators count
    float scale_e;             // the same for the edge table: scale / 2^ceil(log2 F), a position adds its dS once per feature
    bool on;
};
// (id 0 is added too, into a slot that is never read: one test less per position)
__device__ __forceinline__ void acc_spatial(const IdsAcc& c, float ds, uint32_t id) {
    if (ds != 0.f) {
        id = min(id, (uint32_t)c.ns);
        atomicAdd((int)id < c.hot_n ? c.hot_copy + id : c.accS + id, __float2int_rn(ds * c.scale));
    }
}
__device__ __forceinline__ void acc_edge(const IdsAcc& c, float ds, uint32_t e) {
    if (ds != 0.f && e != 0 && (int)e < c.ne) atomicAdd(c.accE + e, __float2int_rn(ds * c.scale_e));
}
// one position whose ids are still in memory
__device__ __forceinline__ void acc_position(const IdsAcc& c, float ds, int64_t at) {
    if (ds != 0.f) {
        acc_spatial(c, ds, c.sp[at]);
        for (int f = 0; f < c.F; ++f) acc_edge(c, ds, c.et[at * c.F + f]);
    }
}

// The keys of a 32-key tile are assigned to the rows of the MFMA A operand in a permuted order,
// row 8j + 4h + t  <->  key 16h + 4j + t, so that in the transposed score tile (lane = query,
// half h = lane / 32) register r of a lane is key 16h + r: sixteen CONSECUTIVE keys per lane,
// which is 32 contiguous bytes of that query's bias row.
__device__ __forceinline__ int key_of_row(int row) { return 16 * ((row >> 2) & 1) + 4 * (row >> 3) + (row & 3); }

// 2^x as the bare hardware instruction (inputs here are <= 0 or row maxima differences; results
// below the normal range flush to zero, which is what a softmax weight of that size is worth)
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ float max3(float a, float b, float c) {
    float d;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));
    return d;
}

constexpr float kLog2e = 1.4426950408889634f;

// dynamic LDS sizes (bytes)
template <int D, int NT> constexpr int fwd_lds_bytes() {
    return 2 * (rm_elems<D, NT * 32>() + tr_elems<D, NT * 32>());
}
template <int D, int NT> constexpr int bwd_lds_bytes() {
    return 2 * (4 * rm_elems<D, NT * 32>() + 3 * tr_elems<D, NT * 32>()) + 4 * 2 * NT * 32;
}
constexpr int kLdsLimit = 160 * 1024;

// ---------------------------------------------------------------------------
// The last tile of a sequence of 32 n + 1 .. 32 n + 4 rows (a virtual node behind a multiple of 32)
// holds one to four rows.  As a matrix tile it would cost its wave as much as a full one, so the wave
// that owns it works on the vector unit instead, lane = key (or query), one row at a time: dot
// products from the LDS images, reductions over the wave.  Probabilities and dS are rounded to bf16
// where the matrix path rounds them.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) x += __shfl_xor(x, off);
    return x;
}
__device__ __forceinline__ float wave_max(float x) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) x = fmaxf(x, __shfl_xor(x, off));
    return x;
}
__device__ __forceinline__ float round_bf(float x) { return bf2f(f2bf(x)); }
template <int D>
__device__ __forceinline__ void lds_row(const short* __restrict__ rm, int row, float (&x)[D]) {
#pragma unroll
    for (int c = 0; c < D / 4; ++c) {
        const short4_t v = *reinterpret_cast<const short4_t*>(&rm[row * D + 4 * c]);
        x[4 * c + 0] = bf2f(v.x); x[4 * c + 1] = bf2f(v.y); x[4 * c + 2] = bf2f(v.z); x[4 * c + 3] = bf2f(v.w);
    }
}
template <int D>
__device__ __forceinline__ float dot_d(const float (&a)[D], const float (&b)[D]) {
    float t = 0.f;
#pragma unroll
    for (int c = 0; c < D; ++c) t = fmaf(a[c], b[c], t);
    return t;
}
template <typename T, int D>
__device__ __forceinline__ void store_row(T* __restrict__ p, const float (&x)[D], float f) {
#pragma unroll
    for (int c = 0; c < D; c += 4) st4(p + c, x[c] * f, x[c + 1] * f, x[c + 2] * f, x[c + 3] * f);
}

// forward of the rows first .. first + count - 1 (all keys), by one wave
template <typename T, typename BT, int D, int SP, bool DROP>
__device__ __forceinline__ void thin_rows_fwd(const T* __restrict__ Q, const short* __restrict__ k_rm,
                                              const short* __restrict__ v_tr, const BT* __restrict__ bias_gh, int bstride,
                                              T* __restrict__ out, float* __restrict__ lse, int g, int h, int S, int H,
                                              float scale, int first, int count, int lane, const DropArgs da) {
    constexpr int NC = (SP + 63) / 64;
    for (int tq = 0; tq < count; ++tq) {
        const int qi = first + tq;
        float qv[D];
#pragma unroll
        for (int c = 0; c < D / 4; ++c) {
            const short4_t v = ld4(Q + (((int64_t)g * S + qi) * H + h) * D + 4 * c);
            qv[4 * c + 0] = bf2f(v.x); qv[4 * c + 1] = bf2f(v.y); qv[4 * c + 2] = bf2f(v.z); qv[4 * c + 3] = bf2f(v.w);
        }
        const BT* brow = bias_gh ? bias_gh + (int64_t)qi * bstride : nullptr;
        float sv[NC], mx = -INFINITY;
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            const int key = c * 64 + lane;
            sv[c] = -INFINITY;
            if (key < S) {
                float kv[D];
                lds_row<D>(k_rm, key, kv);
                sv[c] = fmaf(dot_d<D>(qv, kv), scale, brow ? ld1(brow + key) : 0.f);
            }
            mx = fmaxf(mx, sv[c]);
        }
        mx = wave_max(mx);
        const float m_use = (mx == -INFINITY) ? 0.f : mx;
        float lsum = 0.f, ov[D];
#pragma unroll
        for (int d = 0; d < D; ++d) ov[d] = 0.f;
        const uint32_t rh = DROP ? drop_row_hash(da, g * H + h, qi) : 0u;
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            const int key = c * 64 + lane;
            if (key < S) {
                const float pb = round_bf(fast_exp2((sv[c] - m_use) * kLog2e));
                lsum += pb;
                const float pk = (!DROP || drop_keep(da, rh, key)) ? pb : 0.f;
#pragma unroll
                for (int d = 0; d < D; ++d) ov[d] = fmaf(pk, bf2f(v_tr[d * (SP + 4) + key]), ov[d]);
            }
        }
        lsum = wave_sum(lsum);
#pragma unroll
        for (int d = 0; d < D; ++d) ov[d] = wave_sum(ov[d]);
        if (lane == 0) {
            store_row<T, D>(out + (((int64_t)g * S + qi) * H + h) * D, ov, (DROP ? da.inv_keep : 1.0f) / lsum);
            lse[((int64_t)g * H + h) * S + qi] = m_use + __logf(lsum);
        }
    }
}

// backward, query side, of the rows first .. first + count - 1: dQ and their rows of dBias
template <typename T, typename BT, int D, int SP, bool DROP>
__device__ __forceinline__ void thin_rows_bwd_q(const short* __restrict__ q_rm, const short* __restrict__ k_rm,
                                                const short* __restrict__ v_rm, const short* __restrict__ g_rm,
                                                const float* __restrict__ lse_l, const float* __restrict__ dd_l,
                                                const BT* __restrict__ bias_gh, int bstride, T* __restrict__ dbias_gh,
                                                T* __restrict__ dQ, int g, int h, int S, int H, float scale, int first,
                                                int count, int lane, const DropArgs da, const IdsAcc& acc) {
    constexpr int NC = (SP + 63) / 64;
    const float scale2 = scale * kLog2e;
    for (int tq = 0; tq < count; ++tq) {
        const int qi = first + tq;
        float qv[D], gv[D], dq[D];
        lds_row<D>(q_rm, qi, qv);
        lds_row<D>(g_rm, qi, gv);
#pragma unroll
        for (int d = 0; d < D; ++d) dq[d] = 0.f;
        const float nL2 = -lse_l[qi], Dq = dd_l[qi];
        const uint32_t rh = DROP ? drop_row_hash(da, g * H + h, qi) : 0u;
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            const int key = c * 64 + lane;
            if (key < S) {
                float kv[D], vv[D];
                lds_row<D>(k_rm, key, kv);
                lds_row<D>(v_rm, key, vv);
                const float b = bias_gh ? ld1(bias_gh + (int64_t)qi * bstride + key) : 0.f;
                const float pv = fast_exp2(fmaf(dot_d<D>(qv, kv), scale2, fmaf(b, kLog2e, nL2)));
                const float ks = !DROP ? 1.0f : (drop_keep(da, rh, key) ? da.inv_keep : 0.f);
                const float dS = pv * (dot_d<D>(gv, vv) * ks - Dq);
                if (dbias_gh) st1(dbias_gh + (int64_t)qi * S + key, dS);
                if (acc.on) acc_position(acc, dS, (int64_t)qi * S + key);
                const float dsb = round_bf(dS);
#pragma unroll
                for (int d = 0; d < D; ++d) dq[d] = fmaf(dsb, kv[d], dq[d]);
            }
        }
#pragma unroll
        for (int d = 0; d < D; ++d) dq[d] = wave_sum(dq[d]);
        if (lane == 0) store_row<T, D>(dQ + (((int64_t)g * S + qi) * H + h) * D, dq, scale);
    }
}

// backward, key side, of the keys first .. first + count - 1 (all queries): dK and dV
template <typename T, typename BT, int D, int SP, bool DROP>
__device__ __forceinline__ void thin_rows_bwd_k(const short* __restrict__ q_rm, const short* __restrict__ k_rm,
                                                const short* __restrict__ v_rm, const short* __restrict__ g_rm,
                                                const float* __restrict__ lse_l, const float* __restrict__ dd_l,
                                                const BT* __restrict__ bias_gh, int bstride, T* __restrict__ dK, T* __restrict__ dV,
                                                int g, int h, int S, int H, float scale, int first, int count, int lane,
                                                const DropArgs da, float* __restrict__ dq_slab = nullptr,
                                                T* __restrict__ dbias_gh = nullptr) {
    // dq_slab (one-walk backward): this wave's share of dQ, [query][D] floats in LDS - the sums over these keys of
    // dS k for the queries in front of `first` (the rows from `first` on get their dQ from thin_rows_bwd_q) - and
    // dbias_gh: the keys' column of dBias for the same queries.
    constexpr int NC = (SP + 63) / 64;
    const float scale2 = scale * kLog2e;
    for (int tk = 0; tk < count; ++tk) {
        const int ki = first + tk;
        float kv[D], vv[D], dk[D], dv[D];
        lds_row<D>(k_rm, ki, kv);
        lds_row<D>(v_rm, ki, vv);
#pragma unroll
        for (int d = 0; d < D; ++d) { dk[d] = 0.f; dv[d] = 0.f; }
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            const int qq = c * 64 + lane;
            if (qq < S) {
                float qv[D], gv[D];
                lds_row<D>(q_rm, qq, qv);
                lds_row<D>(g_rm, qq, gv);
                const float b = bias_gh ? ld1(bias_gh + (int64_t)qq * bstride + ki) : 0.f;
                const float pv = fast_exp2(fmaf(dot_d<D>(qv, kv), scale2, fmaf(b, kLog2e, -lse_l[qq])));
                const float ks = !DROP ? 1.0f : (drop_keep(da, drop_row_hash(da, g * H + h, qq), ki) ? da.inv_keep : 0.f);
                const float dS = pv * (dot_d<D>(gv, vv) * ks - dd_l[qq]);
                const float pb = round_bf(pv * ks), dsb = round_bf(dS);
#pragma unroll
                for (int d = 0; d < D; ++d) {
                    dk[d] = fmaf(dsb, qv[d], dk[d]);
                    dv[d] = fmaf(pb, gv[d], dv[d]);
                }
                if (dq_slab != nullptr && qq < first) {       // the same lane owns query qq for every key
#pragma unroll
                    for (int d = 0; d < D; ++d) dq_slab[qq * D + d] = (tk == 0 ? 0.f : dq_slab[qq * D + d]) + dsb * kv[d];
                    if (dbias_gh != nullptr) st1(dbias_gh + (int64_t)qq * S + ki, dS);
                }
            }
        }
#pragma unroll
        for (int d = 0; d < D; ++d) { dk[d] = wave_sum(dk[d]); dv[d] = wave_sum(dv[d]); }
        if (lane == 0) {
            store_row<T, D>(dK + (((int64_t)g * S + ki) * H + h) * D, dk, scale);
            store_row<T, D>(dV + (((int64_t)g * S + ki) * H + h) * D, dv, 1.0f);
        }
    }
}

// ---------------------------------------------------------------------------
// forward: online softmax over key tiles, in the base-2 domain
// ---------------------------------------------------------------------------
template <typename T, int D, int NT, bool DROP, int BSRC>
__global__ __launch_bounds__(64 * NT, 2) void k_dense_fwd(const T* __restrict__ Q, const T* __restrict__ K,
                                                       const T* __restrict__ V, const T* __restrict__ bias,
                                                       T* __restrict__ out, float* __restrict__ lse, int S,
                                                       int H, float scale, int nb, const DropArgs da, const IdsArgs ia) {
    constexpr int KS = D / 8;
    constexpr int SP = NT * 32;
    using BT = typename std::conditional<BSRC == 1, dbf16, T>::type;     // element type of the bias as the walks read it
    extern __shared__ __align__(16) char smem[];
    short* k_rm = reinterpret_cast<short*>(smem);
    short* v_tr = k_rm + rm_elems<D, SP>();
    IdsLds il{};
    if constexpr (BSRC == 1) {
        // the grid is a multiple of 8 H, so every pair of this workgroup has the same head: its tables are loaded once
        il = ids_lds(smem + fwd_lds_bytes<D, NT>(), S, ia.ns, ia.ne);
        ids_load_tables<T>(ia, (blockIdx.x % (8 * H)) >> 3, H, il);
        __syncthreads();
    }
    // XCD-aware placement: workgroups go to the 8 XCDs round-robin, and the H heads of a graph
    // share every 128-byte line of q/k/v ([b,S,H,d] layout), so the heads of graph g are given the
    // workgroup ids congruent to g mod 8 inside a window of 8*H ids - same XCD, same L2, same time.
    // Workgroups are persistent: the grid holds as many as the GPU keeps resident and each walks the
    // (graph, head) pairs pair, pair + gridDim.x, ... (gridDim.x is a multiple of 8, so a workgroup
    // stays on the XCD its pairs were assigned to).
    const int total_pairs = ((nb + 7) / 8) * 8 * H;
    for (int pair = blockIdx.x; pair < total_pairs; pair += gridDim.x) {
    const int win = pair / (8 * H), rem = pair % (8 * H);
    const int g = win * 8 + (rem & 7), h = rem >> 3;
    if (g >= nb) continue;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int col = lane & 31, half = lane >> 5;
    const int q0 = wave * 32, qi = q0 + col;
    const bool qok = qi < S;
    const bool hasb = BSRC == 1 || bias != nullptr;
    // a last tile of at most four rows is not worth a matrix tile: its wave takes the vector path
    const bool vec_wave = wave == NT - 1 && S - (NT - 1) * 32 <= 4;
    // this lane's query row of the bias; the first tile's group of it is requested before anything else
    const T* brow = (BSRC == 0 && hasb) ? bias + (((int64_t)g * H + h) * S + (qok ? qi : 0)) * S : nullptr;
    const short* trow = BSRC == 1 ? il.tile + (qok ? qi : 0) * il.bst : nullptr;      // the same row of the LDS tile
    Bias16<BT> bcur, bnext;
    zero_bias16(bcur);
    zero_bias16(bnext);
    if constexpr (BSRC == 0) {
        if (hasb && qok && !vec_wave) load_bias16(brow + 16 * half, min(16, S - 16 * half), bcur);
    } else {
        ids_build_tile<T, 2>(ia, g, S, il);
    }
    load_head<T, D, SP>(K, g, h, S, H, k_rm, nullptr);
    load_head<T, D, SP>(V, g, h, S, H, nullptr, v_tr);
    short4_t bq[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        bq[s] = zero4();
        if (qok) bq[s] = ld4(Q + (((int64_t)g * S + qi) * H + h) * D + s * 8 + half * 4);
    }
    __syncthreads();
    if constexpr (BSRC == 1) {
        if (qok && !vec_wave && 16 * half < S) load_tile16(trow + 16 * half, bcur);
    }
    if (vec_wave) {
        const BT* bias_gh = nullptr;
        if constexpr (BSRC == 1) bias_gh = reinterpret_cast<const dbf16*>(il.tile);
        else bias_gh = hasb ? bias + ((int64_t)g * H + h) * S * S : nullptr;
        thin_rows_fwd<T, BT, D, SP, DROP>(Q, k_rm, v_tr, bias_gh, BSRC == 1 ? il.bst : S, out, lse, g, h, S, H, scale,
                                          (NT - 1) * 32, S - (NT - 1) * 32, lane, da);
    } else {
    const int krow = key_of_row(col);            // key (inside a tile) of this lane's A-operand row
    // Row sums on the matrix unit: with a head dim below 32 the A operand of O^T = V^T P^T has idle
    // rows, and a row of ones there makes row D of the product the sum of the (bf16-rounded)
    // probabilities, the very numbers the numerator was built from.  It is C register 4*KS of the lower half.
    // (not with dropout: the sum runs over all probabilities, the numerator over the kept ones)
    constexpr bool kSumOnMfma = D < 32 && !DROP;
    const short one_bits = 0x3f80;               // bf16 1.0
    const uint32_t rh = DROP ? drop_row_hash(da, g * H + h, qi) : 0u;
    float m = -INFINITY, l = 0.f;                // running maximum and sum (natural units)
    float16_t o = zero16();
    const int tail = S - (NT - 1) * 32;          // keys in the last tile
    const bool thin = tail <= 4;
    const int nt_full = thin ? NT - 1 : NT;      // tiles that take the general path
#pragma unroll 1
    for (int kt = 0; kt < nt_full; ++kt) {
        const int kb = kt * 32 + 16 * half;      // this lane's keys: kb .. kb + 15
        if (kt + 1 < NT && hasb && qok) {        // the next tile's group, a whole tile ahead of its use
            const int nv = S - (kb + 32);
            if constexpr (BSRC == 1) {
                if (nv > 0) load_tile16(trow + kb + 32, bnext);
            } else {
                if (nv > 0) load_bias16(brow + kb + 32, min(16, nv), bnext);
            }
        }
        float16_t sc = zero16();
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            const short4_t a = *reinterpret_cast<const short4_t*>(&k_rm[(kt * 32 + krow) * D + s * 8 + half * 4]);
            sc = mfma(a, bq[s], sc);
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) sc[r] = fmaf(sc[r], scale, bcur.get(r));
        if (kt * 32 + 32 > S) {                  // the row ends inside this tile (wave-uniform)
#pragma unroll
            for (int r = 0; r < 16; ++r) sc[r] = kb + r < S ? sc[r] : -INFINITY;
        }
        float tmax = max3(sc[0], sc[1], sc[2]);
#pragma unroll
        for (int r = 3; r < 15; r += 2) tmax = max3(tmax, sc[r], sc[r + 1]);
        tmax = fmaxf(tmax, sc[15]);
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32));
        const float m_new = fmaxf(m, tmax);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = fast_exp2((m - m_use) * kLog2e);
        const float nm2 = -m_use * kLog2e;
#pragma unroll
        for (int r = 0; r < 4 * KS + (kSumOnMfma ? 4 : 0); ++r) o[r] *= alpha;
        if (!kSumOnMfma) l *= alpha;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            sc[r] = fast_exp2(fmaf(sc[r], kLog2e, nm2));
            if (!kSumOnMfma) l += sc[r];
            if (DROP) sc[r] = drop_keep(da, rh, kb + r) ? sc[r] : 0.f;
        }
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            short4_t pb;
            pb = pack4(sc[4 * t + 0], sc[4 * t + 1], sc[4 * t + 2], sc[4 * t + 3]);
            short4_t av = zero4();
            if (col < D) av = *reinterpret_cast<const short4_t*>(&v_tr[col * (SP + 4) + kb + 4 * t]);
            if (kSumOnMfma && col == D) { av.x = one_bits; av.y = one_bits; av.z = one_bits; av.w = one_bits; }
            o = mfma(av, pb, o);        // O^T += V^T P^T (the B operand's keys are kb + 4t .. +3)
        }
        m = m_new;
        bcur = bnext;
        }
    if (thin) {
        constexpr int kt = NT - 1;
        const int kb = kt * 32 + 16 * half;
        float16_t sc = zero16();
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            const short4_t a = *reinterpret_cast<const short4_t*>(&k_rm[(kt * 32 + krow) * D + s * 8 + half * 4]);
            sc = mfma(a, bq[s], sc);
        }
        // the last tile holds at most four keys (a virtual node behind a multiple of 32): they are
        // registers 0..3 of the lower half, one group of the second product instead of four
        float s4[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) s4[r] = (half == 0 && r < tail) ? fmaf(sc[r], scale, bcur.get(r)) : -INFINITY;
        float tmax = fmaxf(max3(s4[0], s4[1], s4[2]), s4[3]);
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32));
        const float m_new = fmaxf(m, tmax);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = fast_exp2((m - m_use) * kLog2e);
        const float nm2 = -m_use * kLog2e;
#pragma unroll
        for (int r = 0; r < 4 * KS + (kSumOnMfma ? 4 : 0); ++r) o[r] *= alpha;
        if (!kSumOnMfma) l *= alpha;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            s4[r] = fast_exp2(fmaf(s4[r], kLog2e, nm2));
            if (!kSumOnMfma) l += s4[r];
            if (DROP) s4[r] = drop_keep(da, rh, kb + r) ? s4[r] : 0.f;
        }
        short4_t pb;
        pb = pack4(s4[0], s4[1], s4[2], s4[3]);
        short4_t av = zero4();
        if (col < D) av = *reinterpret_cast<const short4_t*>(&v_tr[col * (SP + 4) + kb]);
        if (kSumOnMfma && col == D) { av.x = one_bits; av.y = one_bits; av.z = one_bits; av.w = one_bits; }
        o = mfma(av, pb, o);
        m = m_new;
    }
    if (kSumOnMfma) l = __shfl(o[4 * KS], col);      // row D sits in the lower half's register 4*KS
    else l += __shfl_xor(l, 32);
    if (qok) {
        const float inv = (DROP ? da.inv_keep : 1.0f) / l;
        T* op = out + (((int64_t)g * S + qi) * H + h) * D;
#pragma unroll
        for (int rb = 0; rb < KS; ++rb)
            st4(op + 8 * rb + 4 * half, o[4 * rb + 0] * inv, o[4 * rb + 1] * inv, o[4 * rb + 2] * inv,
                o[4 * rb + 3] * inv);
        if (half == 0) lse[((int64_t)g * H + h) * S + qi] = (m == -INFINITY ? 0.f : m) + __logf(l);
    }
    }
    __syncthreads();     // the LDS images are rewritten for the next pair
    }
}

// ---------------------------------------------------------------------------
// backward
// ---------------------------------------------------------------------------
// Wave w first acts on query tile w (transposed scores, lane = query): dQ.  Then
// on key tile w (direct scores, lane = key): dK and dV.  dBias = dS is written by the first walk
// (a lane holds 16 consecutive keys of one row there: vector stores).  Both walks read the
// bias straight from global memory in the layout their lanes need (a lane's own row
// in the first, 32 lanes on 32 consecutive keys of one row in the second); the second
// read of a (graph, head) slice comes from L2.
template <typename T, int D, int NT, bool DROP, int BSRC>
__global__ __launch_bounds__(64 * NT, 2) void k_dense_bwd(const T* __restrict__ Q, const T* __restrict__ K,
                                                       const T* __restrict__ V, const T* __restrict__ bias,
                                                       const T* __restrict__ O, const float* __restrict__ lse,
                                                       const T* __restrict__ dO, T* __restrict__ dQ,
                                                       T* __restrict__ dK, T* __restrict__ dV,
                                                       T* __restrict__ dbias, int S, int H, float scale, int nb,
                                                       const DropArgs da, const IdsArgs ia) {
    constexpr int KS = D / 8;
    constexpr int SP = NT * 32;
    using BT = typename std::conditional<BSRC == 1, dbf16, T>::type;
    extern __shared__ __align__(16) char smem[];
    constexpr int RM = rm_elems<D, SP>(), TR = tr_elems<D, SP>();
    short* q_rm = reinterpret_cast<short*>(smem);
    short* k_rm = q_rm + RM;
    short* v_rm = k_rm + RM;
    short* g_rm = v_rm + RM;          // g = dout
    short* q_tr = g_rm + RM;
    short* k_tr = q_tr + TR;
    short* g_tr = k_tr + TR;
    float* lse_l = reinterpret_cast<float*>(g_tr + TR);   // lse * log2(e)
    float* dd_l = lse_l + SP;
    IdsLds il{};
    IdsAcc acc{};
    if constexpr (BSRC == 1) {
        // the grid is a multiple of 8 H: one head per workgroup, whose tables are loaded and whose accumulators are
        // cleared once
        il = ids_lds(smem + bwd_lds_bytes<D, NT>(), S, ia.ns, ia.ne);
        ids_load_tables<T>(ia, (blockIdx.x % (8 * H)) >> 3, H, il);
        for (int i = threadIdx.x; i < kHotCopies * kHotStride + ia.ns + ia.ne + 2 + 2; i += blockDim.x) il.hot[i] = 0;   // .. and the bound words
        acc.F = ia.F; acc.ns = ia.ns; acc.ne = ia.ne; acc.hot_n = min(kHotIds, ia.ns);
        acc.hot_copy = il.hot + (threadIdx.x % kHotCopies) * kHotStride;
        acc.accS = il.accS; acc.accE = il.accE;
        acc.on = ia.partial != nullptr;
        if (acc.on)       // the partial starts at zero (a workgroup whose pairs all lie past the batch adds nothing)
            for (int k = threadIdx.x; k < ia.ns + ia.ne + 1; k += blockDim.x) ia.partial[(int64_t)blockIdx.x * (ia.ns + ia.ne + 1) + k] = 0.f;
        __syncthreads();
    }
    // XCD-aware placement as in the forward.  With the bias in memory one workgroup per (graph, head) pair (it runs
    // longer per pair than the forward, persistence does not pay); with ids the grid is what the GPU keeps resident
    // and a workgroup walks pairs of its head, so that it writes its table partial once.
    const int total_pairs = ((nb + 7) / 8) * 8 * H;
    for (int pair = blockIdx.x; pair < total_pairs; pair += gridDim.x) {
    const int win = pair / (8 * H), rem = pair % (8 * H);
    const int g = win * 8 + (rem & 7), h = rem >> 3;
    if (g >= nb) {
        if constexpr (BSRC == 0) return;
        else continue;
    }
    // In the loop over pairs the compiler would compute everything that depends on the lane alone once, ahead of
    // the loop, and keep it in registers through both walks (256 registers and spills instead of 160): the thread
    // id is handed to it as a value it cannot see through, once per pair.
    int tid = threadIdx.x;
    if constexpr (BSRC == 1) asm volatile("v_mov_b32 %0, %1" : "=v"(tid) : "v"(tid));
    const int wave = BSRC == 1 ? __builtin_amdgcn_readfirstlane(tid >> 6) : tid >> 6, lane = tid & 63;
    const int col = lane & 31, half = lane >> 5;
    const bool hasb = BSRC == 1 || bias != nullptr;
    const int tail = S - (NT - 1) * 32;          // rows / keys in the last tile
    const bool thin = tail <= 4;
    const int nt_full = thin ? NT - 1 : NT;      // tiles that take the general path
    const int bstride = BSRC == 1 ? il.bst : S;  // row stride of the bias as the walks read it
    const BT* bias_gh = nullptr;
    if constexpr (BSRC == 1) bias_gh = reinterpret_cast<const dbf16*>(il.tile);
    else bias_gh = hasb ? bias + ((int64_t)g * H + h) * S * S : nullptr;
    // the first query-major group of this lane's bias row, requested before anything else
    const int qi = wave * 32 + col;
    const bool qok = qi < S;
    const T* brow = nullptr;
    if constexpr (BSRC == 0) brow = hasb ? bias_gh + (int64_t)(qok ? qi : 0) * S : nullptr;
    const short* trow = BSRC == 1 ? il.tile + (qok ? qi : 0) * il.bst : nullptr;
    Bias16<BT> bcur, bnext;
    zero_bias16(bcur);
    zero_bias16(bnext);
    const bool vec_wave = thin && wave == NT - 1;     // the wave of a last tile of at most four rows: vector path
    if constexpr (BSRC == 0) {
        if (hasb && qok && !vec_wave) load_bias16(brow + 16 * half, min(16, S - 16 * half), bcur);
    } else {
        ids_build_tile<T, 4>(ia, g, S, il);
        acc.sp = ia.sp + (int64_t)g * S * S;
        acc.et = ia.et + (int64_t)g * S * S * ia.F;
    }
    load_head<T, D, SP>(Q, g, h, S, H, q_rm, q_tr);
    load_head<T, D, SP>(K, g, h, S, H, k_rm, k_tr);
    load_head<T, D, SP>(V, g, h, S, H, v_rm, nullptr);
    load_head<T, D, SP>(dO, g, h, S, H, g_rm, g_tr);
    for (int i = threadIdx.x; i < SP; i += blockDim.x) {
        float dsum = 0.f, L = 0.f, g1 = 0.f, vm = 0.f;
        if (i < S) {
            L = lse[((int64_t)g * H + h) * S + i];
            const T* op = O + (((int64_t)g * S + i) * H + h) * D;
            const T* gp = dO + (((int64_t)g * S + i) * H + h) * D;
#pragma unroll
            for (int c = 0; c < D; c += 4) {
                const short4_t ov = ld4(op + c);
                const short4_t gv = ld4(gp + c);
                dsum += bf2f(ov.x) * bf2f(gv.x) + bf2f(ov.y) * bf2f(gv.y) + bf2f(ov.z) * bf2f(gv.z) +
                        bf2f(ov.w) * bf2f(gv.w);
                if (BSRC == 1) g1 += fabsf(bf2f(gv.x)) + fabsf(bf2f(gv.y)) + fabsf(bf2f(gv.z)) + fabsf(bf2f(gv.w));
            }
            if (BSRC == 1 && acc.on) {
                const T* vp = V + (((int64_t)g * S + i) * H + h) * D;
#pragma unroll
                for (int c = 0; c < D; c += 4) {
                    const short4_t vv = ld4(vp + c);
                    vm = fmaxf(fmaxf(vm, fmaxf(fabsf(bf2f(vv.x)), fabsf(bf2f(vv.y)))), fmaxf(fabsf(bf2f(vv.z)), fabsf(bf2f(vv.w))));
                }
            }
        }
        lse_l[i] = L * kLog2e;
        dd_l[i] = dsum;          // D[q] = sum_dd dout[q,dd] out[q,dd]
        if (BSRC == 1 && acc.on && i < S) {      // non-negative floats order like their bit patterns (a NaN ends up largest)
            atomicMax(il.bound, __float_as_int(g1));
            atomicMax(il.bound + 1, __float_as_int(vm));
        }
    }
    __syncthreads();
    if constexpr (BSRC == 1) {
        if (qok && !vec_wave && 16 * half < S) load_tile16(trow + 16 * half, bcur);
        // this pair's scale: 2^22 / B', B' = the bound on a row's sum of |dS| rounded up to a power of two (0: nothing to add)
        const float B = 2.f * (DROP ? da.inv_keep : 1.0f) * __int_as_float(il.bound[0]) * __int_as_float(il.bound[1]);
        int e = 0;
        acc.scale = 0.f;
        acc.scale_e = 0.f;
        if (acc.on && B > 0.f && B < INFINITY) {
            (void)frexpf(B, &e);
            acc.scale = ldexpf(1.f, 22 - e);
            // an edge id repeated in all F features of a position collects F dS: the bound of an edge accumulator is
            // F S B, and its unit is 2^ceil(log2 F) times coarser
            acc.scale_e = ldexpf(1.f, 22 - e - (ia.F > 1 ? 32 - __clz(ia.F - 1) : 0));
        }
    }

    // ---- query tile `wave`: dQ -------------------------------------------------
    if (vec_wave) {
        thin_rows_bwd_q<T, BT, D, SP, DROP>(q_rm, k_rm, v_rm, g_rm, lse_l, dd_l, bias_gh, bstride,
                                            dbias != nullptr ? dbias + ((int64_t)g * H + h) * S * S : nullptr, dQ, g, h, S, H,
                                            scale, (NT - 1) * 32, tail, lane, da, acc);
    } else {
        short4_t bq[KS], bg[KS];
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            bq[s] = *reinterpret_cast<const short4_t*>(&q_rm[qi * D + s * 8 + half * 4]);
            bg[s] = *reinterpret_cast<const short4_t*>(&g_rm[qi * D + s * 8 + half * 4]);
        }
        const float nL2 = -lse_l[qi], Dq = dd_l[qi];
        const float scale2 = scale * kLog2e;
        const int krow = key_of_row(col);
        const uint32_t rh = DROP ? drop_row_hash(da, g * H + h, qi) : 0u;
        T* dbrow = dbias != nullptr ? dbias + (((int64_t)g * H + h) * S + (qok ? qi : 0)) * S : nullptr;
        const bool acc_here = BSRC == 1 && acc.on && qok;
        float16_t dq = zero16();
#pragma unroll 1
        for (int kt = 0; kt < nt_full; ++kt) {
            const int kb = kt * 32 + 16 * half;
            if (kt + 1 < NT && hasb && qok) {
                const int nv = S - (kb + 32);
                if constexpr (BSRC == 1) {
                    if (nv > 0) load_tile16(trow + kb + 32, bnext);
                } else {
                    if (nv > 0) load_bias16(brow + kb + 32, min(16, nv), bnext);
                }
            }
            // the ids of this lane's sixteen positions, asked for now and used after the products
            Bias16<dbf16> spraw, etraw;
            zero_bias16(spraw);
            zero_bias16(etraw);
            if (acc_here && kb < S) {
                load_bias16(reinterpret_cast<const dbf16*>(acc.sp) + (int64_t)qi * S + kb, min(16, S - kb), spraw);
                if (acc.F == 1) load_bias16(reinterpret_cast<const dbf16*>(acc.et) + (int64_t)qi * S + kb, min(16, S - kb), etraw);
            }
            float16_t sc = zero16(), dp = zero16();
#pragma unroll
            for (int s = 0; s < KS; ++s) {
                const short4_t ak = *reinterpret_cast<const short4_t*>(&k_rm[(kt * 32 + krow) * D + s * 8 + half * 4]);
                const short4_t av = *reinterpret_cast<const short4_t*>(&v_rm[(kt * 32 + krow) * D + s * 8 + half * 4]);
                sc = mfma(ak, bq[s], sc);     // S^T[key, query]
                dp = mfma(av, bg[s], dp);     // dP^T[key, query] = V dout^T
            }
            // p = 2^(s*scale*log2e + (bias*log2e - lse*log2e)); dS^T = p (dP^T - D)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float pv = fast_exp2(fmaf(sc[r], scale2, fmaf(bcur.get(r), kLog2e, nL2)));
                if (DROP) dp[r] = drop_keep(da, rh, kb + r) ? dp[r] * da.inv_keep : 0.f;
                sc[r] = pv * (dp[r] - Dq);
            }
            if (kt * 32 + 32 > S) {               // the row ends inside this tile (wave-uniform)
#pragma unroll
                for (int r = 0; r < 16; ++r) sc[r] = kb + r < S ? sc[r] : 0.f;
            }
            short4_t db[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                db[t] = pack4(sc[4 * t + 0], sc[4 * t + 1], sc[4 * t + 2], sc[4 * t + 3]);
            }
            if (acc_here && kb < S) {      // dS into the table accumulators (keys past the end carry zeros)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc_spatial(acc, sc[r], (spraw.w[r >> 1] >> (16 * (r & 1))) & 0xffffu);
                // most pairs of nodes are not edges (id 0): a lane whose sixteen edge ids are all zero skips them
                if (acc.F == 1 && (etraw.w[0] | etraw.w[1] | etraw.w[2] | etraw.w[3] | etraw.w[4] | etraw.w[5] | etraw.w[6] | etraw.w[7])) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc_edge(acc, sc[r], (etraw.w[r >> 1] >> (16 * (r & 1))) & 0xffffu);
                }
                if (acc.F != 1) {
                    for (int r = 0; r < 16; ++r)
                        if (sc[r] != 0.f)
                            for (int f = 0; f < acc.F; ++f) acc_edge(acc, sc[r], acc.et[((int64_t)qi * S + kb + r) * acc.F + f]);
                }
            }
            // dBias = dS: this lane holds 16 consecutive keys of its query row, one 32/64-byte piece
            if (dbrow != nullptr && qok) {
                if (kb + 16 <= S) {
                    if (sizeof(T) == 2) {
                        __builtin_memcpy(dbrow + kb, db, 32);
                    } else {
#pragma unroll
                        for (int r = 0; r < 16; ++r) st1(dbrow + kb + r, sc[r]);
                    }
                } else {
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        if (kb + r < S) st1(dbrow + kb + r, sc[r]);
                }
            }
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                short4_t ak = zero4();
                if (col < D) ak = *reinterpret_cast<const short4_t*>(&k_tr[col * (SP + 4) + kb + 4 * t]);
                dq = mfma(ak, db[t], dq);     // dQ^T[dd, query] += K^T dS^T
            }
            bcur = bnext;
        }
        if (thin) {
            constexpr int kt = NT - 1;
            const int kb = kt * 32 + 16 * half;
            float16_t sc = zero16(), dp = zero16();
#pragma unroll
            for (int s = 0; s < KS; ++s) {
                const short4_t ak = *reinterpret_cast<const short4_t*>(&k_rm[(kt * 32 + krow) * D + s * 8 + half * 4]);
                const short4_t av = *reinterpret_cast<const short4_t*>(&v_rm[(kt * 32 + krow) * D + s * 8 + half * 4]);
                sc = mfma(ak, bq[s], sc);
                dp = mfma(av, bg[s], dp);
            }
            // at most four keys in the last tile: registers 0..3 of the lower half
            float s4[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float pv = fast_exp2(fmaf(sc[r], scale2, fmaf(bcur.get(r), kLog2e, nL2)));
                if (DROP) dp[r] = drop_keep(da, rh, kb + r) ? dp[r] * da.inv_keep : 0.f;
                s4[r] = (half == 0 && r < tail) ? pv * (dp[r] - Dq) : 0.f;
            }
            if (dbrow != nullptr && qok && half == 0) {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (r < tail) st1(dbrow + kb + r, s4[r]);
            }
            if (acc_here && half == 0) {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (r < tail) acc_position(acc, s4[r], (int64_t)qi * S + kb + r);
            }
            short4_t db0;
            db0 = pack4(s4[0], s4[1], s4[2], s4[3]);
            short4_t ak = zero4();
            if (col < D) ak = *reinterpret_cast<const short4_t*>(&k_tr[col * (SP + 4) + kb]);
            dq = mfma(ak, db0, dq);
        }
        if (qok) {
            T* p = dQ + (((int64_t)g * S + qi) * H + h) * D;
#pragma unroll
            for (int rb = 0; rb < KS; ++rb)
                st4(p + 8 * rb + 4 * half, dq[4 * rb + 0] * scale, dq[4 * rb + 1] * scale, dq[4 * rb + 2] * scale,
                    dq[4 * rb + 3] * scale);
        }
    }

    // ---- key tile `wave`: dK, dV -------------------------------------------------
    if (vec_wave) {
        thin_rows_bwd_k<T, BT, D, SP, DROP>(q_rm, k_rm, v_rm, g_rm, lse_l, dd_l, bias_gh, bstride, dK, dV, g, h, S, H, scale,
                                            (NT - 1) * 32, tail, lane, da);
    } else {
        const int k0 = wave * 32, ki = k0 + col;
        const bool kok = ki < S;
        short4_t bk[KS], bv[KS];
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            bk[s] = *reinterpret_cast<const short4_t*>(&k_rm[ki * D + s * 8 + half * 4]);
            bv[s] = *reinterpret_cast<const short4_t*>(&v_rm[ki * D + s * 8 + half * 4]);
        }
        // register r of a lane is query qt*32 + 8*(r/4) + 4*half + r%4; for one r the 32 lanes of a
        // half read 32 consecutive keys of that query's bias row (second read of the slice: L2)
        const BT* bcol = hasb ? bias_gh + (kok ? ki : 0) : nullptr;
        decltype(raw1(bcol)) braw[16], braw_next[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) { braw[r] = 0; braw_next[r] = 0; }
        if (hasb && kok) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int qq = 8 * (r / 4) + 4 * half + (r % 4);
                if (qq < S) braw[r] = raw1(bcol + (int64_t)qq * bstride);
            }
        }
        const float scale2 = scale * kLog2e;
        float16_t dk = zero16(), dv = zero16();
#pragma unroll 1
        for (int qt = 0; qt < nt_full; ++qt) {
            if (qt + 1 < NT && hasb && kok) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int qq = (qt + 1) * 32 + 8 * (r / 4) + 4 * half + (r % 4);
                    if (qq < S) braw_next[r] = raw1(bcol + (int64_t)qq * bstride);
                }
            }
            float16_t sc = zero16(), dp = zero16();
#pragma unroll
            for (int s = 0; s < KS; ++s) {
                const short4_t aq = *reinterpret_cast<const short4_t*>(&q_rm[(qt * 32 + col) * D + s * 8 + half * 4]);
                const short4_t ag = *reinterpret_cast<const short4_t*>(&g_rm[(qt * 32 + col) * D + s * 8 + half * 4]);
                sc = mfma(aq, bk[s], sc);     // S[query, key]
                dp = mfma(ag, bv[s], dp);     // dP[query, key] = dout V^T
            }
            const bool full = qt * 32 + 32 <= S;
            float pr[16];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int qb = qt * 32 + 8 * j + 4 * half;          // four consecutive queries
                const float4_t L4 = *reinterpret_cast<const float4_t*>(&lse_l[qb]);
                const float4_t D4 = *reinterpret_cast<const float4_t*>(&dd_l[qb]);
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const int r = 4 * j + t;
                    pr[r] = fast_exp2(fmaf(sc[r], scale2, fmaf(cvt1(braw[r]), kLog2e, -L4[t])));
                    float ks = 1.0f;
                    if (DROP) ks = drop_keep(da, drop_row_hash(da, g * H + h, qb + t), ki) ? da.inv_keep : 0.f;
                    sc[r] = pr[r] * (dp[r] * ks - D4[t]);
                    if (DROP) pr[r] *= ks;
                }
            }
            if (!full) {                          // queries past the end of the batch entry (wave-uniform branch)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const bool in = qt * 32 + 8 * (r / 4) + 4 * half + (r % 4) < S;
                    pr[r] = in ? pr[r] : 0.f;
                    sc[r] = in ? sc[r] : 0.f;
                }
            }
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                short4_t db, pb;
                db = pack4(sc[4 * t + 0], sc[4 * t + 1], sc[4 * t + 2], sc[4 * t + 3]);
                pb = pack4(pr[4 * t + 0], pr[4 * t + 1], pr[4 * t + 2], pr[4 * t + 3]);
                short4_t aq = zero4(), ag = zero4();
                if (col < D) {
                    aq = *reinterpret_cast<const short4_t*>(&q_tr[col * (SP + 4) + qt * 32 + t * 8 + half * 4]);
                    ag = *reinterpret_cast<const short4_t*>(&g_tr[col * (SP + 4) + qt * 32 + t * 8 + half * 4]);
                }
                dk = mfma(aq, db, dk);        // dK^T[dd, key] += Q^T dS
                dv = mfma(ag, pb, dv);        // dV^T[dd, key] += dout^T P
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) braw[r] = braw_next[r];
        }
        if (thin) {
            constexpr int qt = NT - 1;
            float16_t sc = zero16(), dp = zero16();
#pragma unroll
            for (int s = 0; s < KS; ++s) {
                const short4_t aq = *reinterpret_cast<const short4_t*>(&q_rm[(qt * 32 + col) * D + s * 8 + half * 4]);
                const short4_t ag = *reinterpret_cast<const short4_t*>(&g_rm[(qt * 32 + col) * D + s * 8 + half * 4]);
                sc = mfma(aq, bk[s], sc);
                dp = mfma(ag, bv[s], dp);
            }
            // at most four queries in the last tile: registers 0..3 of the lower half
            const int qb = qt * 32 + 4 * half;
            const float4_t L4 = *reinterpret_cast<const float4_t*>(&lse_l[qb]);
            const float4_t D4 = *reinterpret_cast<const float4_t*>(&dd_l[qb]);
            float p4[4], s4[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const bool in = half == 0 && t < tail;
                const float pv = fast_exp2(fmaf(sc[t], scale2, fmaf(cvt1(braw[t]), kLog2e, -L4[t])));
                float ks = 1.0f;
                if (DROP) ks = drop_keep(da, drop_row_hash(da, g * H + h, qb + t), ki) ? da.inv_keep : 0.f;
                p4[t] = in ? pv * ks : 0.f;
                s4[t] = in ? pv * (dp[t] * ks - D4[t]) : 0.f;
            }
            short4_t db, pb;
            db = pack4(s4[0], s4[1], s4[2], s4[3]);
            pb = pack4(p4[0], p4[1], p4[2], p4[3]);
            short4_t aq = zero4(), ag = zero4();
            if (col < D) {
                aq = *reinterpret_cast<const short4_t*>(&q_tr[col * (SP + 4) + qt * 32 + half * 4]);
                ag = *reinterpret_cast<const short4_t*>(&g_tr[col * (SP + 4) + qt * 32 + half * 4]);
            }
            dk = mfma(aq, db, dk);
            dv = mfma(ag, pb, dv);
        }
        if (kok) {
            T* pk = dK + (((int64_t)g * S + ki) * H + h) * D;
            T* pv = dV + (((int64_t)g * S + ki) * H + h) * D;
#pragma unroll
            for (int rb = 0; rb < KS; ++rb) {
                st4(pk + 8 * rb + 4 * half, dk[4 * rb + 0] * scale, dk[4 * rb + 1] * scale, dk[4 * rb + 2] * scale,
                    dk[4 * rb + 3] * scale);
                st4(pv + 8 * rb + 4 * half, dv[4 * rb + 0], dv[4 * rb + 1], dv[4 * rb + 2], dv[4 * rb + 3]);
            }
        }
    }
    if constexpr (BSRC == 0) break;      // one pair per workgroup: no loop as far as the compiler is concerned
    __syncthreads();     // the LDS images and the bias tile are rewritten for the next pair
    if (acc.on) {
        // This pair's integer sums, converted with its scale, go into the workgroup's partial in global memory -
        // [ns] spatial, [ne] edge (with the mean's 1 / F), [1] virtual - and the accumulators start the next pair at
        // zero.  Only this workgroup touches its partial, one thread per entry.
        float* mine = ia.partial + (int64_t)blockIdx.x * (ia.ns + ia.ne + 1);
        const float unit = acc.scale > 0.f ? 1.f / acc.scale : 0.f, unit_e = (acc.scale_e > 0.f ? 1.f / acc.scale_e : 0.f) / (float)ia.F;
        for (int k = threadIdx.x; k <= ia.ns; k += blockDim.x) {
            int t = il.accS[k];
            il.accS[k] = 0;
            if (k < acc.hot_n)
                for (int c = 0; c < kHotCopies; ++c) { t += il.hot[c * kHotStride + k]; il.hot[c * kHotStride + k] = 0; }
            const int at = k < ia.ns ? k : ia.ns + ia.ne;           // slot ns of the spatial accumulators is the virtual distance's
            if (k != 0) mine[at] += (float)t * unit;                // slot 0: the padding index, no gradient
        }
        for (int k = threadIdx.x; k < ia.ne; k += blockDim.x) {
            const int t = il.accE[k];
            il.accE[k] = 0;
            mine[ia.ns + k] += (float)t * unit_e;
        }
        if (threadIdx.x == 0) { il.bound[0] = 0; il.bound[1] = 0; }
        __syncthreads();
    }
    }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
struct DenseCall {
    const void *q, *k, *v, *bias, *out, *dout;
    const float* lse;
    void *o_out, *dq, *dk, *dv, *dbias;
    float* o_lse;
    int b, S, H, d;
    hipStream_t st;
    float p_drop;          // 0: no dropout
    uint64_t seed;
    IdsArgs ids;           // BSRC = 1 only
};

static int device_cus() {
    static int cus = 0;
    if (cus == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess &&
            n > 0)
            cus = n;
        else
            cus = 256;
    }
    return cus;
}
// ---------------------------------------------------------------------------
// Backward in one walk (bias tensor or no bias).  The kernel above forms every score tile twice: once with a lane
// per query (dQ, dBias) and once with a lane per key (dK, dV).  Here wave w owns key tile w only and walks the query
// tiles once.  dS of a tile leaves the lane-per-key registers through a wave-private LDS tile [query][key] (bf16):
// read back with a lane per query it is the B operand of dQ^T += K^T dS^T and the 32-byte pieces of the dBias rows.
// A wave's dQ covers its own 32 keys; it goes to the wave's slab in LDS and the workgroup adds the slabs in wave
// order at the end (fixed order: reproducible).  Per tile that is 16 + 8 LDS accesses and four matrix instructions
// more, two matrix instructions, sixteen exponentials and the whole second pass over the bias less.
// ---------------------------------------------------------------------------
// The bias of one query tile as the lane-per-key walk needs it: 16 queries x this lane's key, one element each from 16
// rows.  2-byte elements sit two to a register, so that the elements of three tiles can be in flight (the walk is
// bound by the latency of these loads: 2 KB per wave and tile).
typedef unsigned short u16x2_t __attribute__((ext_vector_type(2)));
template <typename T> struct ColRegs;
template <> struct ColRegs<dbf16> {
    static constexpr int kDepth = 3;
    u16x2_t v[8];
    __device__ __forceinline__ void set(int r, const dbf16* p) { if (r & 1) v[r >> 1].y = p->x; else v[r >> 1].x = p->x; }
    __device__ __forceinline__ float get(int r) const { return __uint_as_float(((uint32_t)((r & 1) ? v[r >> 1].y : v[r >> 1].x)) << 16); }
};
template <> struct ColRegs<float> {
    static constexpr int kDepth = 2;
    float v[16];
    __device__ __forceinline__ void set(int r, const float* p) { v[r] = *p; }
    __device__ __forceinline__ float get(int r) const { return v[r]; }
};
// bias_gh: the [S, S] bias of this (graph, head), the same in all lanes; key: this lane's column.  Offsets are 32-bit
// byte offsets (S * S elements): the per-element part (8 (r / 4) + r % 4) S is the same in all lanes, so an element costs
// one add and one min next to a scalar base.  The min keeps rows past the end of a last, partial tile on the last
// row of the column (a valid address; their scores are masked): o_last is that row's offset.
template <typename T>
__device__ __forceinline__ void load_col(const T* __restrict__ bias_gh, int key, int qt, int half, int S, uint32_t o_last,
                                         ColRegs<T>& c) {
    const char* base = reinterpret_cast<const char*>(bias_gh);
    uint32_t o0 = (uint32_t)((qt * 32 + 4 * half) * S + key) * (uint32_t)sizeof(T);
    // (kept as one register: the compiler would otherwise carry the 16 element offsets through the tile loop, one
    // increment each per tile, in registers the loop does not have)
    asm volatile("" : "+v"(o0));
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const uint32_t o = min(o0 + (uint32_t)((8 * (r / 4) + (r % 4)) * S) * (uint32_t)sizeof(T), o_last);
        c.set(r, reinterpret_cast<const T*>(base + o));
    }
}
template <typename T>
__device__ __forceinline__ void zero_col(ColRegs<T>& c) {
    if constexpr (sizeof(T) == 2) {
#pragma unroll
        for (int i = 0; i < 8; ++i) { c.v[i].x = 0; c.v[i].y = 0; }
    } else {
#pragma unroll
        for (int i = 0; i < 16; ++i) c.v[i] = 0.f;
    }
}

constexpr int kTqPitch = 36;      // shorts per query row of the dS tile (8-byte reads two to a bank at worst)
// slab_rows: the queries whose dQ the waves share out (all of them, or those in front of a thin last tile)
template <int D, int NT> constexpr int bwd1_lds_bytes(int slab_rows = NT * 32) {
    return bwd_lds_bytes<D, NT>() + NT * 32 * kTqPitch * 2 + NT * slab_rows * D * 4;
}
// the one-walk kernel is used where two workgroups still fit a CU's LDS
template <int D, int NT> constexpr bool bwd1_fits() { return bwd1_lds_bytes<D, NT>() <= 72 * 1024; }

template <typename T, int D, int NT, bool DROP>
__global__ __launch_bounds__(64 * NT, D == 8 ? 4 : 3) void k_dense_bwd1(const T* __restrict__ Q, const T* __restrict__ K,
                                                        const T* __restrict__ V, const T* __restrict__ bias,
                                                        const T* __restrict__ O, const float* __restrict__ lse,
                                                        const T* __restrict__ dO, T* __restrict__ dQ,
                                                        T* __restrict__ dK, T* __restrict__ dV,
                                                        T* __restrict__ dbias, int S, int H, float scale, int nb,
                                                        const DropArgs da) {
    constexpr int KS = D / 8;
    constexpr int SP = NT * 32;
    extern __shared__ __align__(16) char smem[];
    constexpr int RM = rm_elems<D, SP>(), TR = tr_elems<D, SP>();
    short* q_rm = reinterpret_cast<short*>(smem);
    short* k_rm = q_rm + RM;
    short* v_rm = k_rm + RM;
    short* g_rm = v_rm + RM;          // g = dout
    short* q_tr = g_rm + RM;
    short* k_tr = q_tr + TR;
    short* g_tr = k_tr + TR;
    float* lse_l = reinterpret_cast<float*>(g_tr + TR);   // lse * log2(e)
    float* dd_l = lse_l + SP;
    short* tq_all = reinterpret_cast<short*>(dd_l + SP);  // [NT][32][kTqPitch]
    float* slab_all = reinterpret_cast<float*>(tq_all + NT * 32 * kTqPitch);   // [NT][slab_rows][D]
    const int pair = blockIdx.x;
    const int win = pair / (8 * H), rem = pair % (8 * H);
    const int g = win * 8 + (rem & 7), h = rem >> 3;
    if (g >= nb) return;
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int col = lane & 31, half = lane >> 5;
    const bool hasb = bias != nullptr;
    const int tail = S - (NT - 1) * 32;          // rows / keys in the last tile
    const bool thin = tail <= 4;
    const int nt_full = thin ? NT - 1 : NT;      // tiles that take the matrix path
    const T* bias_gh = hasb ? bias + ((int64_t)g * H + h) * S * S : nullptr;
    T* dbias_gh = dbias != nullptr ? dbias + ((int64_t)g * H + h) * S * S : nullptr;
    const bool vec_wave = thin && wave == NT - 1;
    short* tq = tq_all + wave * 32 * kTqPitch;
    const int slab_rows = thin ? (NT - 1) * 32 : SP;
    float* slab = slab_all + wave * slab_rows * D;
    // this lane's key and the first slice of its bias column, requested before anything else
    const int k0 = wave * 32, ki = k0 + col;
    const bool kok = ki < S;
    const int bkey = kok ? ki : 0;
    const uint32_t o_last = (uint32_t)((S - 1) * S + bkey) * (uint32_t)sizeof(T);
    constexpr int kDepth = ColRegs<T>::kDepth;       // tiles whose bias is in flight or in use
    ColRegs<T> b0, b1, b2;                            // of query tiles qt, qt + 1, qt + 2
    zero_col(b0); zero_col(b1); zero_col(b2);
    const bool bload = hasb && kok && !vec_wave;
    if (bload) {
        load_col(bias_gh, bkey, 0, half, S, o_last, b0);
        if (NT > 1) load_col(bias_gh, bkey, 1, half, S, o_last, b1);
    }
    load_head<T, D, SP>(Q, g, h, S, H, q_rm, q_tr);
    load_head<T, D, SP>(K, g, h, S, H, k_rm, k_tr);
    load_head<T, D, SP>(V, g, h, S, H, v_rm, nullptr);
    load_head<T, D, SP>(dO, g, h, S, H, g_rm, g_tr);
    for (int i = threadIdx.x; i < SP; i += blockDim.x) {
        float dsum = 0.f, L = 0.f;
        if (i < S) {
            L = lse[((int64_t)g * H + h) * S + i];
            const T* op = O + (((int64_t)g * S + i) * H + h) * D;
            const T* gp = dO + (((int64_t)g * S + i) * H + h) * D;
#pragma unroll
            for (int c = 0; c < D; c += 4) {
                const short4_t ov = ld4(op + c);
                const short4_t gv = ld4(gp + c);
                dsum += bf2f(ov.x) * bf2f(gv.x) + bf2f(ov.y) * bf2f(gv.y) + bf2f(ov.z) * bf2f(gv.z) +
                        bf2f(ov.w) * bf2f(gv.w);
            }
        }
        lse_l[i] = L * kLog2e;
        dd_l[i] = dsum;          // D[q] = sum_dd dout[q,dd] out[q,dd]
    }
    __syncthreads();

    if (vec_wave) {
        // the one to four rows of the last tile: as queries (dQ and dBias of those rows), then as keys (dK, dV, their
        // column of dBias and their share of everybody's dQ)
        thin_rows_bwd_q<T, T, D, SP, DROP>(q_rm, k_rm, v_rm, g_rm, lse_l, dd_l, bias_gh, S, dbias_gh, dQ, g, h, S, H, scale,
                                           (NT - 1) * 32, tail, lane, da, IdsAcc{});
        thin_rows_bwd_k<T, T, D, SP, DROP>(q_rm, k_rm, v_rm, g_rm, lse_l, dd_l, bias_gh, S, dK, dV, g, h, S, H, scale,
                                           (NT - 1) * 32, tail, lane, da, slab, dbias_gh);
    } else {
        short4_t bk[KS], bv[KS];
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            bk[s] = *reinterpret_cast<const short4_t*>(&k_rm[ki * D + s * 8 + half * 4]);
            bv[s] = *reinterpret_cast<const short4_t*>(&v_rm[ki * D + s * 8 + half * 4]);
        }
        const float scale2 = scale * kLog2e;
        float16_t dk = zero16(), dv = zero16();
#pragma unroll 1
        for (int qt = 0; qt < nt_full; ++qt) {
            if (bload) {      // the tile that will be needed kDepth - 1 tiles from now
                if (kDepth == 3 && qt + 2 < NT) load_col(bias_gh, bkey, qt + 2, half, S, o_last, b2);
                if (kDepth == 2 && qt + 1 < NT) load_col(bias_gh, bkey, qt + 1, half, S, o_last, b1);
            }
            float16_t sc = zero16(), dp = zero16();
#pragma unroll
            for (int s = 0; s < KS; ++s) {
                const short4_t aq = *reinterpret_cast<const short4_t*>(&q_rm[(qt * 32 + col) * D + s * 8 + half * 4]);
                const short4_t ag = *reinterpret_cast<const short4_t*>(&g_rm[(qt * 32 + col) * D + s * 8 + half * 4]);
                sc = mfma(aq, bk[s], sc);     // S[query, key]
                dp = mfma(ag, bv[s], dp);     // dP[query, key] = dout V^T
            }
            const bool full = qt * 32 + 32 <= S;
            float pr[16];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int qb = qt * 32 + 8 * j + 4 * half;          // four consecutive queries
                const float4_t L4 = *reinterpret_cast<const float4_t*>(&lse_l[qb]);
                const float4_t D4 = *reinterpret_cast<const float4_t*>(&dd_l[qb]);
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const int r = 4 * j + t;
                    pr[r] = fast_exp2(fmaf(sc[r], scale2, fmaf(b0.get(r), kLog2e, -L4[t])));
                    float ks = 1.0f;
                    if (DROP) ks = drop_keep(da, drop_row_hash(da, g * H + h, qb + t), ki) ? da.inv_keep : 0.f;
                    sc[r] = pr[r] * (dp[r] * ks - D4[t]);
                    if (DROP) pr[r] *= ks;
                }
            }
            if (!full || !kok) {                  // queries past the end of the batch entry (wave-uniform) or a key past it
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const bool in = kok && qt * 32 + 8 * (r / 4) + 4 * half + (r % 4) < S;
                    pr[r] = in ? pr[r] : 0.f;
                    sc[r] = in ? sc[r] : 0.f;
                }
            }
            // dS of the tile, rounded to bf16 once: into the wave's LDS tile [query][key] ...
            uint32_t dsp[8];          // pairs (r, r + 1), converted two at a time
#pragma unroll
            for (int r = 0; r < 16; r += 2) {
                dsp[r / 2] = cvt_pk(sc[r], sc[r + 1]);
                tq[(8 * (r / 4) + 4 * half + (r % 4)) * kTqPitch + col] = (short)(dsp[r / 2] & 0xffffu);
                tq[(8 * (r / 4) + 4 * half + (r % 4) + 1) * kTqPitch + col] = (short)(dsp[r / 2] >> 16);
            }
            // ... and, as it is, the B operand of dK^T += Q^T dS (P likewise for dV^T += dout^T P)
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                typedef uint32_t u2 __attribute__((ext_vector_type(2)));
                u2 dd2;
                dd2.x = dsp[2 * t]; dd2.y = dsp[2 * t + 1];
                const short4_t db = __builtin_bit_cast(short4_t, dd2);
                const short4_t pb = pack4(pr[4 * t + 0], pr[4 * t + 1], pr[4 * t + 2], pr[4 * t + 3]);
                short4_t aq = zero4(), ag = zero4();
                if (col < D) {
                    aq = *reinterpret_cast<const short4_t*>(&q_tr[col * (SP + 4) + qt * 32 + t * 8 + half * 4]);
                    ag = *reinterpret_cast<const short4_t*>(&g_tr[col * (SP + 4) + qt * 32 + t * 8 + half * 4]);
                }
                dk = mfma(aq, db, dk);        // dK^T[dd, key] += Q^T dS
                dv = mfma(ag, pb, dv);        // dV^T[dd, key] += dout^T P
            }
            // the tile read back with a lane per query: the writes are the wave's own and the LDS serves a wave's
            // accesses in the order they were issued, so only the compiler has to be kept from reordering them
            asm volatile("" ::: "memory");
            const int qi = qt * 32 + col;
            float16_t dq = zero16();
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const short4_t dsT = *reinterpret_cast<const short4_t*>(&tq[col * kTqPitch + 8 * t + 4 * half]);
                short4_t ak = zero4();
                if (col < D) ak = *reinterpret_cast<const short4_t*>(&k_tr[col * (SP + 4) + k0 + 8 * t + 4 * half]);
                dq = mfma(ak, dsT, dq);       // dQ^T[dd, query] += K^T dS^T over this wave's keys
            }
            if (dbias_gh != nullptr && qi < S) {          // 16 keys of the query's dBias row: 32 / 64 contiguous bytes
                const int kb = k0 + 16 * half;
                short4_t piece[4];
#pragma unroll
                for (int t = 0; t < 4; ++t) piece[t] = *reinterpret_cast<const short4_t*>(&tq[col * kTqPitch + 16 * half + 4 * t]);
                T* dbrow = dbias_gh + (int64_t)qi * S;
                if (kb + 16 <= S && sizeof(T) == 2) {
                    __builtin_memcpy(dbrow + kb, piece, 32);
                } else {
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        if (kb + 4 * t + 0 < S) st1(dbrow + kb + 4 * t + 0, bf2f(piece[t].x));
                        if (kb + 4 * t + 1 < S) st1(dbrow + kb + 4 * t + 1, bf2f(piece[t].y));
                        if (kb + 4 * t + 2 < S) st1(dbrow + kb + 4 * t + 2, bf2f(piece[t].z));
                        if (kb + 4 * t + 3 < S) st1(dbrow + kb + 4 * t + 3, bf2f(piece[t].w));
                    }
                }
            }
            // this wave's share of dQ of the 32 queries: rows dd = 8 rb + 4 half .. + 3 of the accumulator
#pragma unroll
            for (int rb = 0; rb < KS; ++rb) {
                float4_t o;
                o[0] = dq[4 * rb + 0]; o[1] = dq[4 * rb + 1]; o[2] = dq[4 * rb + 2]; o[3] = dq[4 * rb + 3];
                *reinterpret_cast<float4_t*>(&slab[qi * D + 8 * rb + 4 * half]) = o;
            }
            asm volatile("" ::: "memory");      // the tile is read before the next one is written (issue order)
            b0 = b1;
            if (kDepth == 3) b1 = b2;
        }
        if (thin) {
            constexpr int qt = NT - 1;
            float16_t sc = zero16(), dp = zero16();
#pragma unroll
            for (int s = 0; s < KS; ++s) {
                const short4_t aq = *reinterpret_cast<const short4_t*>(&q_rm[(qt * 32 + col) * D + s * 8 + half * 4]);
                const short4_t ag = *reinterpret_cast<const short4_t*>(&g_rm[(qt * 32 + col) * D + s * 8 + half * 4]);
                sc = mfma(aq, bk[s], sc);
                dp = mfma(ag, bv[s], dp);
            }
            // at most four queries in the last tile: registers 0..3 of the lower half; their dQ and dBias rows are
            // the vector wave's
            const int qb = qt * 32 + 4 * half;
            const float4_t L4 = *reinterpret_cast<const float4_t*>(&lse_l[qb]);
            const float4_t D4 = *reinterpret_cast<const float4_t*>(&dd_l[qb]);
            float p4[4], s4[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const bool in = half == 0 && t < tail;
                const float pv = fast_exp2(fmaf(sc[t], scale2, fmaf(b0.get(t), kLog2e, -L4[t])));
                float ks = 1.0f;
                if (DROP) ks = drop_keep(da, drop_row_hash(da, g * H + h, qb + t), ki) ? da.inv_keep : 0.f;
                p4[t] = in ? pv * ks : 0.f;
                s4[t] = in ? pv * (dp[t] * ks - D4[t]) : 0.f;
            }
            short4_t db, pb;
            db = pack4(s4[0], s4[1], s4[2], s4[3]);
            pb = pack4(p4[0], p4[1], p4[2], p4[3]);
            short4_t aq = zero4(), ag = zero4();
            if (col < D) {
                aq = *reinterpret_cast<const short4_t*>(&q_tr[col * (SP + 4) + qt * 32 + half * 4]);
                ag = *reinterpret_cast<const short4_t*>(&g_tr[col * (SP + 4) + qt * 32 + half * 4]);
            }
            dk = mfma(aq, db, dk);
            dv = mfma(ag, pb, dv);
        }
        if (kok) {
            T* pk = dK + (((int64_t)g * S + ki) * H + h) * D;
            T* pv = dV + (((int64_t)g * S + ki) * H + h) * D;
#pragma unroll
            for (int rb = 0; rb < KS; ++rb) {
                st4(pk + 8 * rb + 4 * half, dk[4 * rb + 0] * scale, dk[4 * rb + 1] * scale, dk[4 * rb + 2] * scale,
                    dk[4 * rb + 3] * scale);
                st4(pv + 8 * rb + 4 * half, dv[4 * rb + 0], dv[4 * rb + 1], dv[4 * rb + 2], dv[4 * rb + 3]);
            }
        }
    }
    __syncthreads();
    // dQ = scale * (the waves' shares, in wave order); the rows of a thin last tile were written by their wave
    const int q_end = thin ? (NT - 1) * 32 : S;
    for (int c = threadIdx.x; c < q_end * (D / 4); c += blockDim.x) {
        const int row = c / (D / 4), part = c % (D / 4);
        float4_t a = *reinterpret_cast<const float4_t*>(&slab_all[row * D + part * 4]);
#pragma unroll
        for (int w = 1; w < NT; ++w) {
            const float4_t b = *reinterpret_cast<const float4_t*>(&slab_all[(w * slab_rows + row) * D + part * 4]);
            a[0] += b[0]; a[1] += b[1]; a[2] += b[2]; a[3] += b[3];
        }
        st4(dQ + (((int64_t)g * S + row) * H + h) * D + part * 4, a[0] * scale, a[1] * scale, a[2] * scale, a[3] * scale);
    }
}

// Workgroups of the id form's backward: what the GPU keeps resident at two per CU, a multiple of 8 H so that a
// workgroup stays with one head, at most one per pair.  It also sizes the workspace of table partials.
static int ids_bwd_grid(int b, int H) {
    const int unit = 8 * H, total_pairs = ((b + 7) / 8) * unit;
    return std::min(total_pairs, std::max(unit, 2 * device_cus() / unit * unit));
}

template <typename T, int D, int NT, int BSRC>
static int launch_dense(const DenseCall& c, bool bwd) {
    constexpr int lds_f0 = fwd_lds_bytes<D, NT>(), lds_b0 = bwd_lds_bytes<D, NT>();
    if constexpr (lds_f0 > kLdsLimit || lds_b0 > kLdsLimit) {
        set_error("dense attention: S=%d with head dim %d needs %d bytes of LDS (limit %d)", c.S, c.d,
                  lds_b0 > lds_f0 ? lds_b0 : lds_f0, kLdsLimit);
        return TGT_ERR_UNSUPPORTED;
    } else {
        const size_t lds_f = lds_f0 + (BSRC == 1 ? ids_lds_bytes(c.S, c.ids.ns, c.ids.ne, false) : 0);
        const size_t lds_b = lds_b0 + (BSRC == 1 ? ids_lds_bytes(c.S, c.ids.ns, c.ids.ne, true) : 0);
        // the forward refuses what its backward could not run: a training step must not pass the forward and fail
        // inside autograd
        if (std::max(lds_f, lds_b) > (size_t)kLdsLimit) {
            set_error("dense attention from ids: S=%d with tables of %d + %d rows needs %zu bytes of LDS (limit %d); "
                      "build the bias tensor instead", c.S, c.ids.ns, c.ids.ne, std::max(lds_f, lds_b), kLdsLimit);
            return TGT_ERR_UNSUPPORTED;
        }
        const float scale = sqrtf((float)c.d);     // the reference MULTIPLIES q by sqrt(d)
        const dim3 block(64 * NT);
        const bool thin = c.S - (NT - 1) * 32 <= 4;      // a last tile of at most four rows
        static bool attr_done = false;     // raise the dynamic-LDS cap once per instantiation
        if (!attr_done) {
            const int cap_f = BSRC == 1 ? kLdsLimit : lds_f0, cap_b = BSRC == 1 ? kLdsLimit : lds_b0;
            if (cap_f > 48 * 1024) {
                TGT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&k_dense_fwd<T, D, NT, false, BSRC>),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, cap_f));
                TGT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&k_dense_fwd<T, D, NT, true, BSRC>),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, cap_f));
            }
            if (cap_b > 48 * 1024) {
                TGT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&k_dense_bwd<T, D, NT, false, BSRC>),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, cap_b));
                TGT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&k_dense_bwd<T, D, NT, true, BSRC>),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, cap_b));
            }
            attr_done = true;
        }
        const int unit = 8 * c.H, total_pairs = ((c.b + 7) / 8) * unit;
        // Forward: a persistent grid of about three workgroups per CU (measured best; more resident
        // workgroups only add cache pressure), a multiple of 8 (one share per XCD; of 8 H with ids: one
        // head per workgroup).  Backward with the bias in memory: one workgroup per pair.
        int fwd_grid = std::max(8, (3 * device_cus()) & ~7);
        if (BSRC == 1) fwd_grid = std::max(unit, fwd_grid / unit * unit);
        const int nblk = bwd ? (BSRC == 1 ? ids_bwd_grid(c.b, c.H) : total_pairs) : std::min(total_pairs, fwd_grid);
        const dim3 grid((unsigned)nblk);
        const bool drop = c.p_drop > 0.f;
        const DropArgs da = drop_args(c.p_drop, c.seed);
        if (!bwd) {
            KernelTimer t(KS_DENSE_FWD, c.st);
            if (drop)
                hipLaunchKernelGGL((k_dense_fwd<T, D, NT, true, BSRC>), grid, block, lds_f, c.st, (const T*)c.q, (const T*)c.k,
                                   (const T*)c.v, (const T*)c.bias, (T*)c.o_out, c.o_lse, c.S, c.H, scale, c.b, da, c.ids);
            else
                hipLaunchKernelGGL((k_dense_fwd<T, D, NT, false, BSRC>), grid, block, lds_f, c.st, (const T*)c.q, (const T*)c.k,
                                   (const T*)c.v, (const T*)c.bias, (T*)c.o_out, c.o_lse, c.S, c.H, scale, c.b, da, c.ids);
        } else if constexpr (BSRC == 0 && bwd1_fits<D, NT>()) {
            // bias tensor (or none) and a shape whose dQ shares fit the LDS: every score tile is formed once
            constexpr int lds1_max = bwd1_lds_bytes<D, NT>();
            const int lds1 = bwd1_lds_bytes<D, NT>(thin ? (NT - 1) * 32 : NT * 32);
            static bool attr1_done = false;
            if (!attr1_done) {
                TGT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&k_dense_bwd1<T, D, NT, false>),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, lds1_max));
                TGT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&k_dense_bwd1<T, D, NT, true>),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, lds1_max));
                attr1_done = true;
            }
            KernelTimer t(KS_DENSE_BWD, c.st);
            if (drop)
                hipLaunchKernelGGL((k_dense_bwd1<T, D, NT, true>), grid, block, lds1, c.st, (const T*)c.q, (const T*)c.k,
                                   (const T*)c.v, (const T*)c.bias, (const T*)c.out, c.lse, (const T*)c.dout,
                                   (T*)c.dq, (T*)c.dk, (T*)c.dv, (T*)c.dbias, c.S, c.H, scale, c.b, da);
            else
                hipLaunchKernelGGL((k_dense_bwd1<T, D, NT, false>), grid, block, lds1, c.st, (const T*)c.q, (const T*)c.k,
                                   (const T*)c.v, (const T*)c.bias, (const T*)c.out, c.lse, (const T*)c.dout,
                                   (T*)c.dq, (T*)c.dk, (T*)c.dv, (T*)c.dbias, c.S, c.H, scale, c.b, da);
        } else {
            KernelTimer t(KS_DENSE_BWD, c.st);
            if (drop)
                hipLaunchKernelGGL((k_dense_bwd<T, D, NT, true, BSRC>), grid, block, lds_b, c.st, (const T*)c.q, (const T*)c.k,
                                   (const T*)c.v, (const T*)c.bias, (const T*)c.out, c.lse, (const T*)c.dout,
                                   (T*)c.dq, (T*)c.dk, (T*)c.dv, (T*)c.dbias, c.S, c.H, scale, c.b, da, c.ids);
            else
                hipLaunchKernelGGL((k_dense_bwd<T, D, NT, false, BSRC>), grid, block, lds_b, c.st, (const T*)c.q, (const T*)c.k,
                                   (const T*)c.v, (const T*)c.bias, (const T*)c.out, c.lse, (const T*)c.dout,
                                   (T*)c.dq, (T*)c.dk, (T*)c.dv, (T*)c.dbias, c.S, c.H, scale, c.b, da, c.ids);
        }
        TGT_HIP_CHECK(hipGetLastError());
        return TGT_OK;
    }
}

template <typename T, int D, int BSRC>
static int dispatch_nt(const DenseCall& c, bool bwd) {
    switch ((c.S + 31) / 32) {
        case 1: return launch_dense<T, D, 1, BSRC>(c, bwd);
        case 2: return launch_dense<T, D, 2, BSRC>(c, bwd);
        case 3: return launch_dense<T, D, 3, BSRC>(c, bwd);
        case 4: return launch_dense<T, D, 4, BSRC>(c, bwd);
        case 5: return launch_dense<T, D, 5, BSRC>(c, bwd);
        case 6: return launch_dense<T, D, 6, BSRC>(c, bwd);
        case 7: return launch_dense<T, D, 7, BSRC>(c, bwd);
        case 8: return launch_dense<T, D, 8, BSRC>(c, bwd);
        default:
            set_error("dense attention: sequence length %d exceeds 256", c.S);
            return TGT_ERR_UNSUPPORTED;
    }
}

template <typename T, int BSRC>
static int dispatch_d(const DenseCall& c, bool bwd) {
    switch (c.d) {
        case 8: return dispatch_nt<T, 8, BSRC>(c, bwd);
        case 16: return dispatch_nt<T, 16, BSRC>(c, bwd);
        case 32: return dispatch_nt<T, 32, BSRC>(c, bwd);
        default:
            set_error("dense attention: head dim %d not in {8, 16, 32}", c.d);
            return TGT_ERR_UNSUPPORTED;
    }
}

#ifndef TGT_DENSE_PART
#error "compile with -DTGT_DENSE_PART=0 (bias tensor entry points) or 1 (id + table entry points)"
#endif

#if TGT_DENSE_PART == 0
// keep[g, h, q, k] (1 = kept) of the dropout the attention kernels apply for (p, seed)
__global__ void k_dropout_mask(uint8_t* __restrict__ out, int S, int H, int64_t total, const DropArgs da) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int k = (int)(i % S);
    const int64_t r = i / S;
    const int q = (int)(r % S);
    const int pair = (int)(r / S);
    out[i] = drop_keep(da, drop_row_hash(da, pair, q), k) ? 1 : 0;
}

#endif

static int check_dense(const void* q, const void* k, const void* v, int b, int S, int H, int d, int dtype) {
    if (!q || !k || !v) { set_error("dense attention: null q/k/v"); return TGT_ERR_INVALID_ARG; }
    if (b < 1 || S < 1 || H < 1 || d < 1) { set_error("dense attention: non-positive size"); return TGT_ERR_INVALID_ARG; }
    if (dtype != TGT_DTYPE_F32 && dtype != TGT_DTYPE_BF16 && dtype != TGT_DTYPE_F32_BF16_PRODUCTS) {
        set_error("bad dtype %d", dtype);
        return TGT_ERR_INVALID_ARG;
    }
    if (S > 256 && dtype != TGT_DTYPE_F32) { set_error("dense attention: sequence length %d exceeds 256", S); return TGT_ERR_UNSUPPORTED; }
    if ((int64_t)b * H > 0x7fffffffLL) { set_error("dense attention: b*H too large"); return TGT_ERR_INVALID_ARG; }
    return TGT_OK;
}

}  // namespace tgt

#if TGT_DENSE_PART == 0
extern "C" {

int tgt_dense_attn_dropout_fwd(const void* d_q, const void* d_k, const void* d_v, const void* d_bias, int b, int S,
                               int H, int d, int dtype, float p_drop, uint64_t seed, void* d_out, float* d_lse,
                               void* stream) {
    int rc = tgt::check_dense(d_q, d_k, d_v, b, S, H, d, dtype);
    if (rc) return rc;
    if (!d_out || !d_lse) { tgt::set_error("dense attention: null out or lse"); return TGT_ERR_INVALID_ARG; }
    if (!(p_drop >= 0.f && p_drop < 1.f)) { tgt::set_error("dense attention: dropout rate %g outside [0, 1)", p_drop); return TGT_ERR_INVALID_ARG; }
    tgt::DenseCall c{};
    c.q = d_q; c.k = d_k; c.v = d_v; c.bias = d_bias; c.o_out = d_out; c.o_lse = d_lse;
    c.b = b; c.S = S; c.H = H; c.d = d; c.st = (hipStream_t)stream;
    c.p_drop = p_drop; c.seed = seed;
    if (dtype == TGT_DTYPE_F32) {
        tgt::DenseF32Call f{};
        f.q = (const float*)d_q; f.k = (const float*)d_k; f.v = (const float*)d_v; f.bias = (const float*)d_bias;
        f.o_out = (float*)d_out; f.o_lse = d_lse; f.b = b; f.S = S; f.H = H; f.d = d; f.st = c.st;
        f.p_drop = p_drop; f.seed = seed;
        return tgt::dense_attn_f32(f, false);
    }
    return dtype == TGT_DTYPE_F32_BF16_PRODUCTS ? tgt::dispatch_d<float, 0>(c, false) : tgt::dispatch_d<tgt::dbf16, 0>(c, false);
}

int tgt_dense_attn_fwd(const void* d_q, const void* d_k, const void* d_v, const void* d_bias, int b, int S, int H,
                       int d, int dtype, void* d_out, float* d_lse, void* stream) {
    return tgt_dense_attn_dropout_fwd(d_q, d_k, d_v, d_bias, b, S, H, d, dtype, 0.f, 0, d_out, d_lse, stream);
}

int tgt_dense_attn_dropout_mask(int b, int S, int H, float p_drop, uint64_t seed, uint8_t* d_keep, void* stream) {
    if (b < 1 || S < 1 || H < 1 || !d_keep || !(p_drop >= 0.f && p_drop < 1.f)) {
        tgt::set_error("tgt_dense_attn_dropout_mask: bad size, null pointer or rate outside [0, 1)");
        return TGT_ERR_INVALID_ARG;
    }
    const int64_t total = (int64_t)b * H * S * S;
    hipLaunchKernelGGL(tgt::k_dropout_mask, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream, d_keep,
                       S, H, total, tgt::drop_args(p_drop, seed));
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

int tgt_dense_attn_bwd(const void* d_q, const void* d_k, const void* d_v, const void* d_bias, int b, int S, int H,
                       int d, int dtype, const void* d_out, const float* d_lse, const void* d_dout, void* d_dq,
                       void* d_dk, void* d_dv, void* d_dbias, void* stream) {
    return tgt_dense_attn_dropout_bwd(d_q, d_k, d_v, d_bias, b, S, H, d, dtype, 0.f, 0, d_out, d_lse, d_dout, d_dq, d_dk,
                                      d_dv, d_dbias, stream);
}

int tgt_dense_attn_dropout_bwd(const void* d_q, const void* d_k, const void* d_v, const void* d_bias, int b, int S,
                               int H, int d, int dtype, float p_drop, uint64_t seed, const void* d_out,
                               const float* d_lse, const void* d_dout, void* d_dq, void* d_dk, void* d_dv,
                               void* d_dbias, void* stream) {
    int rc = tgt::check_dense(d_q, d_k, d_v, b, S, H, d, dtype);
    if (rc) return rc;
    if (!(p_drop >= 0.f && p_drop < 1.f)) { tgt::set_error("dense attention: dropout rate %g outside [0, 1)", p_drop); return TGT_ERR_INVALID_ARG; }
    if (!d_out || !d_lse || !d_dout || !d_dq || !d_dk || !d_dv) {
        tgt::set_error("dense attention backward: null out/lse/dout/dq/dk/dv");
        return TGT_ERR_INVALID_ARG;
    }
    tgt::DenseCall c{};
    c.q = d_q; c.k = d_k; c.v = d_v; c.bias = d_bias; c.out = d_out; c.lse = d_lse; c.dout = d_dout;
    c.dq = d_dq; c.dk = d_dk; c.dv = d_dv; c.dbias = d_dbias;
    c.b = b; c.S = S; c.H = H; c.d = d; c.st = (hipStream_t)stream;
    c.p_drop = p_drop; c.seed = seed;
    if (dtype == TGT_DTYPE_F32) {
        tgt::DenseF32Call f{};
        f.q = (const float*)d_q; f.k = (const float*)d_k; f.v = (const float*)d_v; f.bias = (const float*)d_bias;
        f.out = (const float*)d_out; f.lse = d_lse; f.dout = (const float*)d_dout;
        f.dq = (float*)d_dq; f.dk = (float*)d_dk; f.dv = (float*)d_dv; f.dbias = (float*)d_dbias;
        f.b = b; f.S = S; f.H = H; f.d = d; f.st = c.st; f.p_drop = p_drop; f.seed = seed;
        return tgt::dense_attn_f32(f, true);
    }
    return dtype == TGT_DTYPE_F32_BF16_PRODUCTS ? tgt::dispatch_d<float, 0>(c, true) : tgt::dispatch_d<tgt::dbf16, 0>(c, true);
}

}  // extern "C"
#endif

#if TGT_DENSE_PART == 1
// ---------------------------------------------------------------------------
// The id + table form: entry points
// ---------------------------------------------------------------------------
namespace tgt {

__device__ __forceinline__ uint16_t pack_id(int64_t v, int n) { return (uint16_t)(v < 0 ? 0 : (v >= n ? n - 1 : v)); }

// one thread per position of the padded [S1, S1] index space
__global__ __launch_bounds__(256) void k_ids_pack(const int64_t* __restrict__ spatial_pos, const int64_t* __restrict__ edge_type,
                                                  int b, int s, int F, int ns, int ne, uint16_t* __restrict__ sp16,
                                                  uint16_t* __restrict__ et16) {
    const int S1 = s + 1;
    const int64_t total = (int64_t)b * S1 * S1;
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= total) return;
    const int j = (int)(t % S1), i = (int)((t / S1) % S1);
    const int64_t g = t / ((int64_t)S1 * S1);
    if (i >= 1 && j >= 1) {
        const int64_t pos = (g * s + (i - 1)) * s + (j - 1);
        sp16[t] = pack_id(spatial_pos[pos], ns);
        for (int f = 0; f < F; ++f) et16[t * F + f] = pack_id(edge_type[pos * F + f], ne);
    } else {
        sp16[t] = (uint16_t)ns;                       // the virtual distance's slot
        for (int f = 0; f < F; ++f) et16[t * F + f] = (uint16_t)ne;     // a slot that holds 0
    }
}

// Table gradients from the workgroup partials: thread (h, k) adds the partials of the workgroups of head h
// (ids 8 h .. 8 h + 7 in every window of 8 H) in workgroup order.
template <typename T>
__global__ __launch_bounds__(256) void k_ids_reduce(const float* __restrict__ partial, int grid, int H, int ns, int ne,
                                                    T* __restrict__ d_sp, T* __restrict__ d_e, T* __restrict__ d_v) {
    const int n_acc = ns + ne + 1;
    const int idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= n_acc * H) return;
    const int h = idx / n_acc, k = idx - h * n_acc;
    float t = 0.f;
    for (int w0 = 8 * h; w0 < grid; w0 += 8 * H)
        for (int x = 0; x < 8; ++x) t += partial[(int64_t)(w0 + x) * n_acc + k];
    if (k < ns) st1(d_sp + (int64_t)k * H + h, t);
    else if (k < ns + ne) st1(d_e + (int64_t)(k - ns) * H + h, t);
    else st1(d_v + h, t);
}

static int check_ids(const void* sp16, const void* et16, int F, const void* sp_tab, int ns, const void* e_tab, int ne,
                     const void* vd, int H, int dtype) {
    if (!sp16 || !et16 || !sp_tab || !e_tab || !vd) { set_error("dense attention from ids: null ids or tables"); return TGT_ERR_INVALID_ARG; }
    if (F < 1 || ns < 1 || ne < 1 || ns > 65534 || ne > 65534) {
        set_error("dense attention from ids: F >= 1 and table sizes in 1..65534 needed (F=%d, %d, %d)", F, ns, ne);
        return TGT_ERR_INVALID_ARG;
    }
    if (dtype == TGT_DTYPE_F32) {
        set_error("dense attention from ids: the float32-arithmetic kernels read a bias tensor; build it with "
                  "tgt_graph_attn_bias_fwd, or pass TGT_DTYPE_F32_BF16_PRODUCTS");
        return TGT_ERR_UNSUPPORTED;
    }
    if (H > 32) { set_error("dense attention from ids: at most 32 heads"); return TGT_ERR_UNSUPPORTED; }
    return TGT_OK;
}

}  // namespace tgt

extern "C" {

int tgt_dense_ids_pack(const int64_t* d_spatial_pos, const int64_t* d_edge_type, int b, int s, int F, int num_spatial,
                       int num_edges, uint16_t* d_sp16, uint16_t* d_et16, void* stream) {
    using namespace tgt;
    if (b < 1 || s < 0 || F < 1 || num_spatial < 1 || num_edges < 1 || num_spatial > 65534 || num_edges > 65534 || !d_sp16 ||
        !d_et16 || (s > 0 && (!d_spatial_pos || !d_edge_type))) {
        set_error("tgt_dense_ids_pack: bad size (table sizes must be 1..65534) or null pointer");
        return TGT_ERR_INVALID_ARG;
    }
    const int64_t total = (int64_t)b * (s + 1) * (s + 1);
    hipLaunchKernelGGL(k_ids_pack, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream, d_spatial_pos,
                       d_edge_type, b, s, F, num_spatial, num_edges, d_sp16, d_et16);
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

int tgt_dense_attn_ids_fwd(const void* d_q, const void* d_k, const void* d_v, const void* d_attn_bias,
                           const uint16_t* d_sp16, const uint16_t* d_et16, int F, const void* d_spatial_table, int num_spatial,
                           const void* d_edge_table, int num_edges, const void* d_virtual_dist, int b, int S, int H, int d,
                           int dtype, float p_drop, uint64_t seed, void* d_out, float* d_lse, void* stream) {
    using namespace tgt;
    int rc = check_dense(d_q, d_k, d_v, b, S, H, d, dtype);
    if (rc) return rc;
    rc = check_ids(d_sp16, d_et16, F, d_spatial_table, num_spatial, d_edge_table, num_edges, d_virtual_dist, H, dtype);
    if (rc) return rc;
    if (!d_out || !d_lse) { set_error("dense attention: null out or lse"); return TGT_ERR_INVALID_ARG; }
    if (!(p_drop >= 0.f && p_drop < 1.f)) { set_error("dense attention: dropout rate %g outside [0, 1)", p_drop); return TGT_ERR_INVALID_ARG; }
    DenseCall c{};
    c.q = d_q; c.k = d_k; c.v = d_v; c.o_out = d_out; c.o_lse = d_lse;
    c.b = b; c.S = S; c.H = H; c.d = d; c.st = (hipStream_t)stream;
    c.p_drop = p_drop; c.seed = seed;
    c.ids = IdsArgs{d_attn_bias, d_sp16, d_et16, d_spatial_table, d_edge_table, d_virtual_dist, nullptr, F, num_spatial, num_edges};
    return dtype == TGT_DTYPE_F32_BF16_PRODUCTS ? dispatch_d<float, 1>(c, false) : dispatch_d<dbf16, 1>(c, false);
}

int64_t tgt_dense_attn_ids_bwd_workspace_bytes(int b, int H, int num_spatial, int num_edges) {
    using namespace tgt;
    if (b < 1 || H < 1 || num_spatial < 1 || num_edges < 1) return 0;
    return (int64_t)sizeof(float) * ids_bwd_grid(b, H) * (num_spatial + num_edges + 1);
}

int tgt_dense_attn_ids_bwd(const void* d_q, const void* d_k, const void* d_v, const void* d_attn_bias,
                           const uint16_t* d_sp16, const uint16_t* d_et16, int F, const void* d_spatial_table, int num_spatial,
                           const void* d_edge_table, int num_edges, const void* d_virtual_dist, int b, int S, int H, int d,
                           int dtype, float p_drop, uint64_t seed, const void* d_out, const float* d_lse, const void* d_dout,
                           void* d_dq, void* d_dk, void* d_dv, void* d_dspatial_table, void* d_dedge_table,
                           void* d_dvirtual_dist, void* d_workspace, int64_t workspace_bytes, void* stream) {
    using namespace tgt;
    int rc = check_dense(d_q, d_k, d_v, b, S, H, d, dtype);
    if (rc) return rc;
    rc = check_ids(d_sp16, d_et16, F, d_spatial_table, num_spatial, d_edge_table, num_edges, d_virtual_dist, H, dtype);
    if (rc) return rc;
    if (!(p_drop >= 0.f && p_drop < 1.f)) { set_error("dense attention: dropout rate %g outside [0, 1)", p_drop); return TGT_ERR_INVALID_ARG; }
    if (!d_out || !d_lse || !d_dout || !d_dq || !d_dk || !d_dv) {
        set_error("dense attention backward: null out/lse/dout/dq/dk/dv");
        return TGT_ERR_INVALID_ARG;
    }
    const bool tables = d_dspatial_table || d_dedge_table || d_dvirtual_dist;
    if (tables && !(d_dspatial_table && d_dedge_table && d_dvirtual_dist)) {
        set_error("dense attention from ids, backward: the three table gradients come together (all or none)");
        return TGT_ERR_INVALID_ARG;
    }
    if (tables && (!d_workspace || ((uintptr_t)d_workspace & 15) ||
                   workspace_bytes < tgt_dense_attn_ids_bwd_workspace_bytes(b, H, num_spatial, num_edges))) {
        set_error("dense attention from ids, backward: workspace of %lld bytes (16-byte aligned) needed, got %lld",
                  (long long)tgt_dense_attn_ids_bwd_workspace_bytes(b, H, num_spatial, num_edges), (long long)workspace_bytes);
        return TGT_ERR_WORKSPACE;
    }
    DenseCall c{};
    c.q = d_q; c.k = d_k; c.v = d_v; c.out = d_out; c.lse = d_lse; c.dout = d_dout;
    c.dq = d_dq; c.dk = d_dk; c.dv = d_dv;
    c.b = b; c.S = S; c.H = H; c.d = d; c.st = (hipStream_t)stream;
    c.p_drop = p_drop; c.seed = seed;
    c.ids = IdsArgs{d_attn_bias, d_sp16, d_et16, d_spatial_table, d_edge_table, d_virtual_dist,
                    tables ? (float*)d_workspace : nullptr, F, num_spatial, num_edges};
    rc = dtype == TGT_DTYPE_F32_BF16_PRODUCTS ? dispatch_d<float, 1>(c, true) : dispatch_d<dbf16, 1>(c, true);
    if (rc != TGT_OK || !tables) return rc;
    const int grid = ids_bwd_grid(b, H), n = (num_spatial + num_edges + 1) * H;
    if (dtype == TGT_DTYPE_F32_BF16_PRODUCTS)
        hipLaunchKernelGGL((k_ids_reduce<float>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, c.st, (const float*)d_workspace,
                           grid, H, num_spatial, num_edges, (float*)d_dspatial_table, (float*)d_dedge_table, (float*)d_dvirtual_dist);
    else
        hipLaunchKernelGGL((k_ids_reduce<dbf16>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, c.st, (const float*)d_workspace,
                           grid, H, num_spatial, num_edges, (dbf16*)d_dspatial_table, (dbf16*)d_dedge_table, (dbf16*)d_dvirtual_dist);
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

}  // extern "C"
#endif
