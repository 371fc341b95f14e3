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

// four consecutive elements as bf16 bits
__device__ __forceinline__ short4_t ld4(const dbf16* p) {
    return *reinterpret_cast<const short4_t*>(p);
}
__device__ __forceinline__ short4_t ld4(const float* p) {
    const float4_t f = *reinterpret_cast<const float4_t*>(p);
    short4_t r;
    r.x = f2bf(f.x); r.y = f2bf(f.y); r.z = f2bf(f.z); r.w = f2bf(f.w);
    return r;
}
__device__ __forceinline__ void st4(dbf16* p, float a, float b, float c, float d) {
    short4_t r;
    r.x = f2bf(a); r.y = f2bf(b); r.z = f2bf(c); r.w = f2bf(d);
    *reinterpret_cast<short4_t*>(p) = r;
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
template <typename T, int D, int SP, bool DROP>
__device__ __forceinline__ void thin_rows_fwd(const T* __restrict__ Q, const short* __restrict__ k_rm,
                                              const short* __restrict__ v_tr, const T* __restrict__ bias_gh,
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
        const T* brow = bias_gh ? bias_gh + (int64_t)qi * S : nullptr;
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
template <typename T, int D, int SP, bool DROP>
__device__ __forceinline__ void thin_rows_bwd_q(const short* __restrict__ q_rm, const short* __restrict__ k_rm,
                                                const short* __restrict__ v_rm, const short* __restrict__ g_rm,
                                                const float* __restrict__ lse_l, const float* __restrict__ dd_l,
                                                const T* __restrict__ bias_gh, T* __restrict__ dbias_gh, T* __restrict__ dQ,
                                                int g, int h, int S, int H, float scale, int first, int count, int lane,
                                                const DropArgs da) {
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
                const float b = bias_gh ? ld1(bias_gh + (int64_t)qi * S + key) : 0.f;
                const float pv = fast_exp2(fmaf(dot_d<D>(qv, kv), scale2, fmaf(b, kLog2e, nL2)));
                const float ks = !DROP ? 1.0f : (drop_keep(da, rh, key) ? da.inv_keep : 0.f);
                const float dS = pv * (dot_d<D>(gv, vv) * ks - Dq);
                if (dbias_gh) st1(dbias_gh + (int64_t)qi * S + key, dS);
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
template <typename T, int D, int SP, bool DROP>
__device__ __forceinline__ void thin_rows_bwd_k(const short* __restrict__ q_rm, const short* __restrict__ k_rm,
                                                const short* __restrict__ v_rm, const short* __restrict__ g_rm,
                                                const float* __restrict__ lse_l, const float* __restrict__ dd_l,
                                                const T* __restrict__ bias_gh, T* __restrict__ dK, T* __restrict__ dV,
                                                int g, int h, int S, int H, float scale, int first, int count, int lane,
                                                const DropArgs da) {
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
                const float b = bias_gh ? ld1(bias_gh + (int64_t)qq * S + ki) : 0.f;
                const float pv = fast_exp2(fmaf(dot_d<D>(qv, kv), scale2, fmaf(b, kLog2e, -lse_l[qq])));
                const float ks = !DROP ? 1.0f : (drop_keep(da, drop_row_hash(da, g * H + h, qq), ki) ? da.inv_keep : 0.f);
                const float dS = pv * (dot_d<D>(gv, vv) * ks - dd_l[qq]);
                const float pb = round_bf(pv * ks), dsb = round_bf(dS);
#pragma unroll
                for (int d = 0; d < D; ++d) {
                    dk[d] = fmaf(dsb, qv[d], dk[d]);
                    dv[d] = fmaf(pb, gv[d], dv[d]);
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
template <typename T, int D, int NT, bool DROP>
__global__ __launch_bounds__(64 * NT) void k_dense_fwd(const T* __restrict__ Q, const T* __restrict__ K,
                                                       const T* __restrict__ V, const T* __restrict__ bias,
                                                       T* __restrict__ out, float* __restrict__ lse, int S,
                                                       int H, float scale, int nb, const DropArgs da) {
    constexpr int KS = D / 8;
    constexpr int SP = NT * 32;
    extern __shared__ __align__(16) char smem[];
    short* k_rm = reinterpret_cast<short*>(smem);
    short* v_tr = k_rm + rm_elems<D, SP>();
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
    const bool hasb = bias != nullptr;
    // a last tile of at most four rows is not worth a matrix tile: its wave takes the vector path
    const bool vec_wave = wave == NT - 1 && S - (NT - 1) * 32 <= 4;
    // this lane's query row of the bias; the first tile's group of it is requested before anything else
    const T* brow = hasb ? bias + (((int64_t)g * H + h) * S + (qok ? qi : 0)) * S : nullptr;
    Bias16<T> bcur, bnext;
    zero_bias16(bcur);
    zero_bias16(bnext);
    if (hasb && qok && !vec_wave) load_bias16(brow + 16 * half, min(16, S - 16 * half), bcur);
    load_head<T, D, SP>(K, g, h, S, H, k_rm, nullptr);
    load_head<T, D, SP>(V, g, h, S, H, nullptr, v_tr);
    short4_t bq[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        bq[s] = zero4();
        if (qok) bq[s] = ld4(Q + (((int64_t)g * S + qi) * H + h) * D + s * 8 + half * 4);
    }
    __syncthreads();
    if (vec_wave) {
        thin_rows_fwd<T, D, SP, DROP>(Q, k_rm, v_tr, hasb ? bias + ((int64_t)g * H + h) * S * S : nullptr, out, lse, g, h, S,
                                      H, scale, (NT - 1) * 32, S - (NT - 1) * 32, lane, da);
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
            if (nv > 0) load_bias16(brow + kb + 32, min(16, nv), bnext);
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
            pb.x = f2bf(sc[4 * t + 0]); pb.y = f2bf(sc[4 * t + 1]);
            pb.z = f2bf(sc[4 * t + 2]); pb.w = f2bf(sc[4 * t + 3]);
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
        pb.x = f2bf(s4[0]); pb.y = f2bf(s4[1]); pb.z = f2bf(s4[2]); pb.w = f2bf(s4[3]);
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
template <typename T, int D, int NT, bool DROP>
__global__ __launch_bounds__(64 * NT) void k_dense_bwd(const T* __restrict__ Q, const T* __restrict__ K,
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
    // XCD-aware placement as in the forward; one workgroup per (graph, head) pair
    const int win = blockIdx.x / (8 * H), rem = blockIdx.x % (8 * H);
    const int g = win * 8 + (rem & 7), h = rem >> 3;
    if (g >= nb) return;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int col = lane & 31, half = lane >> 5;
    const bool hasb = bias != nullptr;
    const int tail = S - (NT - 1) * 32;          // rows / keys in the last tile
    const bool thin = tail <= 4;
    const int nt_full = thin ? NT - 1 : NT;      // tiles that take the general path
    const T* bias_gh = hasb ? bias + ((int64_t)g * H + h) * S * S : nullptr;
    // the first query-major group of this lane's bias row, requested before anything else
    const int qi = wave * 32 + col;
    const bool qok = qi < S;
    const T* brow = hasb ? bias_gh + (int64_t)(qok ? qi : 0) * S : nullptr;
    Bias16<T> bcur, bnext;
    zero_bias16(bcur);
    zero_bias16(bnext);
    const bool vec_wave = thin && wave == NT - 1;     // the wave of a last tile of at most four rows: vector path
    if (hasb && qok && !vec_wave) load_bias16(brow + 16 * half, min(16, S - 16 * half), bcur);
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

    // ---- query tile `wave`: dQ -------------------------------------------------
    if (vec_wave) {
        thin_rows_bwd_q<T, D, SP, DROP>(q_rm, k_rm, v_rm, g_rm, lse_l, dd_l, bias_gh,
                                        dbias != nullptr ? dbias + ((int64_t)g * H + h) * S * S : nullptr, dQ, g, h, S, H,
                                        scale, (NT - 1) * 32, tail, lane, da);
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
        float16_t dq = zero16();
#pragma unroll 1
        for (int kt = 0; kt < nt_full; ++kt) {
            const int kb = kt * 32 + 16 * half;
            if (kt + 1 < NT && hasb && qok) {
                const int nv = S - (kb + 32);
                if (nv > 0) load_bias16(brow + kb + 32, min(16, nv), bnext);
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
                db[t].x = f2bf(sc[4 * t + 0]); db[t].y = f2bf(sc[4 * t + 1]);
                db[t].z = f2bf(sc[4 * t + 2]); db[t].w = f2bf(sc[4 * t + 3]);
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
            short4_t db0;
            db0.x = f2bf(s4[0]); db0.y = f2bf(s4[1]); db0.z = f2bf(s4[2]); db0.w = f2bf(s4[3]);
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
        thin_rows_bwd_k<T, D, SP, DROP>(q_rm, k_rm, v_rm, g_rm, lse_l, dd_l, bias_gh, dK, dV, g, h, S, H, scale,
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
        const T* bcol = hasb ? bias_gh + (kok ? ki : 0) : nullptr;
        decltype(raw1(bcol)) braw[16], braw_next[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) { braw[r] = 0; braw_next[r] = 0; }
        if (hasb && kok) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int qq = 8 * (r / 4) + 4 * half + (r % 4);
                if (qq < S) braw[r] = raw1(bcol + (int64_t)qq * S);
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
                    if (qq < S) braw_next[r] = raw1(bcol + (int64_t)qq * S);
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
                db.x = f2bf(sc[4 * t + 0]); db.y = f2bf(sc[4 * t + 1]);
                db.z = f2bf(sc[4 * t + 2]); db.w = f2bf(sc[4 * t + 3]);
                pb.x = f2bf(pr[4 * t + 0]); pb.y = f2bf(pr[4 * t + 1]);
                pb.z = f2bf(pr[4 * t + 2]); pb.w = f2bf(pr[4 * t + 3]);
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
            db.x = f2bf(s4[0]); db.y = f2bf(s4[1]); db.z = f2bf(s4[2]); db.w = f2bf(s4[3]);
            pb.x = f2bf(p4[0]); pb.y = f2bf(p4[1]); pb.z = f2bf(p4[2]); pb.w = f2bf(p4[3]);
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
};

template <typename T, int D, int NT>
static int launch_dense(const DenseCall& c, bool bwd) {
    constexpr int lds_f = fwd_lds_bytes<D, NT>(), lds_b = bwd_lds_bytes<D, NT>();
    if constexpr (lds_f > kLdsLimit || lds_b > kLdsLimit) {
        set_error("dense attention: S=%d with head dim %d needs %d bytes of LDS (limit %d)", c.S, c.d,
                  lds_b > lds_f ? lds_b : lds_f, kLdsLimit);
        return TGT_ERR_UNSUPPORTED;
    } else {
        const float scale = sqrtf((float)c.d);     // the reference MULTIPLIES q by sqrt(d)
        const dim3 block(64 * NT);
        static bool attr_done = false;     // raise the dynamic-LDS cap once per instantiation
        if (!attr_done) {
            if (lds_f > 48 * 1024) {
                TGT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&k_dense_fwd<T, D, NT, false>),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, lds_f));
                TGT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&k_dense_fwd<T, D, NT, true>),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, lds_f));
            }
            if (lds_b > 48 * 1024) {
                TGT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&k_dense_bwd<T, D, NT, false>),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, lds_b));
                TGT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&k_dense_bwd<T, D, NT, true>),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, lds_b));
            }
            attr_done = true;
        }
        const int total_pairs = ((c.b + 7) / 8) * 8 * c.H;
        // Forward: a persistent grid of about three workgroups per CU (measured best; more resident
        // workgroups only add cache pressure), a multiple of 8 (one share per XCD).  Backward: one
        // workgroup per pair (it runs longer per pair, persistence does not pay there).
        static int fwd_grid = 0;
        if (fwd_grid == 0) {
            int dev = 0, cus = 0;
            TGT_HIP_CHECK(hipGetDevice(&dev));
            TGT_HIP_CHECK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
            fwd_grid = std::max(8, (3 * cus) & ~7);
        }
        const int nblk = bwd ? total_pairs : std::min(total_pairs, fwd_grid);
        const dim3 grid((unsigned)nblk);
        const bool drop = c.p_drop > 0.f;
        const DropArgs da = drop_args(c.p_drop, c.seed);
        if (!bwd) {
            KernelTimer t(KS_DENSE_FWD, c.st);
            if (drop)
                hipLaunchKernelGGL((k_dense_fwd<T, D, NT, true>), grid, block, lds_f, c.st, (const T*)c.q, (const T*)c.k,
                                   (const T*)c.v, (const T*)c.bias, (T*)c.o_out, c.o_lse, c.S, c.H, scale, c.b, da);
            else
                hipLaunchKernelGGL((k_dense_fwd<T, D, NT, false>), grid, block, lds_f, c.st, (const T*)c.q, (const T*)c.k,
                                   (const T*)c.v, (const T*)c.bias, (T*)c.o_out, c.o_lse, c.S, c.H, scale, c.b, da);
        } else {
            KernelTimer t(KS_DENSE_BWD, c.st);
            if (drop)
                hipLaunchKernelGGL((k_dense_bwd<T, D, NT, true>), grid, block, lds_b, c.st, (const T*)c.q, (const T*)c.k,
                                   (const T*)c.v, (const T*)c.bias, (const T*)c.out, c.lse, (const T*)c.dout,
                                   (T*)c.dq, (T*)c.dk, (T*)c.dv, (T*)c.dbias, c.S, c.H, scale, c.b, da);
            else
                hipLaunchKernelGGL((k_dense_bwd<T, D, NT, false>), grid, block, lds_b, c.st, (const T*)c.q, (const T*)c.k,
                                   (const T*)c.v, (const T*)c.bias, (const T*)c.out, c.lse, (const T*)c.dout,
                                   (T*)c.dq, (T*)c.dk, (T*)c.dv, (T*)c.dbias, c.S, c.H, scale, c.b, da);
        }
        TGT_HIP_CHECK(hipGetLastError());
        return TGT_OK;
    }
}

template <typename T, int D>
static int dispatch_nt(const DenseCall& c, bool bwd) {
    switch ((c.S + 31) / 32) {
        case 1: return launch_dense<T, D, 1>(c, bwd);
        case 2: return launch_dense<T, D, 2>(c, bwd);
        case 3: return launch_dense<T, D, 3>(c, bwd);
        case 4: return launch_dense<T, D, 4>(c, bwd);
        case 5: return launch_dense<T, D, 5>(c, bwd);
        case 6: return launch_dense<T, D, 6>(c, bwd);
        case 7: return launch_dense<T, D, 7>(c, bwd);
        case 8: return launch_dense<T, D, 8>(c, bwd);
        default:
            set_error("dense attention: sequence length %d exceeds 256", c.S);
            return TGT_ERR_UNSUPPORTED;
    }
}

template <typename T>
static int dispatch_d(const DenseCall& c, bool bwd) {
    switch (c.d) {
        case 8: return dispatch_nt<T, 8>(c, bwd);
        case 16: return dispatch_nt<T, 16>(c, bwd);
        case 32: return dispatch_nt<T, 32>(c, bwd);
        default:
            set_error("dense attention: head dim %d not in {8, 16, 32}", c.d);
            return TGT_ERR_UNSUPPORTED;
    }
}

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
    return dtype == TGT_DTYPE_F32_BF16_PRODUCTS ? tgt::dispatch_d<float>(c, false) : tgt::dispatch_d<tgt::dbf16>(c, false);
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
    return dtype == TGT_DTYPE_F32_BF16_PRODUCTS ? tgt::dispatch_d<float>(c, true) : tgt::dispatch_d<tgt::dbf16>(c, true);
}

}  // extern "C"
