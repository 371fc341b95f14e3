// Topology-aware sparse attention for gfx950: forward and backward.
//
// One fused kernel replaces the reference's chain of gathers, elementwise ops
// and atomic scatter-adds (attn_module.py:146-187): for every destination row
// of the CSR-by-destination view it forms the per-edge scores, the exponentials,
// Z and the weighted sum of V in registers and writes the row once.  The
// backward runs the same walk over the destination view (dQ, dBias) and over the
// source view (dK, dV); every output element has exactly one writer, so there
// are no atomics and the result is bit-reproducible.
//
// Lane mapping (wave = 64 lanes).  A node row holds H*d elements; each lane owns
// a chunk of 8 consecutive elements, so LPE = H*d/8 lanes cover one edge and
// LPH = d/8 lanes cover one head.  S "edge slots" work on S edges of the same
// row at once (S*LPE lanes per row); short rows use small S and several rows
// share a wave, rows up to kWaveRowMax edges use a whole wave, longer rows are
// walked by whole workgroups in segments of kBlockSeg edges whose partial sums the
// last-arriving workgroup adds in a fixed order.
#include "common.h"
#include <stdlib.h>
#include <algorithm>
#include <mutex>

namespace tgt {

struct bf16_t { uint16_t x; };

__device__ __forceinline__ float bf16_to_f32(uint32_t bits16) { return __uint_as_float(bits16 << 16); }
__device__ __forceinline__ uint32_t f32_to_bf16(float f) {   // gfx950 converts in hardware (round to nearest even)
    const __bf16 b = static_cast<__bf16>(f);
    return (uint32_t)__builtin_bit_cast(uint16_t, b);
}

__device__ __forceinline__ void load8(const float* __restrict__ p, float (&x)[8]) {
    const float4 a = *reinterpret_cast<const float4*>(p);
    const float4 b = *reinterpret_cast<const float4*>(p + 4);
    x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w;
    x[4] = b.x; x[5] = b.y; x[6] = b.z; x[7] = b.w;
}
__device__ __forceinline__ void load8(const bf16_t* __restrict__ p, float (&x)[8]) {
    const uint4 u = *reinterpret_cast<const uint4*>(p);
    x[0] = bf16_to_f32(u.x & 0xffffu); x[1] = __uint_as_float(u.x & 0xffff0000u);
    x[2] = bf16_to_f32(u.y & 0xffffu); x[3] = __uint_as_float(u.y & 0xffff0000u);
    x[4] = bf16_to_f32(u.z & 0xffffu); x[5] = __uint_as_float(u.z & 0xffff0000u);
    x[6] = bf16_to_f32(u.w & 0xffffu); x[7] = __uint_as_float(u.w & 0xffff0000u);
}
__device__ __forceinline__ void store8(float* __restrict__ p, const float (&x)[8]) {
    *reinterpret_cast<float4*>(p) = make_float4(x[0], x[1], x[2], x[3]);
    *reinterpret_cast<float4*>(p + 4) = make_float4(x[4], x[5], x[6], x[7]);
}
__device__ __forceinline__ void store8(bf16_t* __restrict__ p, const float (&x)[8]) {
    uint4 u;
    u.x = f32_to_bf16(x[0]) | (f32_to_bf16(x[1]) << 16);
    u.y = f32_to_bf16(x[2]) | (f32_to_bf16(x[3]) << 16);
    u.z = f32_to_bf16(x[4]) | (f32_to_bf16(x[5]) << 16);
    u.w = f32_to_bf16(x[6]) | (f32_to_bf16(x[7]) << 16);
    *reinterpret_cast<uint4*>(p) = u;
}
// A gathered row chunk as it arrives from memory.  The walk issues all gathers of a step first and
// converts only when a value is used: a conversion placed next to its load would make the wave
// wait for that load before the next one is issued.
template <typename T> struct Raw8;
template <> struct Raw8<float> { float x[8]; };
template <> struct Raw8<bf16_t> { uint4 u; };
__device__ __forceinline__ void load_raw(const float* __restrict__ p, Raw8<float>& r) { load8(p, r.x); }
__device__ __forceinline__ void load_raw(const bf16_t* __restrict__ p, Raw8<bf16_t>& r) {
    r.u = *reinterpret_cast<const uint4*>(p);
}
__device__ __forceinline__ void unpack(const Raw8<float>& r, float (&x)[8]) {
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] = r.x[i];
}
__device__ __forceinline__ void unpack(const Raw8<bf16_t>& r, float (&x)[8]) {
    x[0] = bf16_to_f32(r.u.x & 0xffffu); x[1] = __uint_as_float(r.u.x & 0xffff0000u);
    x[2] = bf16_to_f32(r.u.y & 0xffffu); x[3] = __uint_as_float(r.u.y & 0xffff0000u);
    x[4] = bf16_to_f32(r.u.z & 0xffffu); x[5] = __uint_as_float(r.u.z & 0xffff0000u);
    x[6] = bf16_to_f32(r.u.w & 0xffffu); x[7] = __uint_as_float(r.u.w & 0xffff0000u);
}
__device__ __forceinline__ void zero_raw(Raw8<float>& r) {
#pragma unroll
    for (int i = 0; i < 8; ++i) r.x[i] = 0.f;
}
__device__ __forceinline__ void zero_raw(Raw8<bf16_t>& r) { r.u = make_uint4(0u, 0u, 0u, 0u); }
// Dot product of two chunks as they arrived.  bf16 pairs go through v_dot2_f32_bf16 (exact products,
// fp32 sum): four instructions and no conversion of either operand.
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float dot2_bf16(uint32_t a, uint32_t b, float c) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b), c, false);
}
__device__ __forceinline__ float dot_raw(const Raw8<float>& a, const Raw8<float>& b) {
    float s = a.x[0] * b.x[0];
#pragma unroll
    for (int c = 1; c < 8; ++c) s = fmaf(a.x[c], b.x[c], s);
    return s;
}
__device__ __forceinline__ float dot_raw(const Raw8<bf16_t>& a, const Raw8<bf16_t>& b) {
    float s = dot2_bf16(a.u.x, b.u.x, 0.f);
    s = dot2_bf16(a.u.y, b.u.y, s);
    s = dot2_bf16(a.u.z, b.u.z, s);
    return dot2_bf16(a.u.w, b.u.w, s);
}
__device__ __forceinline__ float raw1(const float* p) { return *p; }
__device__ __forceinline__ uint32_t raw1(const bf16_t* p) { return p->x; }
__device__ __forceinline__ float cvt1(float x) { return x; }
__device__ __forceinline__ float cvt1(uint32_t x) { return bf16_to_f32(x); }
__device__ __forceinline__ float load1(const float* p) { return *p; }
__device__ __forceinline__ float load1(const bf16_t* p) { return bf16_to_f32(p->x); }
__device__ __forceinline__ void store1(float* p, float v) { *p = v; }
__device__ __forceinline__ void store1(bf16_t* p, float v) { p->x = (uint16_t)f32_to_bf16(v); }

// Partial sums of a split row travel between workgroups that may sit on different XCDs, whose L2s
// are not coherent with each other.  A device-wide fence would write back and invalidate a whole
// L2 for every segment; instead the few floats of a partial slot are stored and loaded with
// device-scope accesses (they go through to the memory side), nothing else is disturbed.
__device__ __forceinline__ void store_dev(float* p, float v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_dev(const float* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Eight consecutive floats (32-byte aligned) at device scope: two 16-byte accesses with the sc1 bit, which the
// atomic builtins above would split into eight 4-byte ones.
typedef float f32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void store8_dev(float* p, const float (&x)[8]) {
    const f32x4_t a = {x[0], x[1], x[2], x[3]}, b = {x[4], x[5], x[6], x[7]};
    asm volatile("global_store_dwordx4 %0, %1, off sc1\n\tglobal_store_dwordx4 %0, %2, off offset:16 sc1"
                 :: "v"(p), "v"(a), "v"(b) : "memory");
}
// The load in two steps, so that several can be in flight: dev_load8 asks, dev_arrived waits for everything asked
// (the registers pass through it, which keeps their uses behind it).
struct Dev8 { f32x4_t a, b; };
__device__ __forceinline__ void dev_load8(const float* p, Dev8& r) {
    asm volatile("global_load_dwordx4 %0, %2, off sc1\n\tglobal_load_dwordx4 %1, %2, off offset:16 sc1"
                 : "=&v"(r.a), "=&v"(r.b) : "v"(p) : "memory");
}
__device__ __forceinline__ void dev_arrived(Dev8& r0, Dev8& r1) {
    asm volatile("s_waitcnt vmcnt(0)" : "+v"(r0.a), "+v"(r0.b), "+v"(r1.a), "+v"(r1.b) :: "memory");
}
__device__ __forceinline__ void dev_arrived(Dev8& r0, Dev8& r1, Dev8& r2, Dev8& r3) {
    asm volatile("s_waitcnt vmcnt(0)"
                 : "+v"(r0.a), "+v"(r0.b), "+v"(r1.a), "+v"(r1.b), "+v"(r2.a), "+v"(r2.b), "+v"(r3.a), "+v"(r3.b) :: "memory");
}
__device__ __forceinline__ void dev_unpack(const Dev8& r, float (&x)[8]) {
    x[0] = r.a.x; x[1] = r.a.y; x[2] = r.a.z; x[3] = r.a.w; x[4] = r.b.x; x[5] = r.b.y; x[6] = r.b.z; x[7] = r.b.w;
}

__device__ __forceinline__ float dot8(const float (&a)[8], const float (&b)[8]) {
    float s = a[0] * b[0];
#pragma unroll
    for (int c = 1; c < 8; ++c) s = fmaf(a[c], b[c], s);
    return s;
}
// sum over the LPH lanes that share a head (adjacent lanes)
template <int LPH>
__device__ __forceinline__ float head_sum(float x) {
#pragma unroll
    for (int off = 1; off < LPH; off <<= 1) x += __shfl_xor(x, off);
    return x;
}
// clamp that keeps NaN (like torch.clamp)
__device__ __forceinline__ float clamp5(float x) { return x < -5.0f ? -5.0f : (x > 5.0f ? 5.0f : x); }

constexpr float kEps = 1e-6f;   // attn_module.py:187
constexpr int kUnroll = 4;      // edges in flight per slot

// Which walk a workgroup performs.
enum { MODE_FWD = 0, MODE_BWD_DST = 1, MODE_BWD_SRC = 2 };

// Operands shared by both views.
struct Common {
    const void* q;
    const void* k;
    const void* v;
    const void* g;        // dout (backward)
    const void* bias;
    const void* bias_src; // the bias as the walk by source reads it (same array, or its source-sorted copy)
    const float2* nd;     // [N, H] (1/(Z+eps), D) (backward)
    int32_t bias_mode;
    int32_t bias_se, bias_sh;   // element strides of the bias per edge / per head: (H, 1) or (1, 0)
    float inv_scale;
};

// One sorted view (by destination or by source) with its schedule and outputs.
struct SideArgs {
    const Item* items;
    const int32_t* col;
    const int32_t* eid;
    const int32_t* split_off;
    const int32_t* part2split;
    const int32_t* split_grp;     // first combine group of each split row (rows with more than kCombineFan segments have groups)
    int32_t eid_is_map;           // `eid` is not the caller's edge ids (which the wave records hold too) but another map
    int32_t n_split, n_parts;     // group counters follow the n_split row counters, group slots the n_parts segment slots
    void* out0;           // fwd: out      bwd_dst: dq     bwd_src: dk
    void* out1;           // fwd: -        bwd_dst: dbias  bwd_src: dv
    float* Z;             // fwd: Z
    float* part;          // partial sums of split rows
    int32_t* counters;    // one arrival counter per split row, zero between calls
    // optional sums computed elsewhere for the same rows (dense tiles of the block path), fp32,
    // added when the row is written: fwd (sum w v, Z) | bwd_dst dq | bwd_src (dk, dv)
    const float* init0;
    const float* init1;
    const float* initZ;
    const uint8_t* cover; // [N] 1 where the row has such sums
};

struct Acc {
    float a0[8];   // fwd: sum w v | bwd_dst: dq | bwd_src: dk
    float a1[8];   // bwd_src: dv
    float z;       // fwd: sum w
};

// Floats one partial slot holds.
template <int MODE, int HD, int H>
__host__ __device__ constexpr int part_stride() {
    return MODE == MODE_FWD ? HD + H : (MODE == MODE_BWD_DST ? HD : 2 * HD);
}

// What a lane group keeps of its own row while it walks the row's edges.
template <typename T>
struct RowRegs {
    Raw8<T> r0, r1;      // as loaded (only dot products use them): fwd q | bwd_dst q, g | bwd_src k, v
    float rz, Dh;        // bwd_dst: 1 / (Z + eps) and dout . out of the row's head
};

template <typename T, int LPE, int LPH, int MODE>
__device__ __forceinline__ void load_row(const Common& c, const int row, const int el, const bool valid,
                                         RowRegs<T>& rr, Acc& acc) {
    constexpr int H = LPE / LPH;
    constexpr int HD = LPE * 8;
    const T* __restrict__ Q = static_cast<const T*>(c.q);
    const T* __restrict__ K = static_cast<const T*>(c.k);
    const T* __restrict__ V = static_cast<const T*>(c.v);
    const T* __restrict__ Gd = static_cast<const T*>(c.g);
    const int64_t row_off = (int64_t)row * HD + el * 8;
    rr.rz = 0.f; rr.Dh = 0.f;
    zero_raw(rr.r0); zero_raw(rr.r1);
#pragma unroll
    for (int i = 0; i < 8; ++i) { acc.a0[i] = 0.f; acc.a1[i] = 0.f; }
    acc.z = 0.f;
    if (valid) {
        if (MODE == MODE_FWD) {
            load_raw(Q + row_off, rr.r0);
        } else if (MODE == MODE_BWD_DST) {
            load_raw(Q + row_off, rr.r0);
            load_raw(Gd + row_off, rr.r1);
            const float2 nd = c.nd[(int64_t)row * H + el / LPH];
            rr.rz = nd.x; rr.Dh = nd.y;
        } else {
            load_raw(K + row_off, rr.r0);
            load_raw(V + row_off, rr.r1);
        }
    }
}

// kUnroll edges of one slot: nb[u] = the other endpoint, ed[u] = the row of the bias / dbias arrays, ok[u] =
// whether the edge exists.  All gathers of the step are issued before anything is used.  For 4-byte
// elements the lanes of a missing edge load nothing; for 2-byte elements every lane loads (a missing edge
// must then name a valid node and bias row - callers repeat the row's last edge - and only the
// arithmetic is skipped): with no lane-dependent branch around them the loads go out back to back, and
// the rows stay packed until they are used.
template <typename T, int LPE, int LPH, int MODE, int HASB>
__device__ __forceinline__ void edge_step(const Common& c, const SideArgs& s, const RowRegs<T>& rr,
                                          const int (&nb)[kUnroll], const int (&ed)[kUnroll],
                                          const bool (&ok)[kUnroll], const int el, Acc& acc) {
    constexpr int H = LPE / LPH;
    constexpr int HD = LPE * 8;
    const int head = el / LPH;
    const T* __restrict__ Q = static_cast<const T*>(c.q);
    const T* __restrict__ K = static_cast<const T*>(c.k);
    const T* __restrict__ V = static_cast<const T*>(c.v);
    const T* __restrict__ Gd = static_cast<const T*>(c.g);
    const T* __restrict__ B = static_cast<const T*>(MODE == MODE_BWD_SRC ? c.bias_src : c.bias);
    const int bias_se = c.bias_se, bias_sh = c.bias_sh;
    const float inv_scale = c.inv_scale;
    Raw8<T> g0[kUnroll], g1[kUnroll];          // gathered rows, unconverted
    decltype(raw1(B)) braw[kUnroll];
    float2 ndv[kUnroll];
    if constexpr (sizeof(T) == 4) {
        // The edge ids are waited for here, on every path.  Otherwise the wait sits inside the first lane-masked
        // block below, and behind that block the compiler must assume the ids may still be in flight: it then
        // waits for everything outstanding - the first edge's rows - before it asks for the second edge's.
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) asm volatile("" ::"v"(nb[u]), "v"(ed[u]));
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        braw[u] = 0;
        ndv[u] = make_float2(0.f, 0.f);
        if constexpr (sizeof(T) == 4) { zero_raw(g0[u]); zero_raw(g1[u]); }
        if (sizeof(T) != 4 || ok[u]) {
            const int64_t o = (int64_t)nb[u] * HD + el * 8;
            if (MODE == MODE_BWD_SRC) {
                load_raw(Q + o, g0[u]);
                load_raw(Gd + o, g1[u]);
                ndv[u] = c.nd[(int64_t)nb[u] * H + head];
            } else {
                load_raw(K + o, g0[u]);
                load_raw(V + o, g1[u]);
            }
            if (HASB) braw[u] = raw1(B + (int64_t)ed[u] * bias_se + head * bias_sh);
        }
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        if constexpr (sizeof(T) == 2) {
            // The edge's rows are named here, outside the lane-masked block that uses them: the compiler otherwise
            // moves their loads into that block (its only user), where they are asked for and waited for one edge
            // at a time instead of with the other gathers of the step.
            asm volatile("" ::"v"(g0[u].u.x), "v"(g0[u].u.y), "v"(g0[u].u.z), "v"(g0[u].u.w), "v"(g1[u].u.x), "v"(g1[u].u.y),
                         "v"(g1[u].u.z), "v"(g1[u].u.w));
        }
        if (ok[u]) {
            float x0[8], x1[8];
            unpack(g0[u], x0);
            unpack(g1[u], x1);
            const float bbu = HASB ? cvt1(braw[u]) : 0.f;
            // raw score: identical arithmetic in all three walks so that the
            // recomputed weights and the clamp mask agree bit for bit
            const float raw = head_sum<LPH>(dot_raw(rr.r0, g0[u])) * inv_scale;
            const float w = __expf(clamp5(raw) + bbu);
            if (MODE == MODE_FWD) {
                acc.z += w;
#pragma unroll
                for (int i = 0; i < 8; ++i) acc.a0[i] = fmaf(w, x1[i], acc.a0[i]);
            } else {
                const bool inside = (raw >= -5.0f) & (raw <= 5.0f);   // torch clamp backward: inclusive
                if (MODE == MODE_BWD_DST) {
                    const float t = head_sum<LPH>(dot_raw(rr.r1, g1[u]));   // g_dst . v_src
                    const float dS = w * rr.rz * (t - rr.Dh);
                    T* __restrict__ dB = static_cast<T*>(s.out1);
                    if (HASB && dB != nullptr) {
                        if (bias_sh != 0) {       // one value per edge and head
                            if (el % LPH == 0) store1(dB + (int64_t)ed[u] * H + head, dS);
                        } else {                  // one value per edge: sum over heads
                            float t2 = dS;   // sum over heads; every head is held by LPH lanes
#pragma unroll
                            for (int off = 1; off < LPE; off <<= 1) t2 += __shfl_xor(t2, off);
                            if (el == 0) store1(dB + ed[u], t2 * (1.0f / LPH));
                        }
                    }
                    const float md = inside ? dS : 0.f;
#pragma unroll
                    for (int i = 0; i < 8; ++i) acc.a0[i] = fmaf(md, x0[i], acc.a0[i]);
                } else {
                    const float p = w * ndv[u].x;
                    const float t = head_sum<LPH>(dot_raw(g1[u], rr.r1));   // g_dst . v_src
                    const float dS = p * (t - ndv[u].y);
                    const float md = inside ? dS : 0.f;
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        acc.a0[i] = fmaf(md, x0[i], acc.a0[i]);   // dk += m dS q_dst
                        acc.a1[i] = fmaf(p, x1[i], acc.a1[i]);    // dv += p g_dst
                    }
                }
            }
        }
    }
}

// add the S edge slots of a lane group (all lanes take part)
template <int LPE, int S, int MODE>
__device__ __forceinline__ void add_slots(Acc& acc) {
    constexpr int G = LPE * S;
#pragma unroll
    for (int off = LPE; off < G; off <<= 1) {
        if (MODE == MODE_FWD) acc.z += __shfl_xor(acc.z, off);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            acc.a0[i] += __shfl_xor(acc.a0[i], off);
            if (MODE == MODE_BWD_SRC) acc.a1[i] += __shfl_xor(acc.a1[i], off);
        }
    }
}

// x of lane (l ^ OFF).  The exchange between the two halves of a row of 16 lanes is a DPP operand of the
// add that uses it, the others go through the LDS crossbar.
template <int OFF>
__device__ __forceinline__ float lane_xor(float x) {
    if constexpr (OFF == 8) {
        return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x128 /* row_ror:8 */,
                                                                     0xf, 0xf, false));
    } else {
        return __shfl_xor(x, OFF);
    }
}

// One level of the reduce-scatter below: the 2 N values of a lane become N, the sums with lane (l ^ OFF) of
// the lower (bit OFF of the lane clear) or upper (set) half of them.
template <int N, int OFF>
__device__ __forceinline__ void halve(float (&a)[8], const bool upper) {
    if constexpr (N >= 1) {
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const float keep = upper ? a[i + N] : a[i];
            const float send = upper ? a[i] : a[i + N];
            a[i] = keep + lane_xor<OFF>(send);
        }
    }
}

// Adds the S edge slots of a lane group so that the sums end up spread over the slots: afterwards the
// lane of slot t holds, in a[0 .. 8/S), the sums of the elements t * (8/S) ... of its chunk - log2(S) levels
// with 4, 2, 1 exchanges instead of 8 each, and every lane has a share of the row to finish and store.
// The additions pair the same values as add_slots does, so both give the same bits.
template <int LPE, int S>
__device__ __forceinline__ void reduce_slots(float (&a)[8], const int slot) {
    if constexpr (S >= 2) halve<4, LPE * S / 2>(a, (slot & (S / 2)) != 0);
    if constexpr (S >= 4) halve<2, LPE * S / 4>(a, (slot & (S / 4)) != 0);
    if constexpr (S >= 8) halve<1, LPE * S / 8>(a, (slot & (S / 8)) != 0);
}

template <int CNT>
__device__ __forceinline__ void store_n(float* __restrict__ p, const float (&x)[8]) {
    if constexpr (CNT == 1) *p = x[0];
    else if constexpr (CNT == 2) *reinterpret_cast<float2*>(p) = make_float2(x[0], x[1]);
    else {
        *reinterpret_cast<float4*>(p) = make_float4(x[0], x[1], x[2], x[3]);
        if constexpr (CNT == 8) *reinterpret_cast<float4*>(p + 4) = make_float4(x[4], x[5], x[6], x[7]);
    }
}
template <int CNT>
__device__ __forceinline__ void store_n(bf16_t* __restrict__ p, const float (&x)[8]) {
    if constexpr (CNT == 1) p->x = (uint16_t)f32_to_bf16(x[0]);
    else if constexpr (CNT == 2) *reinterpret_cast<uint32_t*>(p) = f32_to_bf16(x[0]) | (f32_to_bf16(x[1]) << 16);
    else if constexpr (CNT == 4)
        *reinterpret_cast<uint2*>(p) = make_uint2(f32_to_bf16(x[0]) | (f32_to_bf16(x[1]) << 16),
                                                  f32_to_bf16(x[2]) | (f32_to_bf16(x[3]) << 16));
    else store8(p, x);
}
template <int CNT>
__device__ __forceinline__ void add_n(const float* __restrict__ p, float (&x)[8]) {
#pragma unroll
    for (int i = 0; i < CNT; ++i) x[i] += p[i];
}

// Final value of a row of a wave item from the sums of its S slots: all S * LPE lanes of the row's lane
// group take part, each finishes and stores 8 / S elements.
template <typename T, int LPE, int LPH, int S, int MODE, bool TILES>
__device__ __forceinline__ void finish_row(const Common& c, const SideArgs& s, const int row, const int slot,
                                           const int el, const bool valid, Acc& acc) {
    constexpr int H = LPE / LPH;
    constexpr int HD = LPE * 8;
    constexpr int SR = S > 8 ? 8 : S;     // slots the 8 elements of a chunk are spread over
    constexpr int CNT = 8 / SR;
    if constexpr (S > SR) {               // more slots than elements: the upper slot bits are plain sums
#pragma unroll
        for (int off = LPE * SR; off < LPE * S; off <<= 1) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                acc.a0[i] += __shfl_xor(acc.a0[i], off);
                if (MODE == MODE_BWD_SRC) acc.a1[i] += __shfl_xor(acc.a1[i], off);
            }
        }
    }
    const int sl = slot % SR;
    reduce_slots<LPE, SR>(acc.a0, sl);
    if (MODE == MODE_BWD_SRC) reduce_slots<LPE, SR>(acc.a1, sl);
    if (MODE == MODE_FWD) {
#pragma unroll
        for (int off = LPE; off < LPE * S; off <<= 1) acc.z += __shfl_xor(acc.z, off);
    }
    if (!valid || slot >= SR) return;
    const int64_t off = (int64_t)row * HD + el * 8 + sl * CNT;
    if (MODE != MODE_FWD) {
#pragma unroll
        for (int i = 0; i < CNT; ++i) acc.a0[i] *= c.inv_scale;
    }
    if (TILES) {   // sums of the dense tiles of the block path for this row, if it has any
        if (s.cover[row] != 0) {
            add_n<CNT>(s.init0 + off, acc.a0);
            if (MODE == MODE_FWD) acc.z += s.initZ[(int64_t)row * H + el / LPH];
            if (MODE == MODE_BWD_SRC) add_n<CNT>(s.init1 + off, acc.a1);
        }
    }
    if (MODE == MODE_FWD) {
        const float inv = 1.0f / (acc.z + kEps);
#pragma unroll
        for (int i = 0; i < CNT; ++i) acc.a0[i] *= inv;
        if (sl == 0 && el % LPH == 0) s.Z[(int64_t)row * H + el / LPH] = acc.z;
    }
    store_n<CNT>(static_cast<T*>(s.out0) + off, acc.a0);
    if (MODE == MODE_BWD_SRC) store_n<CNT>(static_cast<T*>(s.out1) + off, acc.a1);
}

// Walks `len` edges starting at sorted position `start` of node `row` with S edge
// slots (this lane is slot `slot`, element chunk `el`), reading the plan's sorted view.  On return
// every lane holds the sums of its own slot (add_slots or reduce_slots adds the slots).
template <typename T, int LPE, int LPH, int S, int MODE, int HASB>
__device__ __forceinline__ void walk_range(const Common& c, const SideArgs& s, const int row, const int start,
                                           const int len, const int slot, const int el, const bool valid,
                                           Acc& acc) {
    RowRegs<T> rr;
    load_row<T, LPE, LPH, MODE>(c, row, el, valid, rr, acc);
    const int32_t* __restrict__ col = s.col + start;
    // HASB == 2: no edge-id array, the bias rows are in this side's own sorted order (row = sorted position)
    constexpr bool ident = HASB == 2;
    const int32_t* __restrict__ eid = ident ? nullptr : s.eid + start;
    const int n = valid ? len : 0;
    // endpoints and bias rows of the step that starts at edge e0 of the row
    auto load_ids = [&](const int e0, int (&nb)[kUnroll], int (&ed)[kUnroll]) {
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const int e = e0 + u * S;
            if constexpr (sizeof(T) == 4) {
                nb[u] = 0; ed[u] = 0;
                if (e < n) {
                    nb[u] = col[e];
                    if (HASB) ed[u] = ident ? start + e : eid[e];
                }
            } else {   // lanes past the end of the row repeat its last edge (a line the wave is reading anyway)
                const int ec = min(e, n - 1);
                nb[u] = col[ec];
                ed[u] = HASB ? (ident ? start + ec : eid[ec]) : 0;
            }
        }
    };
    if (n <= 0) return;
    if constexpr (sizeof(T) == 4) {
#pragma unroll 1
        for (int e0 = slot; e0 < n; e0 += S * kUnroll) {
            int nb[kUnroll], ed[kUnroll];
            bool ok[kUnroll];
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) ok[u] = e0 + u * S < n;
            load_ids(e0, nb, ed);
            edge_step<T, LPE, LPH, MODE, HASB>(c, s, rr, nb, ed, ok, el, acc);
        }
    } else {
        // the ids of the next step are asked for before this step's gathers: a step waits for one memory
        // round trip, not for two in a row (2-byte elements leave the registers for it)
        int nb[kUnroll], ed[kUnroll];
        load_ids(slot, nb, ed);
#pragma unroll 1
        for (int e0 = slot; e0 < n; e0 += S * kUnroll) {
            int nb2[kUnroll], ed2[kUnroll];
            bool ok[kUnroll];
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) ok[u] = e0 + u * S < n;
            load_ids(e0 + S * kUnroll, nb2, ed2);
            edge_step<T, LPE, LPH, MODE, HASB>(c, s, rr, nb, ed, ok, el, acc);
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) { nb[u] = nb2[u]; ed[u] = ed2[u]; }
        }
    }
}

// What one lane takes from its wave's record, asked for in one go when the kernel starts: none of the addresses
// depends on the row class (the record lists row, start and length per lane group), so the wave has its rows and
// its edges after one memory round trip, whatever the code then says they are.
struct RecLane {
    uint32_t code;
    int row, start, len;     // of the row this lane group works on (zeros behind the record's last row)
    int4 cols, eids;         // inline classes: the lane group's four edges (other endpoint, bias row)
    const int32_t* col_p;    // EDGES == false: where cols and eids are, for a read at the point of use
    const int32_t* eid_p;
};
// EDGES: whether the four edges come along at once.  The 4-byte backward holds two gathered rows per edge in
// registers and has none to spare for edges that wait through the class dispatch: it reads them where it uses them.
template <int LPE, bool EDGES>
__device__ __forceinline__ RecLane load_rec_lane(const WaveRec<LPE>& rec) {
    const int lg = (threadIdx.x & (kWave - 1)) / LPE;
    RecLane r;
    r.code = rec.code;
    r.row = rec.row[lg];
    r.start = rec.start[lg];
    r.len = rec.len[lg];
    r.col_p = rec.col + lg * kUnroll;
    r.eid_p = rec.eid + lg * kUnroll;
    if (EDGES) {
        r.cols = *reinterpret_cast<const int4*>(r.col_p);
        r.eids = *reinterpret_cast<const int4*>(r.eid_p);
    }
    return r;
}
template <typename T, int MODE> constexpr bool rec_edges_early() { return sizeof(T) == 2 || MODE == MODE_FWD; }

// The same for a row of at most S * kUnroll edges whose endpoints and bias rows come with the wave's
// record (one step, no loop): the record lists them in lane order, four consecutive entries per
// (row, slot), an edge past the end of the row repeats the row's last one.
template <typename T, int LPE, int LPH, int S, int MODE, int HASB>
__device__ __forceinline__ void walk_record(const Common& c, const SideArgs& s, const RecLane& rec, const int row,
                                            const int start, const int len, const int slot, const int el,
                                            const bool valid, Acc& acc) {
    const int4 cols = rec_edges_early<T, MODE>() ? rec.cols : *reinterpret_cast<const int4*>(rec.col_p);
    int nb[kUnroll] = {cols.x, cols.y, cols.z, cols.w};
    int ed[kUnroll] = {0, 0, 0, 0};
    bool ok[kUnroll];
    const int n = valid ? len : 0;
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) ok[u] = slot + u * S < n;
    if (HASB == 2) {          // bias rows in this view's sorted order: row = sorted position
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) ed[u] = start + min(slot + u * S, max(n - 1, 0));
    } else if (HASB) {
        if (s.eid_is_map) {   // the bias rows are named by a map from sorted positions, not by the caller's edge ids
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) ed[u] = s.eid[start + min(slot + u * S, max(n - 1, 0))];
        } else {
            const int4 e4 = rec_edges_early<T, MODE>() ? rec.eids : *reinterpret_cast<const int4*>(rec.eid_p);
            ed[0] = e4.x; ed[1] = e4.y; ed[2] = e4.z; ed[3] = e4.w;
        }
    }
    // The ids are complete here, on every path (the map above is a second look-up that only some calls make), and
    // only then is the row's own data asked for: it and the gathers of the step go out back to back, and nothing
    // behind a branch makes the gathers wait for the row.
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) asm volatile("" ::"v"(nb[u]), "v"(ed[u]));
    RowRegs<T> rr;
    load_row<T, LPE, LPH, MODE>(c, row, el, valid, rr, acc);
    edge_step<T, LPE, LPH, MODE, HASB>(c, s, rr, nb, ed, ok, el, acc);
}

// Final value of a row from its sums, written by the LPE lanes that own the chunks.
template <typename T, int LPE, int LPH, int MODE, bool TILES>
__device__ __forceinline__ void write_row(const Common& c, const SideArgs& s, const int row, const int el,
                                          Acc& acc) {
    constexpr int H = LPE / LPH;
    constexpr int HD = LPE * 8;
    const int64_t row_off = (int64_t)row * HD + el * 8;
    if (MODE != MODE_FWD) {
#pragma unroll
        for (int i = 0; i < 8; ++i) acc.a0[i] *= c.inv_scale;
    }
    if (TILES) {   // sums of the dense tiles of the block path for this row, if it has any
        if (s.cover[row] != 0) {
            float t[8];
            load8(s.init0 + row_off, t);
#pragma unroll
            for (int i = 0; i < 8; ++i) acc.a0[i] += t[i];
            if (MODE == MODE_FWD) acc.z += s.initZ[(int64_t)row * H + el / LPH];
            if (MODE == MODE_BWD_SRC) {
                load8(s.init1 + row_off, t);
#pragma unroll
                for (int i = 0; i < 8; ++i) acc.a1[i] += t[i];
            }
        }
    }
    if (MODE == MODE_FWD) {
        const float inv = 1.0f / (acc.z + kEps);
#pragma unroll
        for (int i = 0; i < 8; ++i) acc.a0[i] *= inv;
        store8(static_cast<T*>(s.out0) + row_off, acc.a0);
        if (el % LPH == 0) s.Z[(int64_t)row * H + el / LPH] = acc.z;
    } else {
        store8(static_cast<T*>(s.out0) + row_off, acc.a0);
        if (MODE == MODE_BWD_SRC) store8(static_cast<T*>(s.out1) + row_off, acc.a1);
    }
}

// Rows of one wave: 64 / (LPE*S) rows of one length class, named by the wave's record.  The longest
// class walks the plan's sorted view step by step; the others find their (at most S * kUnroll) edges
// in the record itself.
template <typename T, int LPE, int LPH, int S, int MODE, int HASB, bool TILES, bool INLINE>
__device__ __forceinline__ void wave_rows(const Common& c, const SideArgs& s, const RecLane& rec) {
    constexpr int G = LPE * S;
    const int lane = threadIdx.x & (kWave - 1);
    const int sub = lane / G, gl = lane % G;
    const int slot = gl / LPE, el = gl % LPE;
    bool valid = sub < (int)(__builtin_amdgcn_readfirstlane(rec.code) >> 8);
    int row = rec.row, start = rec.start, len = rec.len;
    // The record's words are waited for here, by all lanes: a wait that first happens inside a lane-masked block
    // (the row's own loads below) makes the compiler wait for everything outstanding behind that block - the
    // row's data - before the gathers may go out.
    asm volatile("" ::"v"(row), "v"(start), "v"(len));
    if (INLINE && rec_edges_early<T, MODE>())
        asm volatile("" ::"v"(rec.cols.x), "v"(rec.cols.y), "v"(rec.cols.z), "v"(rec.cols.w), "v"(rec.eids.x), "v"(rec.eids.y),
                     "v"(rec.eids.z), "v"(rec.eids.w));
    if (!valid) { row = 0; start = 0; len = 0; }
    // block path: a row that has tiles and no edge here was written by the tile kernels (they see the same row
    // pointers); nothing of it is loaded or stored
    if (TILES) valid = valid && !(len == 0 && s.cover[row] != 0);
    Acc acc;
    if (INLINE) walk_record<T, LPE, LPH, S, MODE, HASB>(c, s, rec, row, start, len, slot, el, valid, acc);
    else walk_range<T, LPE, LPH, S, MODE, HASB>(c, s, row, start, len, slot, el, valid, acc);
    finish_row<T, LPE, LPH, S, MODE, TILES>(c, s, row, slot, el, valid, acc);
}

template <typename T, int LPE, int LPH, int MODE, int HASB, bool TILES>
__device__ __forceinline__ void wave_dispatch(const Common& c, const SideArgs& s, const RecLane& rec, const int kind) {
    switch (kind) {
        case 0: wave_rows<T, LPE, LPH, slots_for_class(LPE, 0), MODE, HASB, TILES, false>(c, s, rec); break;
        case 1: wave_rows<T, LPE, LPH, slots_for_class(LPE, 1), MODE, HASB, TILES, class_inline(LPE, 1)>(c, s, rec); break;
        case 2: wave_rows<T, LPE, LPH, slots_for_class(LPE, 2), MODE, HASB, TILES, class_inline(LPE, 2)>(c, s, rec); break;
        case 3: wave_rows<T, LPE, LPH, slots_for_class(LPE, 3), MODE, HASB, TILES, class_inline(LPE, 3)>(c, s, rec); break;
        default: wave_rows<T, LPE, LPH, slots_for_class(LPE, 4), MODE, HASB, TILES, class_inline(LPE, 4)>(c, s, rec); break;
    }
}

// LDS of one workgroup: sums of its lane groups, then (last arriver only) sums of
// the partial slots of a split row.
template <int LPE>
struct BlockLds {
    static constexpr int HD = LPE * 8;
    static constexpr int STRIDE = 2 * HD + LPE;               // a0 | a1 | z (one float per chunk)
    static constexpr int NGROUP = kBlock / LPE;               // combine groups
    float red[NGROUP * STRIDE];
    int last;
};

// Adds the partial slots [first, first + count) of s.part with all threads of the workgroup: the
// NGROUP groups of LPE threads take slots first + grp, first + grp + NGROUP, ... (two per step, so
// that the device-scope loads of two slots are in flight together), LDS adds the groups in group order.
// On return threads 0 .. LPE-1 hold the sums.  The order of the additions is fixed by (first, count).
template <int LPE, int LPH, int MODE>
__device__ __forceinline__ void sum_slots(const SideArgs& s, const int first, const int count, BlockLds<LPE>& lds,
                                          Acc& acc) {
    constexpr int H = LPE / LPH;
    constexpr int HD = LPE * 8;
    constexpr int STRIDE = BlockLds<LPE>::STRIDE;
    constexpr int NGROUP = BlockLds<LPE>::NGROUP;
    constexpr int PS = part_stride<MODE, HD, H>();
    const int tid = threadIdx.x;
    const int grp2 = tid / LPE, el2 = tid % LPE;
    {
        float a0[8], a1[8], z = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) { a0[i] = 0.f; a1[i] = 0.f; }
        for (int p = grp2; p < count; p += 2 * NGROUP) {
            const bool two = p + NGROUP < count;
            const float* srcA = s.part + (int64_t)(first + p) * PS;
            const float* srcB = s.part + (int64_t)(first + (two ? p + NGROUP : p)) * PS;
            float tA[8], tB[8], uA[8], uB[8], zA = 0.f, zB = 0.f;
            Dev8 rA, rB, sA, sB;
            dev_load8(srcA + el2 * 8, rA);
            dev_load8(srcB + el2 * 8, rB);
            if (MODE == MODE_BWD_SRC) {
                dev_load8(srcA + HD + el2 * 8, sA);
                dev_load8(srcB + HD + el2 * 8, sB);
            }
            if (MODE == MODE_FWD) {
                zA = load_dev(srcA + HD + el2 / LPH);
                zB = load_dev(srcB + HD + el2 / LPH);
            }
            if (MODE == MODE_BWD_SRC) {
                dev_arrived(rA, rB, sA, sB);
                dev_unpack(sA, uA);
                dev_unpack(sB, uB);
            } else {
                dev_arrived(rA, rB);
            }
            dev_unpack(rA, tA);
            dev_unpack(rB, tB);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                a0[i] += tA[i];
                if (two) a0[i] += tB[i];
                if (MODE == MODE_BWD_SRC) {
                    a1[i] += uA[i];
                    if (two) a1[i] += uB[i];
                }
            }
            if (MODE == MODE_FWD) {
                z += zA;
                if (two) z += zB;
            }
        }
        float* r = lds.red + grp2 * STRIDE;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            r[el2 * 8 + i] = a0[i];
            if (MODE == MODE_BWD_SRC) r[HD + el2 * 8 + i] = a1[i];
        }
        if (MODE == MODE_FWD) r[2 * HD + el2] = z;
    }
    __syncthreads();
    if (tid < LPE) {
#pragma unroll
        for (int i = 0; i < 8; ++i) { acc.a0[i] = 0.f; acc.a1[i] = 0.f; }
        acc.z = 0.f;
        const int ng = count < NGROUP ? count : NGROUP;     // groups that added anything
        for (int gI = 0; gI < ng; ++gI) {
            const float* r = lds.red + gI * STRIDE;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                acc.a0[i] += r[tid * 8 + i];
                if (MODE == MODE_BWD_SRC) acc.a1[i] += r[HD + tid * 8 + i];
            }
            if (MODE == MODE_FWD) acc.z += r[2 * HD + tid];
        }
    }
}

// Threads 0 .. LPE-1 store their sums into partial slot `slot` with device-scope stores.
template <int LPE, int LPH, int MODE>
__device__ __forceinline__ void store_slot(const SideArgs& s, const int slot, const Acc& acc) {
    constexpr int H = LPE / LPH;
    constexpr int HD = LPE * 8;
    constexpr int PS = part_stride<MODE, HD, H>();
    const int tid = threadIdx.x;
    float* p = s.part + (int64_t)slot * PS;
    store8_dev(p + tid * 8, acc.a0);
    if (MODE == MODE_BWD_SRC) store8_dev(p + HD + tid * 8, acc.a1);
    if (MODE == MODE_FWD && tid % LPH == 0) store_dev(p + HD + tid / LPH, acc.z);
}

// Arrival at counter `idx`: the slot written by threads 0 .. LPE-1 (all in wave 0) is published before
// the counter moves: once wave 0's device-scope stores are acknowledged the slot is visible to all
// XCDs.  Returns (to every thread) whether this workgroup is the last of `expected` to arrive; the last
// one also puts the counter back to zero for the next call.
template <int LPE>
__device__ __forceinline__ bool arrive(const SideArgs& s, const int idx, const int expected, BlockLds<LPE>& lds) {
    const int tid = threadIdx.x;
    if (tid < kWave) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        if (tid == 0) {
            const int old = __hip_atomic_fetch_add(&s.counters[idx], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const int last = (old == expected - 1) ? 1 : 0;
            if (last) __hip_atomic_store(&s.counters[idx], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            lds.last = last;
        }
    }
    __syncthreads();
    const bool last = lds.last != 0;
    __syncthreads();          // lds.last may be written again by the next arrival
    return last;
}

// Workgroup item: one segment (<= kBlockSeg edges) of a long row.  The lane groups
// of the 4 waves each walk a share of the segment, LDS adds them in a fixed order.
// If the row has several segments each workgroup stores its sums in a partial
// slot, and the workgroup that arrives last adds the slots in slot order and
// writes the row - no second launch, no floating-point atomics, and the order of
// the additions does not depend on which workgroup is last.  A row with more than
// kCombineFan segments does this in two levels: the last arriver of every run of
// kCombineFan consecutive slots adds them into a group slot, and the last group adds the
// group slots - the sums of a row with hundreds of segments are formed while the
// launch is under way, not by one workgroup at its end.
template <typename T, int LPE, int LPH, int MODE, int HASB, bool TILES>
__device__ __forceinline__ void block_item(const Common& c, const SideArgs& s, const Item it,
                                           BlockLds<LPE>& lds) {
    constexpr int S = slots_for_class(LPE, 0);
    constexpr int G = LPE * S;
    constexpr int IPW = kWave / G;
    constexpr int NG = (kBlock / kWave) * IPW;    // lane groups in the workgroup
    constexpr int HD = LPE * 8;
    constexpr int STRIDE = BlockLds<LPE>::STRIDE;
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int sub = lane / G, gl = lane % G;
    const int slot = gl / LPE, el = gl % LPE;
    const int grp = (tid >> 6) * IPW + sub;
    // share of this lane group: consecutive chunk of the segment
    const int share = (it.len + NG - 1) / NG;
    const int lo = min(grp * share, it.len);
    const int hi = min(lo + share, it.len);
    Acc acc;
    walk_range<T, LPE, LPH, S, MODE, HASB>(c, s, it.row, it.start + lo, hi - lo, slot, el, true, acc);
    add_slots<LPE, S, MODE>(acc);
    if (slot == 0) {
        float* r = lds.red + grp * STRIDE;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            r[el * 8 + i] = acc.a0[i];
            if (MODE == MODE_BWD_SRC) r[HD + el * 8 + i] = acc.a1[i];
        }
        if (MODE == MODE_FWD) r[2 * HD + el] = acc.z;
    }
    __syncthreads();
    if (tid < LPE) {   // tid == el here
#pragma unroll
        for (int i = 0; i < 8; ++i) { acc.a0[i] = 0.f; acc.a1[i] = 0.f; }
        acc.z = 0.f;
        for (int gI = 0; gI < NG; ++gI) {
            const float* r = lds.red + gI * STRIDE;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                acc.a0[i] += r[tid * 8 + i];
                if (MODE == MODE_BWD_SRC) acc.a1[i] += r[HD + tid * 8 + i];
            }
            if (MODE == MODE_FWD) acc.z += r[2 * HD + tid];
        }
        if (it.part < 0) write_row<T, LPE, LPH, MODE, TILES>(c, s, it.row, tid, acc);
        else store_slot<LPE, LPH, MODE>(s, it.part, acc);
    }
    if (it.part < 0) return;   // uniform over the workgroup
    __syncthreads();           // the LDS sums are read; sum_slots writes them again

    const int sidx = s.part2split[it.part];
    const int p0 = s.split_off[sidx], p1 = s.split_off[sidx + 1];
    const int n = p1 - p0;
    if (n <= kCombineFan) {
        if (!arrive<LPE>(s, sidx, n, lds)) return;
        sum_slots<LPE, LPH, MODE>(s, p0, n, lds, acc);
    } else {
        const int g0 = s.split_grp[sidx];                 // first group of this row (groups are numbered over the view)
        const int ngrp = (n + kCombineFan - 1) / kCombineFan;
        const int g = (it.part - p0) / kCombineFan;
        const int gfirst = p0 + g * kCombineFan;
        const int gcount = min(kCombineFan, p1 - gfirst);
        if (!arrive<LPE>(s, s.n_split + g0 + g, gcount, lds)) return;
        sum_slots<LPE, LPH, MODE>(s, gfirst, gcount, lds, acc);
        if (tid < LPE) store_slot<LPE, LPH, MODE>(s, s.n_parts + g0 + g, acc);
        __syncthreads();
        if (!arrive<LPE>(s, sidx, ngrp, lds)) return;
        sum_slots<LPE, LPH, MODE>(s, s.n_parts + g0, ngrp, lds, acc);
    }
    if (tid < LPE) write_row<T, LPE, LPH, MODE, TILES>(c, s, it.row, tid, acc);
}

// Forward.  Workgroup b does what the records 4b .. 4b+3 say: one workgroup item, or four waves of
// rows.  Which rows meet in which workgroup, on which XCD and when is the plan's business.
template <typename T, int LPE, int LPH, int HASB, bool TILES>
__global__ __launch_bounds__(kBlock) void k_attn_fwd(const Common c, const SideArgs s,
                                                     const WaveRec<LPE>* __restrict__ recs) {
    __shared__ BlockLds<LPE> lds;
    const WaveRec<LPE>* r0 = recs + (int64_t)blockIdx.x * (kBlock / kWave);
    const RecLane rec = load_rec_lane<LPE, true>(r0[threadIdx.x >> 6]);      // in flight while the workgroup's code is looked at
    const uint32_t code0 = r0->code;
    if ((code0 & 7u) == kDescBlock) {          // uniform over the workgroup
        block_item<T, LPE, LPH, MODE_FWD, HASB, TILES>(c, s, r0->item, lds);
        return;
    }
    const uint32_t code = __builtin_amdgcn_readfirstlane(rec.code);
    if ((code & 7u) == kDescNone) return;
    wave_dispatch<T, LPE, LPH, MODE_FWD, HASB, TILES>(c, s, rec, code & 7u);
}

// Backward: both views in one launch (they are independent once nd is known); the record tells the view.
template <typename T, int LPE, int LPH, int HASB, bool TILES>
__global__ __launch_bounds__(kBlock, 4) void k_attn_bwd(const Common c, const SideArgs sd, const SideArgs ss,
                                                        const WaveRec<LPE>* __restrict__ recs) {
    __shared__ BlockLds<LPE> lds;
    constexpr int HB_D = HASB == 3 ? 2 : HASB;
    constexpr int HB_S = HASB == 3 ? 2 : (HASB ? 1 : 0);
    const WaveRec<LPE>* r0 = recs + (int64_t)blockIdx.x * (kBlock / kWave);
    const RecLane rec = load_rec_lane<LPE, sizeof(T) == 2>(r0[threadIdx.x >> 6]);      // in flight while the workgroup's code is looked at
    const uint32_t code0 = r0->code;
    if ((code0 & 7u) == kDescBlock) {          // uniform over the workgroup
        if (code0 & kDescSrcSide) block_item<T, LPE, LPH, MODE_BWD_SRC, HB_S, TILES>(c, ss, r0->item, lds);
        else block_item<T, LPE, LPH, MODE_BWD_DST, HB_D, TILES>(c, sd, r0->item, lds);
        return;
    }
    const uint32_t code = __builtin_amdgcn_readfirstlane(rec.code);
    if ((code & 7u) == kDescNone) return;
    if (code & kDescSrcSide) wave_dispatch<T, LPE, LPH, MODE_BWD_SRC, HB_S, TILES>(c, ss, rec, code & 7u);
    else wave_dispatch<T, LPE, LPH, MODE_BWD_DST, HB_D, TILES>(c, sd, rec, code & 7u);
}

// Per-node side vector of the backward: nd[i,h] = (1 / (Z[i,h] + eps), sum_c dout[i,h,c] out[i,h,c]).
template <typename T, int LPE, int LPH>
__global__ __launch_bounds__(kBlock) void k_node_side(const T* __restrict__ out, const T* __restrict__ dout,
                                                      const float* __restrict__ Z, int64_t N,
                                                      float2* __restrict__ nd) {
    constexpr int H = LPE / LPH;
    constexpr int HD = LPE * 8;
    constexpr int RPB = kBlock / LPE;   // rows per workgroup
    const int el = threadIdx.x % LPE;
    const int64_t row = (int64_t)blockIdx.x * RPB + threadIdx.x / LPE;
    const bool valid = row < N;
    float o[8], g[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) { o[i] = 0.f; g[i] = 0.f; }
    if (valid) {
        load8(out + row * HD + el * 8, o);
        load8(dout + row * HD + el * 8, g);
    }
    const float D = head_sum<LPH>(dot8(g, o));
    if (valid && el % LPH == 0) {
        const int h = el / LPH;
        nd[row * H + h] = make_float2(1.0f / (Z[row * H + h] + kEps), D);
    }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
static inline int64_t align256(int64_t x) { return (x + 255) & ~(int64_t)255; }

struct WsLayout {
    int64_t nd, fwd_part, dq_part, dkv_part, counters, total;
};
static WsLayout ws_layout(const tgt_plan* p, int H, int d) {
    const int64_t HD = (int64_t)H * d;
    WsLayout w;
    w.nd = 0;
    const int64_t slots_d = (int64_t)p->dst.n_parts + p->dst.n_groups, slots_s = (int64_t)p->src.n_parts + p->src.n_groups;
    const int64_t cnt_d = (int64_t)p->dst.n_split + p->dst.n_groups, cnt_s = (int64_t)p->src.n_split + p->src.n_groups;
    w.fwd_part = align256(p->N * H * 8);
    w.dq_part = w.fwd_part + align256(slots_d * (HD + H) * 4);
    w.dkv_part = w.dq_part + align256(slots_d * HD * 4);
    w.counters = w.dkv_part + align256(slots_s * 2 * HD * 4);
    w.total = w.counters + align256((2 * cnt_d + cnt_s + 1) * 4);
    return w;
}

static void fill_side(SideArgs& a, const Side& s) {
    a.items = s.items; a.col = s.col; a.eid = s.eid;
    a.split_off = s.split_off; a.part2split = s.part2split; a.split_grp = s.split_grp;
    a.n_split = s.n_split; a.n_parts = s.n_parts;
}
// shapes for which the variant that adds the block path's tile sums is compiled
template <int LPE, int LPH>
constexpr bool kTilesShape = (LPE == 8 && LPH == 1) || (LPE == 8 && LPH == 2) || (LPE == 16 && LPH == 2) ||
                             (LPE == 2 && LPH == 1);

struct Call {
    const tgt_plan* plan;
    const void *q, *k, *v, *bias;
    int bias_mode, H, d;
    const void *out, *dout;
    const float* Z;
    void *o_out, *dq, *dk, *dv, *dbias;
    float* o_Z;
    char* ws;
    hipStream_t st;
    const TileInit* init;
    bool skip_node_side;   // nd was already computed into the workspace by sparse_attn_node_side
    bool only_node_side;
    float* fwd_part;       // forward only: partial slots and arrival counters somewhere else than in `ws`
    int32_t* fwd_counters;
    bool no_alloc;         // fail instead of building the launch descriptors of a shape seen for the first time
};

template <typename T, int LPE, int LPH>
static int run_fwd(const Call& c) {
    const WsLayout L = ws_layout(c.plan, c.H, c.d);
    Common cm{};
    cm.q = c.q; cm.k = c.k; cm.v = c.v; cm.g = nullptr; cm.bias = c.bias; cm.bias_src = c.bias; cm.nd = nullptr;
    cm.bias_mode = c.bias_mode;
    cm.bias_se = (c.bias_mode & 0xf) == TGT_BIAS_EDGE_HEAD ? c.H : 1;
    cm.bias_sh = (c.bias_mode & 0xf) == TGT_BIAS_EDGE_HEAD ? 1 : 0;
    cm.inv_scale = 1.0f / sqrtf((float)c.d);
    SideArgs a{};
    fill_side(a, c.plan->dst);
    const Schedule* sch = c.no_alloc ? plan_schedule_if_ready(c.plan, LPE) : plan_schedule(c.plan, LPE, c.st);
    if (!sch) {
        if (c.no_alloc) {
            set_error("no launch descriptors for H*d = %d yet: call tgt_plan_prepare(plan, H, d, stream) first", LPE * 8);
            return TGT_ERR_INVALID_ARG;
        }
        return TGT_ERR_HIP;
    }
    const WaveRec<LPE>* desc = static_cast<const WaveRec<LPE>*>(sch->fwd);
    if (c.bias_mode & TGT_BIAS_PLAN_ORDER) a.eid = nullptr;             // bias rows in destination-sorted order
    a.out0 = c.o_out; a.out1 = nullptr; a.Z = c.o_Z;
    if (c.init) { a.init0 = c.init->acc; a.initZ = c.init->Z; a.cover = c.init->cover_dst; }
    a.part = c.fwd_part ? c.fwd_part : reinterpret_cast<float*>(c.ws + L.fwd_part);
    a.counters = c.fwd_counters ? c.fwd_counters : reinterpret_cast<int32_t*>(c.ws + L.counters);
    const int nb = sch->fwd_blocks;
    if (nb > 0) {
        KernelTimer t(KS_FWD, c.st, !c.no_alloc);       // the entry point that allocates nothing creates no events either
        const bool hb = c.bias_mode != TGT_BIAS_NONE;
        if (c.init != nullptr && (c.bias_mode & TGT_BIAS_PLAN_ORDER)) {
            set_error("block attention takes the bias in the caller's edge order");
            return TGT_ERR_UNSUPPORTED;
        }
        if (c.init != nullptr) {
            if constexpr (kTilesShape<LPE, LPH>) {
                if (hb) hipLaunchKernelGGL((k_attn_fwd<T, LPE, LPH, 1, true>), dim3(nb), dim3(kBlock), 0, c.st, cm, a, desc);
                else hipLaunchKernelGGL((k_attn_fwd<T, LPE, LPH, 0, true>), dim3(nb), dim3(kBlock), 0, c.st, cm, a, desc);
            } else {
                set_error("block attention: no kernel for this (H, d)");
                return TGT_ERR_UNSUPPORTED;
            }
        } else if (hb && (c.bias_mode & TGT_BIAS_PLAN_ORDER)) {
            hipLaunchKernelGGL((k_attn_fwd<T, LPE, LPH, 2, false>), dim3(nb), dim3(kBlock), 0, c.st, cm, a, desc);
        } else if (hb) {
            hipLaunchKernelGGL((k_attn_fwd<T, LPE, LPH, 1, false>), dim3(nb), dim3(kBlock), 0, c.st, cm, a, desc);
        } else {
            hipLaunchKernelGGL((k_attn_fwd<T, LPE, LPH, 0, false>), dim3(nb), dim3(kBlock), 0, c.st, cm, a, desc);
        }
    }
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

template <typename T, int LPE, int LPH>
static int run_bwd(const Call& c) {
    const WsLayout L = ws_layout(c.plan, c.H, c.d);
    const int64_t N = c.plan->N;
    float2* nd = reinterpret_cast<float2*>(c.ws + L.nd);
    if (!c.skip_node_side) {
        constexpr int RPB = kBlock / LPE;
        const int nb = (int)((N + RPB - 1) / RPB);
        KernelTimer t(KS_NODE_SIDE, c.st);
        hipLaunchKernelGGL((k_node_side<T, LPE, LPH>), dim3(nb), dim3(kBlock), 0, c.st,
                           static_cast<const T*>(c.out), static_cast<const T*>(c.dout), c.Z, N, nd);
        TGT_HIP_CHECK(hipGetLastError());
    }
    if (c.only_node_side) return TGT_OK;
    Common cm{};
    cm.q = c.q; cm.k = c.k; cm.v = c.v; cm.g = c.dout; cm.bias = c.bias; cm.nd = nd;
    const bool both_orders = (c.bias_mode & TGT_BIAS_BOTH_ORDERS) != 0;
    // two copies: rows [0, E) destination-sorted, rows [E, 2E) source-sorted
    cm.bias_src = both_orders ? static_cast<const char*>(c.bias) +
                                    (size_t)c.plan->E * ((c.bias_mode & 0xf) == TGT_BIAS_EDGE_HEAD ? c.H : 1) * sizeof(T)
                              : c.bias;
    cm.bias_mode = c.bias_mode;
    cm.bias_se = (c.bias_mode & 0xf) == TGT_BIAS_EDGE_HEAD ? c.H : 1;
    cm.bias_sh = (c.bias_mode & 0xf) == TGT_BIAS_EDGE_HEAD ? 1 : 0;
    cm.inv_scale = 1.0f / sqrtf((float)c.d);
    int32_t* counters = reinterpret_cast<int32_t*>(c.ws + L.counters);
    SideArgs sd{}, ss{};
    fill_side(sd, c.plan->dst);
    const Schedule* sch = plan_schedule(c.plan, LPE, c.st);
    if (!sch) return TGT_ERR_HIP;
    const WaveRec<LPE>* desc = static_cast<const WaveRec<LPE>*>(sch->bwd);
    if (c.bias_mode & TGT_BIAS_PLAN_ORDER) sd.eid = nullptr;
    sd.out0 = c.dq; sd.out1 = c.dbias; sd.Z = nullptr;
    if (c.init) { sd.init0 = c.init->dq; sd.cover = c.init->cover_dst; }
    sd.part = reinterpret_cast<float*>(c.ws + L.dq_part);
    sd.counters = counters + c.plan->dst.n_split + c.plan->dst.n_groups;
    fill_side(ss, c.plan->src);
    if (c.bias_mode & TGT_BIAS_PLAN_ORDER) { ss.eid = c.plan->src.pos; ss.eid_is_map = 1; }   // source-sorted -> destination-sorted position
    if (c.bias_mode & TGT_BIAS_BOTH_ORDERS) ss.eid = nullptr;           // its own source-sorted copy
    ss.out0 = c.dk; ss.out1 = c.dv; ss.Z = nullptr;
    if (c.init) { ss.init0 = c.init->dk; ss.init1 = c.init->dv; ss.cover = c.init->cover_src; }
    ss.part = reinterpret_cast<float*>(c.ws + L.dkv_part);
    ss.counters = counters + 2 * (c.plan->dst.n_split + c.plan->dst.n_groups);
    const int nb = sch->bwd_blocks;
    if (nb > 0) {
        KernelTimer t(KS_BWD, c.st);
        const bool hb = c.bias_mode != TGT_BIAS_NONE;
        if (c.init != nullptr && (c.bias_mode & TGT_BIAS_PLAN_ORDER)) {
            set_error("block attention takes the bias in the caller's edge order");
            return TGT_ERR_UNSUPPORTED;
        }
        if (c.init != nullptr) {
            if constexpr (kTilesShape<LPE, LPH>) {
                if (hb) hipLaunchKernelGGL((k_attn_bwd<T, LPE, LPH, 1, true>), dim3(nb), dim3(kBlock), 0, c.st, cm, sd, ss, desc);
                else hipLaunchKernelGGL((k_attn_bwd<T, LPE, LPH, 0, true>), dim3(nb), dim3(kBlock), 0, c.st, cm, sd, ss, desc);
            } else {
                set_error("block attention: no kernel for this (H, d)");
                return TGT_ERR_UNSUPPORTED;
            }
        } else if (hb && (c.bias_mode & TGT_BIAS_BOTH_ORDERS)) {
            hipLaunchKernelGGL((k_attn_bwd<T, LPE, LPH, 3, false>), dim3(nb), dim3(kBlock), 0, c.st, cm, sd, ss, desc);
        } else if (hb && (c.bias_mode & TGT_BIAS_PLAN_ORDER)) {
            hipLaunchKernelGGL((k_attn_bwd<T, LPE, LPH, 2, false>), dim3(nb), dim3(kBlock), 0, c.st, cm, sd, ss, desc);
        } else if (hb) {
            hipLaunchKernelGGL((k_attn_bwd<T, LPE, LPH, 1, false>), dim3(nb), dim3(kBlock), 0, c.st, cm, sd, ss, desc);
        } else {
            hipLaunchKernelGGL((k_attn_bwd<T, LPE, LPH, 0, false>), dim3(nb), dim3(kBlock), 0, c.st, cm, sd, ss, desc);
        }
    }
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

// The kernels of one (lanes per edge, lanes per head) shape take minutes to compile, so this file can be
// compiled as several translation units: -DTGT_SPARSE_PART=k (k = 0..3) emits the shapes of part k only, and
// part 0 also holds the entry points.  Without the macro one translation unit holds everything.
template <typename T, int LPE, int LPH> int run_shape(const Call& c, bool bwd);
#define TGT_DECLARE_SHAPE(LPE_, LPH_)                                      \
    template <> int run_shape<float, LPE_, LPH_>(const Call& c, bool bwd); \
    template <> int run_shape<bf16_t, LPE_, LPH_>(const Call& c, bool bwd);
#define TGT_DEFINE_SHAPE(LPE_, LPH_)                                                        \
    template <> int run_shape<float, LPE_, LPH_>(const Call& c, bool bwd) {                 \
        return bwd ? run_bwd<float, LPE_, LPH_>(c) : run_fwd<float, LPE_, LPH_>(c);         \
    }                                                                                       \
    template <> int run_shape<bf16_t, LPE_, LPH_>(const Call& c, bool bwd) {                \
        return bwd ? run_bwd<bf16_t, LPE_, LPH_>(c) : run_fwd<bf16_t, LPE_, LPH_>(c);       \
    }
TGT_DECLARE_SHAPE(8, 1)    // H=8  d=8   (Graphormer-Slim / GT node level, hidden 64)
#ifndef TGT_ONLY_8x8       // -DTGT_ONLY_8x8: compile one shape only (quick experiments)
TGT_DECLARE_SHAPE(8, 2)    // H=4  d=16  (attention micro-benchmark, attn_module.py:387)
TGT_DECLARE_SHAPE(16, 2)   // H=8  d=16  (hidden 128, the parser default)
TGT_DECLARE_SHAPE(16, 1)   // H=16 d=8
TGT_DECLARE_SHAPE(4, 1)    // H=4  d=8
TGT_DECLARE_SHAPE(2, 1)    // H=2  d=8
TGT_DECLARE_SHAPE(1, 1)    // H=1  d=8
TGT_DECLARE_SHAPE(4, 2)    // H=2  d=16
TGT_DECLARE_SHAPE(2, 2)    // H=1  d=16
TGT_DECLARE_SHAPE(16, 4)   // H=4  d=32  (hidden 128 with 4 heads)
TGT_DECLARE_SHAPE(8, 4)    // H=2  d=32
TGT_DECLARE_SHAPE(4, 4)    // H=1  d=32
#endif
#if !defined(TGT_SPARSE_PART) || TGT_SPARSE_PART == 0
TGT_DEFINE_SHAPE(8, 1)
#ifndef TGT_ONLY_8x8
TGT_DEFINE_SHAPE(1, 1)
TGT_DEFINE_SHAPE(16, 4)
#endif
#endif
#ifndef TGT_ONLY_8x8
#if !defined(TGT_SPARSE_PART) || TGT_SPARSE_PART == 1
TGT_DEFINE_SHAPE(8, 2)
TGT_DEFINE_SHAPE(4, 2)
TGT_DEFINE_SHAPE(8, 4)
#endif
#if !defined(TGT_SPARSE_PART) || TGT_SPARSE_PART == 2
TGT_DEFINE_SHAPE(16, 2)
TGT_DEFINE_SHAPE(2, 2)
TGT_DEFINE_SHAPE(4, 4)
#endif
#if !defined(TGT_SPARSE_PART) || TGT_SPARSE_PART == 3
TGT_DEFINE_SHAPE(2, 1)
TGT_DEFINE_SHAPE(16, 1)
TGT_DEFINE_SHAPE(4, 1)
#endif
#endif
#undef TGT_DECLARE_SHAPE
#undef TGT_DEFINE_SHAPE

#if !defined(TGT_SPARSE_PART) || TGT_SPARSE_PART == 0
template <typename T>
static int dispatch(const Call& c, bool bwd) {
    const int lph = c.d / 8, lpe = c.H * c.d / 8;
#define TGT_CASE(LPE_, LPH_) \
    if (lpe == LPE_ && lph == LPH_) return run_shape<T, LPE_, LPH_>(c, bwd);
    TGT_CASE(8, 1)
#ifndef TGT_ONLY_8x8
    TGT_CASE(8, 2)
    TGT_CASE(16, 2)
    TGT_CASE(16, 1)
    TGT_CASE(4, 1)
    TGT_CASE(2, 1)
    TGT_CASE(1, 1)
    TGT_CASE(4, 2)
    TGT_CASE(2, 2)
    TGT_CASE(16, 4)
    TGT_CASE(8, 4)
    TGT_CASE(4, 4)
#endif
#undef TGT_CASE
    set_error("no kernel for H=%d d=%d (d must be 8, 16 or 32 and H*d/8 one of 1,2,4,8,16, at least d/8)", c.H, c.d);
    return TGT_ERR_UNSUPPORTED;
}

static int check_common(const tgt_plan* plan, const void* q, const void* k, const void* v, const void* bias,
                        int bias_mode, int H, int d, int dtype, const void* ws, int64_t ws_bytes, bool needs_ws = true) {
    if (!plan || !q || !k || !v) { set_error("null plan or q/k/v"); return TGT_ERR_INVALID_ARG; }
    {
        const int base = bias_mode & 0xf;
        if (bias_mode < 0 || (bias_mode & ~(0xf | TGT_BIAS_PLAN_ORDER | TGT_BIAS_BOTH_ORDERS)) || base > TGT_BIAS_EDGE ||
            (base == TGT_BIAS_NONE && bias_mode != TGT_BIAS_NONE) ||
            ((bias_mode & TGT_BIAS_BOTH_ORDERS) && !(bias_mode & TGT_BIAS_PLAN_ORDER))) {
            set_error("bad bias_mode %d", bias_mode);
            return TGT_ERR_INVALID_ARG;
        }
        if ((bias_mode & TGT_BIAS_PLAN_ORDER) && !(bias_mode & TGT_BIAS_BOTH_ORDERS) && !plan->src.pos) {
            set_error("TGT_BIAS_PLAN_ORDER needs tgt_plan_enable_bias_order(plan) first");
            return TGT_ERR_INVALID_ARG;
        }
    }
    if (bias_mode != TGT_BIAS_NONE && !bias && plan->E > 0) { set_error("bias_mode %d needs a bias pointer", bias_mode); return TGT_ERR_INVALID_ARG; }
    if (dtype != TGT_DTYPE_F32 && dtype != TGT_DTYPE_BF16) { set_error("bad dtype %d", dtype); return TGT_ERR_INVALID_ARG; }
    if (H < 1 || d < 1) { set_error("H and d must be positive"); return TGT_ERR_INVALID_ARG; }
    if (d % 8 != 0) { set_error("head dim %d is not a multiple of 8", d); return TGT_ERR_UNSUPPORTED; }
    const int64_t need = needs_ws ? ws_layout(plan, H, d).total : 0;
    if (need > 0 && (!ws || ws_bytes < need || (reinterpret_cast<uintptr_t>(ws) & 255u))) {
        set_error("workspace: need %lld bytes, 256-byte aligned; got %lld", (long long)need, (long long)ws_bytes);
        return TGT_ERR_WORKSPACE;
    }
    return TGT_OK;
}

int sparse_attn_fwd_impl(const tgt_plan_t* plan, const void* d_q, const void* d_k, const void* d_v,
                         const void* d_bias, int bias_mode, int H, int d, int dtype, void* d_out, float* d_Z,
                         void* d_workspace, int64_t workspace_bytes, void* stream, const TileInit* init) {
    int rc = check_common(plan, d_q, d_k, d_v, d_bias, bias_mode, H, d, dtype, d_workspace, workspace_bytes);
    if (rc) return rc;
    if (!d_out || !d_Z) { set_error("null out or Z"); return TGT_ERR_INVALID_ARG; }
    Call c{};
    c.plan = plan; c.q = d_q; c.k = d_k; c.v = d_v; c.bias = d_bias; c.bias_mode = bias_mode;
    c.H = H; c.d = d; c.o_out = d_out; c.o_Z = d_Z; c.ws = static_cast<char*>(d_workspace);
    c.st = static_cast<hipStream_t>(stream);
    c.init = init;
    return dtype == TGT_DTYPE_F32 ? dispatch<float>(c, false) : dispatch<bf16_t>(c, false);
}

int sparse_attn_bwd_impl(const tgt_plan_t* plan, const void* d_q, const void* d_k, const void* d_v,
                         const void* d_bias, int bias_mode, int H, int d, int dtype, const void* d_out,
                         const float* d_Z, const void* d_dout, void* d_dq, void* d_dk, void* d_dv,
                         void* d_dbias, void* d_workspace, int64_t workspace_bytes, void* stream,
                         const TileInit* init, bool skip_node_side) {
    int rc = check_common(plan, d_q, d_k, d_v, d_bias, bias_mode, H, d, dtype, d_workspace, workspace_bytes);
    if (rc) return rc;
    if (!d_out || !d_Z || !d_dout || !d_dq || !d_dk || !d_dv) {
        set_error("null out/Z/dout/dq/dk/dv");
        return TGT_ERR_INVALID_ARG;
    }
    Call c{};
    c.plan = plan; c.q = d_q; c.k = d_k; c.v = d_v; c.bias = d_bias; c.bias_mode = bias_mode;
    c.H = H; c.d = d; c.out = d_out; c.Z = d_Z; c.dout = d_dout;
    c.dq = d_dq; c.dk = d_dk; c.dv = d_dv; c.dbias = (bias_mode == TGT_BIAS_NONE) ? nullptr : d_dbias;
    c.ws = static_cast<char*>(d_workspace);
    c.st = static_cast<hipStream_t>(stream);
    c.init = init;
    c.skip_node_side = skip_node_side;
    return dtype == TGT_DTYPE_F32 ? dispatch<float>(c, true) : dispatch<bf16_t>(c, true);
}

int sparse_attn_node_side(const tgt_plan_t* plan, int H, int d, int dtype, const void* d_out, const float* d_Z,
                          const void* d_dout, void* d_workspace, void* stream) {
    Call c{};
    c.plan = plan; c.H = H; c.d = d; c.out = d_out; c.Z = d_Z; c.dout = d_dout;
    c.ws = static_cast<char*>(d_workspace);
    c.st = static_cast<hipStream_t>(stream);
    c.only_node_side = true;
    return dtype == TGT_DTYPE_F32 ? dispatch<float>(c, true) : dispatch<bf16_t>(c, true);
}

const float2* sparse_attn_nd_ptr(void* d_workspace) { return reinterpret_cast<const float2*>(d_workspace); }

// ---------------------------------------------------------------------------
// forward that allocates nothing: partial slots and arrival counters of split rows in a fixed array
// ---------------------------------------------------------------------------
constexpr int64_t kScratchBytes = 4ll << 20;      // per GPU, held until the process ends
constexpr int kMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
// `scratch` is a host-side stand-in in host code, not a device address: the address of each GPU's copy
// is looked up once per device and used from then on.
static void* g_scratch_ptr[kMaxDevices];
static std::mutex g_scratch_mutex;

static int scratch_for_current_device(void** out) {
    int dev = 0;
    TGT_HIP_CHECK(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) { set_error("device %d: at most %d devices", dev, kMaxDevices); return TGT_ERR_UNSUPPORTED; }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        TGT_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return TGT_OK;
}

__global__ void k_zero_i32(int32_t* __restrict__ p, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}

int sparse_attn_fwd_noalloc_impl(const tgt_plan_t* plan, const void* d_q, const void* d_k, const void* d_v,
                                 const void* d_bias, int bias_mode, int H, int d, int dtype, void* d_out, float* d_Z,
                                 void* stream) {
    int rc = check_common(plan, d_q, d_k, d_v, d_bias, bias_mode, H, d, dtype, nullptr, 0, false);
    if (rc) return rc;
    if (!d_out || !d_Z) { set_error("null out or Z"); return TGT_ERR_INVALID_ARG; }
    int dev = 0;
    TGT_HIP_CHECK(hipGetDevice(&dev));
    if (dev != plan->device) { set_error("the plan lives on device %d, the current device is %d", plan->device, dev); return TGT_ERR_INVALID_ARG; }
    // scratch layout: arrival counters (rows, then groups), then the partial slots
    const int64_t n_cnt = (int64_t)plan->dst.n_split + plan->dst.n_groups;
    const int64_t slots = (int64_t)plan->dst.n_parts + plan->dst.n_groups;
    const int64_t part_off = align256(n_cnt * 4);
    const int64_t need = part_off + slots * ((int64_t)H * d + H) * 4;
    if (need > kScratchBytes) {
        set_error("tgt_sparse_attn_fwd_noalloc: the split rows of this graph need %lld bytes of scratch, the fixed array holds %lld; "
                  "use tgt_sparse_attn_fwd with a workspace", (long long)need, (long long)kScratchBytes);
        return TGT_ERR_WORKSPACE;
    }
    void* base = nullptr;
    rc = scratch_for_current_device(&base);
    if (rc) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (n_cnt > 0) {   // the array keeps what the last call left: the counters must start at zero
        hipLaunchKernelGGL(k_zero_i32, dim3((unsigned)((n_cnt + 255) / 256)), dim3(256), 0, st,
                           static_cast<int32_t*>(base), (int)n_cnt);
        TGT_HIP_CHECK(hipGetLastError());
    }
    Call c{};
    c.plan = plan; c.q = d_q; c.k = d_k; c.v = d_v; c.bias = d_bias; c.bias_mode = bias_mode;
    c.H = H; c.d = d; c.o_out = d_out; c.o_Z = d_Z; c.ws = nullptr;
    c.st = st;
    c.fwd_counters = static_cast<int32_t*>(base);
    c.fwd_part = reinterpret_cast<float*>(static_cast<char*>(base) + part_off);
    c.no_alloc = true;
    return dtype == TGT_DTYPE_F32 ? dispatch<float>(c, false) : dispatch<bf16_t>(c, false);
}
#endif  // part 0: dispatch and entry points

}  // namespace tgt

#if !defined(TGT_SPARSE_PART) || TGT_SPARSE_PART == 0
// A plan made by tgt_plan_create_remaining schedules no row without edges: only the block path, whose tile
// kernels write those rows, may run it.
static int refuse_remaining(const tgt_plan_t* plan) {
    if (plan && plan->rows_with_edges_only) {
        tgt::set_error("this plan holds the edges beside a tile set (tgt_plan_create_remaining): use tgt_block_attn_*");
        return TGT_ERR_INVALID_ARG;
    }
    return TGT_OK;
}

extern "C" {

int64_t tgt_sparse_attn_workspace_bytes(const tgt_plan_t* plan, int H, int d) {
    if (!plan || H < 1 || d < 1) return -1;
    return tgt::ws_layout(plan, H, d).total;
}

int tgt_sparse_attn_fwd(const tgt_plan_t* plan, const void* d_q, const void* d_k, const void* d_v,
                        const void* d_bias, int bias_mode, int H, int d, int dtype, void* d_out, float* d_Z,
                        void* d_workspace, int64_t workspace_bytes, void* stream) {
    if (int rc = refuse_remaining(plan)) return rc;
    return tgt::sparse_attn_fwd_impl(plan, d_q, d_k, d_v, d_bias, bias_mode, H, d, dtype, d_out, d_Z, d_workspace,
                                     workspace_bytes, stream, nullptr);
}

int tgt_sparse_attn_fwd_noalloc(const tgt_plan_t* plan, const void* d_q, const void* d_k, const void* d_v,
                                const void* d_bias, int bias_mode, int H, int d, int dtype, void* d_out, float* d_Z,
                                void* stream) {
    if (int rc = refuse_remaining(plan)) return rc;
    return tgt::sparse_attn_fwd_noalloc_impl(plan, d_q, d_k, d_v, d_bias, bias_mode, H, d, dtype, d_out, d_Z, stream);
}

int tgt_plan_prepare(tgt_plan_t* plan, int H, int d, void* stream) {
    if (!plan || H < 1 || d < 1 || (H * d) % 8) { tgt::set_error("tgt_plan_prepare: null plan or H*d not a multiple of 8"); return TGT_ERR_INVALID_ARG; }
    return tgt::plan_schedule(plan, H * d / 8, static_cast<hipStream_t>(stream)) ? TGT_OK : TGT_ERR_UNSUPPORTED;
}

int tgt_sparse_attn_bwd(const tgt_plan_t* plan, const void* d_q, const void* d_k, const void* d_v,
                        const void* d_bias, int bias_mode, int H, int d, int dtype, const void* d_out,
                        const float* d_Z, const void* d_dout, void* d_dq, void* d_dk, void* d_dv,
                        void* d_dbias, void* d_workspace, int64_t workspace_bytes, void* stream) {
    if (int rc = refuse_remaining(plan)) return rc;
    return tgt::sparse_attn_bwd_impl(plan, d_q, d_k, d_v, d_bias, bias_mode, H, d, dtype, d_out, d_Z, d_dout, d_dq,
                                     d_dk, d_dv, d_dbias, d_workspace, workspace_bytes, stream, nullptr, false);
}

}  // extern "C"
#endif  // part 0: C entry points
