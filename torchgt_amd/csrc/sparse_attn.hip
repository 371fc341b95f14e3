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
// share a wave, long rows use the whole wave, rows longer than kSegLen are split
// into segments whose partial sums a small second kernel adds in a fixed order.
#include "common.h"

namespace tgt {

struct bf16_t { uint16_t x; };

__device__ __forceinline__ float bf16_to_f32(uint32_t bits16) { return __uint_as_float(bits16 << 16); }
__device__ __forceinline__ uint32_t f32_to_bf16(float f) {   // round to nearest even, NaN kept quiet
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
    return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
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
__device__ __forceinline__ float load1(const float* p) { return *p; }
__device__ __forceinline__ float load1(const bf16_t* p) { return bf16_to_f32(p->x); }
__device__ __forceinline__ void store1(float* p, float v) { *p = v; }
__device__ __forceinline__ void store1(bf16_t* p, float v) { p->x = (uint16_t)f32_to_bf16(v); }

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

__host__ __device__ constexpr int slots_for_class(int lpe, int cls) {
    // natural slot count of the length classes (>32, <=32, <=16, <=8, <=4), capped by the wave
    const int nat = cls == 0 ? 16 : (cls == 1 ? 8 : (cls == 2 ? 4 : (cls == 3 ? 2 : 1)));
    const int cap = kWave / lpe;
    return nat < cap ? nat : cap;
}

// Which walk a launch performs.
enum { MODE_FWD = 0, MODE_BWD_DST = 1, MODE_BWD_SRC = 2 };

struct WalkArgs {
    // row-side and edge-side node features; meaning depends on the mode
    const void* q;
    const void* k;
    const void* v;
    const void* g;        // dout (backward)
    const void* bias;
    const float2* nd;     // [N, H] (1/(Z+eps), D) (backward)
    const Item* items;
    const int32_t* col;
    const int32_t* eid;
    void* out0;           // fwd: out      bwd_dst: dq     bwd_src: dk
    void* out1;           // fwd: -        bwd_dst: dbias  bwd_src: dv
    float* Z;             // fwd: Z
    float* part;          // partial slots of split rows
    int32_t class_off[kNumClass + 1];
    int32_t wave_off[kNumClass + 1];
    int32_t n_parts;
    int32_t bias_mode;
    float inv_scale;
};

template <typename T, int LPE, int LPH, int S, int MODE>
__device__ __forceinline__ void walk_items(const WalkArgs& a, const int item_begin, const int item_end,
                                           const int wave_in_class) {
    constexpr int G = LPE * S;        // lanes per item
    constexpr int IPW = kWave / G;    // items per wave
    constexpr int H = LPE / LPH;
    constexpr int HD = LPE * 8;
    const int lane = threadIdx.x & (kWave - 1);
    const int sub = lane / G;
    const int gl = lane % G;
    const int slot = gl / LPE;
    const int el = gl % LPE;
    const int head = el / LPH;
    const int item = item_begin + wave_in_class * IPW + sub;
    const bool valid = item < item_end;
    Item it{0, 0, 0, -1};
    if (valid) it = a.items[item];

    const T* __restrict__ Q = static_cast<const T*>(a.q);
    const T* __restrict__ K = static_cast<const T*>(a.k);
    const T* __restrict__ V = static_cast<const T*>(a.v);
    const T* __restrict__ Gd = static_cast<const T*>(a.g);
    const T* __restrict__ B = static_cast<const T*>(a.bias);
    const int64_t row_off = (int64_t)it.row * HD + el * 8;

    // row-resident operands
    float r0[8], r1[8];      // fwd: q | bwd_dst: q, g | bwd_src: k, v
    float rz = 0.f, Dh = 0.f;
#pragma unroll
    for (int c = 0; c < 8; ++c) { r0[c] = 0.f; r1[c] = 0.f; }
    if (valid) {
        if (MODE == MODE_FWD) {
            load8(Q + row_off, r0);
        } else if (MODE == MODE_BWD_DST) {
            load8(Q + row_off, r0);
            load8(Gd + row_off, r1);
            const float2 nd = a.nd[(int64_t)it.row * H + head];
            rz = nd.x; Dh = nd.y;
        } else {
            load8(K + row_off, r0);
            load8(V + row_off, r1);
        }
    }
    float acc0[8], acc1[8];  // fwd: sum w v | bwd_dst: dq | bwd_src: dk, dv
    float z = 0.f;
#pragma unroll
    for (int c = 0; c < 8; ++c) { acc0[c] = 0.f; acc1[c] = 0.f; }

    const int32_t* __restrict__ col = a.col + it.start;
    const int32_t* __restrict__ eid = a.eid + it.start;
    const int bias_mode = a.bias_mode;
    const float inv_scale = a.inv_scale;

    for (int e0 = slot; e0 < it.len; e0 += S * kUnroll) {
        int nb[kUnroll], ed[kUnroll];
        bool ok[kUnroll];
        float x0[kUnroll][8], x1[kUnroll][8], bb[kUnroll];
        float2 ndv[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const int e = e0 + u * S;
            ok[u] = e < it.len;
            nb[u] = 0; ed[u] = 0;
            if (ok[u]) {
                nb[u] = col[e];
                if (bias_mode != TGT_BIAS_NONE) ed[u] = eid[e];
            }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            bb[u] = 0.f;
            ndv[u] = make_float2(0.f, 0.f);
#pragma unroll
            for (int c = 0; c < 8; ++c) { x0[u][c] = 0.f; x1[u][c] = 0.f; }
            if (ok[u]) {
                const int64_t o = (int64_t)nb[u] * HD + el * 8;
                if (MODE == MODE_BWD_SRC) {
                    load8(Q + o, x0[u]);
                    load8(Gd + o, x1[u]);
                    ndv[u] = a.nd[(int64_t)nb[u] * H + head];
                } else {
                    load8(K + o, x0[u]);
                    load8(V + o, x1[u]);
                }
                if (bias_mode == TGT_BIAS_EDGE_HEAD) bb[u] = load1(B + (int64_t)ed[u] * H + head);
                else if (bias_mode == TGT_BIAS_EDGE) bb[u] = load1(B + ed[u]);
            }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            if (ok[u]) {
                // raw score: identical arithmetic in all three walks so that the
                // recomputed weights and the clamp mask agree bit for bit
                const float raw = head_sum<LPH>(dot8(r0, x0[u])) * inv_scale;
                const float w = expf(clamp5(raw) + bb[u]);
                if (MODE == MODE_FWD) {
                    z += w;
#pragma unroll
                    for (int c = 0; c < 8; ++c) acc0[c] = fmaf(w, x1[u][c], acc0[c]);
                } else {
                    const bool inside = (raw >= -5.0f) & (raw <= 5.0f);   // torch clamp backward: inclusive
                    if (MODE == MODE_BWD_DST) {
                        const float t = head_sum<LPH>(dot8(r1, x1[u]));   // g_dst . v_src
                        const float dS = w * rz * (t - Dh);
                        T* __restrict__ dB = static_cast<T*>(a.out1);
                        if (dB != nullptr) {
                            if (bias_mode == TGT_BIAS_EDGE_HEAD) {
                                if (el % LPH == 0) store1(dB + (int64_t)ed[u] * H + head, dS);
                            } else if (bias_mode == TGT_BIAS_EDGE) {
                                float s = dS;   // sum over heads; every head is held by LPH lanes
#pragma unroll
                                for (int off = 1; off < LPE; off <<= 1) s += __shfl_xor(s, off);
                                if (el == 0) store1(dB + ed[u], s * (1.0f / LPH));
                            }
                        }
                        const float md = inside ? dS : 0.f;
#pragma unroll
                        for (int c = 0; c < 8; ++c) acc0[c] = fmaf(md, x0[u][c], acc0[c]);
                    } else {
                        const float p = w * ndv[u].x;
                        const float t = head_sum<LPH>(dot8(x1[u], r1));   // g_dst . v_src
                        const float dS = p * (t - ndv[u].y);
                        const float md = inside ? dS : 0.f;
#pragma unroll
                        for (int c = 0; c < 8; ++c) {
                            acc0[c] = fmaf(md, x0[u][c], acc0[c]);   // dk += m dS q_dst
                            acc1[c] = fmaf(p, x1[u][c], acc1[c]);    // dv += p g_dst
                        }
                    }
                }
            }
        }
    }

    // add the S edge slots of an item (all lanes take part)
#pragma unroll
    for (int off = LPE; off < G; off <<= 1) {
        if (MODE == MODE_FWD) z += __shfl_xor(z, off);
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            acc0[c] += __shfl_xor(acc0[c], off);
            if (MODE == MODE_BWD_SRC) acc1[c] += __shfl_xor(acc1[c], off);
        }
    }
    if (!valid || slot != 0) return;

    if (MODE != MODE_FWD) {
#pragma unroll
        for (int c = 0; c < 8; ++c) acc0[c] *= inv_scale;
    }
    if (it.part < 0) {
        if (MODE == MODE_FWD) {
            const float den = z + kEps;
#pragma unroll
            for (int c = 0; c < 8; ++c) acc0[c] = acc0[c] / den;
            store8(static_cast<T*>(a.out0) + row_off, acc0);
            if (el % LPH == 0) a.Z[(int64_t)it.row * H + head] = z;
        } else if (MODE == MODE_BWD_DST) {
            store8(static_cast<T*>(a.out0) + row_off, acc0);
        } else {
            store8(static_cast<T*>(a.out0) + row_off, acc0);
            store8(static_cast<T*>(a.out1) + row_off, acc1);
        }
    } else {
        // partial slot layout: fwd [n_parts][HD] then [n_parts][H]; bwd_dst [n_parts][HD];
        // bwd_src [n_parts][2][HD]
        if (MODE == MODE_FWD) {
            store8(a.part + (int64_t)it.part * HD + el * 8, acc0);
            if (el % LPH == 0) a.part[(int64_t)a.n_parts * HD + (int64_t)it.part * H + head] = z;
        } else if (MODE == MODE_BWD_DST) {
            store8(a.part + (int64_t)it.part * HD + el * 8, acc0);
        } else {
            store8(a.part + (int64_t)it.part * 2 * HD + el * 8, acc0);
            store8(a.part + (int64_t)it.part * 2 * HD + HD + el * 8, acc1);
        }
    }
}

template <typename T, int LPE, int LPH, int MODE>
__global__ __launch_bounds__(kBlock) void k_walk(const WalkArgs a) {
    const int gw = blockIdx.x * (kBlock / kWave) + (threadIdx.x >> 6);   // global wave index
    int cls = 0;
#pragma unroll
    for (int c = 1; c < kNumClass; ++c) cls += (gw >= a.wave_off[c]) ? 1 : 0;
    cls = __builtin_amdgcn_readfirstlane(cls);
    if (gw >= a.wave_off[kNumClass]) return;
    const int w = gw - a.wave_off[cls];
    const int b = a.class_off[cls], e = a.class_off[cls + 1];
    switch (cls) {
        case 0: walk_items<T, LPE, LPH, slots_for_class(LPE, 0), MODE>(a, b, e, w); break;
        case 1: walk_items<T, LPE, LPH, slots_for_class(LPE, 1), MODE>(a, b, e, w); break;
        case 2: walk_items<T, LPE, LPH, slots_for_class(LPE, 2), MODE>(a, b, e, w); break;
        case 3: walk_items<T, LPE, LPH, slots_for_class(LPE, 3), MODE>(a, b, e, w); break;
        default: walk_items<T, LPE, LPH, slots_for_class(LPE, 4), MODE>(a, b, e, w); break;
    }
}

// Adds the partial slots of every split row in slot order (fixed order ->
// reproducible) and writes the row.  One workgroup of 64 threads per split row.
template <typename T, int MODE>
__global__ __launch_bounds__(64) void k_combine(const int32_t* __restrict__ split_row,
                                                const int32_t* __restrict__ split_off,
                                                const float* __restrict__ part, int n_parts, int H, int d,
                                                void* out0, void* out1, float* Z) {
    const int r = blockIdx.x;
    const int row = split_row[r];
    const int p0 = split_off[r], p1 = split_off[r + 1];
    const int HD = H * d;
    for (int c = threadIdx.x; c < HD; c += 64) {
        if (MODE == MODE_FWD) {
            float acc = 0.f, z = 0.f;
            const int h = c / d;
            for (int p = p0; p < p1; ++p) {
                acc += part[(int64_t)p * HD + c];
                z += part[(int64_t)n_parts * HD + (int64_t)p * H + h];
            }
            store1(static_cast<T*>(out0) + (int64_t)row * HD + c, acc / (z + kEps));
            if (c % d == 0) Z[(int64_t)row * H + h] = z;
        } else if (MODE == MODE_BWD_DST) {
            float acc = 0.f;
            for (int p = p0; p < p1; ++p) acc += part[(int64_t)p * HD + c];
            store1(static_cast<T*>(out0) + (int64_t)row * HD + c, acc);
        } else {
            float a0 = 0.f, a1 = 0.f;
            for (int p = p0; p < p1; ++p) {
                a0 += part[(int64_t)p * 2 * HD + c];
                a1 += part[(int64_t)p * 2 * HD + HD + c];
            }
            store1(static_cast<T*>(out0) + (int64_t)row * HD + c, a0);
            store1(static_cast<T*>(out1) + (int64_t)row * HD + c, a1);
        }
    }
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
    for (int c = 0; c < 8; ++c) { o[c] = 0.f; g[c] = 0.f; }
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
    int64_t nd, fwd_part, dq_part, dkv_part, total;
};
static WsLayout ws_layout(const tgt_plan* p, int H, int d) {
    const int64_t HD = (int64_t)H * d;
    WsLayout w;
    w.nd = 0;
    w.fwd_part = align256(p->N * H * 8);
    w.dq_part = w.fwd_part + align256((int64_t)p->dst.n_parts * (HD + H) * 4);
    w.dkv_part = w.dq_part + align256((int64_t)p->dst.n_parts * HD * 4);
    w.total = w.dkv_part + align256((int64_t)p->src.n_parts * 2 * HD * 4);
    return w;
}

static void fill_schedule(WalkArgs& a, const Side& s, int lpe, int* n_blocks) {
    int waves = 0;
    for (int c = 0; c < kNumClass; ++c) {
        a.class_off[c] = s.class_off[c];
        a.wave_off[c] = waves;
        const int ipw = kWave / (lpe * slots_for_class(lpe, c));
        const int n = s.class_off[c + 1] - s.class_off[c];
        waves += (n + ipw - 1) / ipw;
    }
    a.class_off[kNumClass] = s.class_off[kNumClass];
    a.wave_off[kNumClass] = waves;
    a.n_parts = s.n_parts;
    *n_blocks = (waves + (kBlock / kWave) - 1) / (kBlock / kWave);
}

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
};

template <typename T, int LPE, int LPH>
static int run_fwd(const Call& c) {
    const WsLayout L = ws_layout(c.plan, c.H, c.d);
    WalkArgs a{};
    a.q = c.q; a.k = c.k; a.v = c.v; a.g = nullptr; a.bias = c.bias; a.nd = nullptr;
    a.items = c.plan->dst.items; a.col = c.plan->dst.col; a.eid = c.plan->dst.eid;
    a.out0 = c.o_out; a.out1 = nullptr; a.Z = c.o_Z;
    a.part = reinterpret_cast<float*>(c.ws + L.fwd_part);
    a.bias_mode = c.bias_mode;
    a.inv_scale = 1.0f / sqrtf((float)c.d);
    int nb = 0;
    fill_schedule(a, c.plan->dst, LPE, &nb);
    if (nb > 0) hipLaunchKernelGGL((k_walk<T, LPE, LPH, MODE_FWD>), dim3(nb), dim3(kBlock), 0, c.st, a);
    if (c.plan->dst.n_split > 0)
        hipLaunchKernelGGL((k_combine<T, MODE_FWD>), dim3(c.plan->dst.n_split), dim3(64), 0, c.st,
                           c.plan->dst.split_row, c.plan->dst.split_off, a.part, c.plan->dst.n_parts, c.H,
                           c.d, c.o_out, nullptr, c.o_Z);
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

template <typename T, int LPE, int LPH>
static int run_bwd(const Call& c) {
    const WsLayout L = ws_layout(c.plan, c.H, c.d);
    const int64_t N = c.plan->N;
    float2* nd = reinterpret_cast<float2*>(c.ws + L.nd);
    {
        constexpr int RPB = kBlock / LPE;
        const int nb = (int)((N + RPB - 1) / RPB);
        hipLaunchKernelGGL((k_node_side<T, LPE, LPH>), dim3(nb), dim3(kBlock), 0, c.st,
                           static_cast<const T*>(c.out), static_cast<const T*>(c.dout), c.Z, N, nd);
    }
    WalkArgs a{};
    a.q = c.q; a.k = c.k; a.v = c.v; a.g = c.dout; a.bias = c.bias; a.nd = nd;
    a.bias_mode = c.bias_mode;
    a.inv_scale = 1.0f / sqrtf((float)c.d);
    a.Z = nullptr;
    int nb = 0;
    // destination view: dq, dbias
    a.items = c.plan->dst.items; a.col = c.plan->dst.col; a.eid = c.plan->dst.eid;
    a.out0 = c.dq; a.out1 = c.dbias;
    a.part = reinterpret_cast<float*>(c.ws + L.dq_part);
    fill_schedule(a, c.plan->dst, LPE, &nb);
    if (nb > 0) hipLaunchKernelGGL((k_walk<T, LPE, LPH, MODE_BWD_DST>), dim3(nb), dim3(kBlock), 0, c.st, a);
    if (c.plan->dst.n_split > 0)
        hipLaunchKernelGGL((k_combine<T, MODE_BWD_DST>), dim3(c.plan->dst.n_split), dim3(64), 0, c.st,
                           c.plan->dst.split_row, c.plan->dst.split_off, a.part, c.plan->dst.n_parts, c.H,
                           c.d, c.dq, nullptr, nullptr);
    // source view: dk, dv
    a.items = c.plan->src.items; a.col = c.plan->src.col; a.eid = c.plan->src.eid;
    a.out0 = c.dk; a.out1 = c.dv;
    a.part = reinterpret_cast<float*>(c.ws + L.dkv_part);
    fill_schedule(a, c.plan->src, LPE, &nb);
    if (nb > 0) hipLaunchKernelGGL((k_walk<T, LPE, LPH, MODE_BWD_SRC>), dim3(nb), dim3(kBlock), 0, c.st, a);
    if (c.plan->src.n_split > 0)
        hipLaunchKernelGGL((k_combine<T, MODE_BWD_SRC>), dim3(c.plan->src.n_split), dim3(64), 0, c.st,
                           c.plan->src.split_row, c.plan->src.split_off, a.part, c.plan->src.n_parts, c.H,
                           c.d, c.dk, c.dv, nullptr);
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

template <typename T>
static int dispatch(const Call& c, bool bwd) {
    const int lph = c.d / 8, lpe = c.H * c.d / 8;
#define TGT_CASE(LPE_, LPH_)                                                   \
    if (lpe == LPE_ && lph == LPH_)                                            \
        return bwd ? run_bwd<T, LPE_, LPH_>(c) : run_fwd<T, LPE_, LPH_>(c);
    TGT_CASE(8, 1)    // H=8  d=8   (Graphormer-Slim / GT node level, hidden 64)
    TGT_CASE(8, 2)    // H=4  d=16  (attention micro-benchmark, attn_module.py:387)
    TGT_CASE(16, 2)   // H=8  d=16  (hidden 128, the parser default)
    TGT_CASE(16, 1)   // H=16 d=8
    TGT_CASE(4, 1)    // H=4  d=8
    TGT_CASE(2, 1)    // H=2  d=8
    TGT_CASE(1, 1)    // H=1  d=8
    TGT_CASE(4, 2)    // H=2  d=16
    TGT_CASE(2, 2)    // H=1  d=16
#undef TGT_CASE
    set_error("no kernel for H=%d d=%d (d must be 8 or 16 and H*d/8 one of 1,2,4,8,16)", c.H, c.d);
    return TGT_ERR_UNSUPPORTED;
}

static int check_common(const tgt_plan* plan, const void* q, const void* k, const void* v, const void* bias,
                        int bias_mode, int H, int d, int dtype, const void* ws, int64_t ws_bytes) {
    if (!plan || !q || !k || !v) { set_error("null plan or q/k/v"); return TGT_ERR_INVALID_ARG; }
    if (bias_mode < TGT_BIAS_NONE || bias_mode > TGT_BIAS_EDGE) { set_error("bad bias_mode %d", bias_mode); return TGT_ERR_INVALID_ARG; }
    if (bias_mode != TGT_BIAS_NONE && !bias && plan->E > 0) { set_error("bias_mode %d needs a bias pointer", bias_mode); return TGT_ERR_INVALID_ARG; }
    if (dtype != TGT_DTYPE_F32 && dtype != TGT_DTYPE_BF16) { set_error("bad dtype %d", dtype); return TGT_ERR_INVALID_ARG; }
    if (H < 1 || d < 1) { set_error("H and d must be positive"); return TGT_ERR_INVALID_ARG; }
    if (d % 8 != 0) { set_error("head dim %d is not a multiple of 8", d); return TGT_ERR_UNSUPPORTED; }
    const int64_t need = ws_layout(plan, H, d).total;
    if (need > 0 && (!ws || ws_bytes < need || (reinterpret_cast<uintptr_t>(ws) & 255u))) {
        set_error("workspace: need %lld bytes, 256-byte aligned; got %lld", (long long)need, (long long)ws_bytes);
        return TGT_ERR_WORKSPACE;
    }
    return TGT_OK;
}

}  // namespace tgt

extern "C" {

int64_t tgt_sparse_attn_workspace_bytes(const tgt_plan_t* plan, int H, int d) {
    if (!plan || H < 1 || d < 1) return -1;
    return tgt::ws_layout(plan, H, d).total;
}

int tgt_sparse_attn_fwd(const tgt_plan_t* plan, const void* d_q, const void* d_k, const void* d_v,
                        const void* d_bias, int bias_mode, int H, int d, int dtype, void* d_out, float* d_Z,
                        void* d_workspace, int64_t workspace_bytes, void* stream) {
    int rc = tgt::check_common(plan, d_q, d_k, d_v, d_bias, bias_mode, H, d, dtype, d_workspace, workspace_bytes);
    if (rc) return rc;
    if (!d_out || !d_Z) { tgt::set_error("null out or Z"); return TGT_ERR_INVALID_ARG; }
    tgt::Call c{};
    c.plan = plan; c.q = d_q; c.k = d_k; c.v = d_v; c.bias = d_bias; c.bias_mode = bias_mode;
    c.H = H; c.d = d; c.o_out = d_out; c.o_Z = d_Z; c.ws = static_cast<char*>(d_workspace);
    c.st = static_cast<hipStream_t>(stream);
    return dtype == TGT_DTYPE_F32 ? tgt::dispatch<float>(c, false) : tgt::dispatch<tgt::bf16_t>(c, false);
}

int tgt_sparse_attn_bwd(const tgt_plan_t* plan, const void* d_q, const void* d_k, const void* d_v,
                        const void* d_bias, int bias_mode, int H, int d, int dtype, const void* d_out,
                        const float* d_Z, const void* d_dout, void* d_dq, void* d_dk, void* d_dv,
                        void* d_dbias, void* d_workspace, int64_t workspace_bytes, void* stream) {
    int rc = tgt::check_common(plan, d_q, d_k, d_v, d_bias, bias_mode, H, d, dtype, d_workspace, workspace_bytes);
    if (rc) return rc;
    if (!d_out || !d_Z || !d_dout || !d_dq || !d_dk || !d_dv) {
        tgt::set_error("null out/Z/dout/dq/dk/dv");
        return TGT_ERR_INVALID_ARG;
    }
    tgt::Call c{};
    c.plan = plan; c.q = d_q; c.k = d_k; c.v = d_v; c.bias = d_bias; c.bias_mode = bias_mode;
    c.H = H; c.d = d; c.out = d_out; c.Z = d_Z; c.dout = d_dout;
    c.dq = d_dq; c.dk = d_dk; c.dv = d_dv; c.dbias = (bias_mode == TGT_BIAS_NONE) ? nullptr : d_dbias;
    c.ws = static_cast<char*>(d_workspace);
    c.st = static_cast<hipStream_t>(stream);
    return dtype == TGT_DTYPE_F32 ? tgt::dispatch<float>(c, true) : tgt::dispatch<tgt::bf16_t>(c, true);
}

}  // extern "C"
