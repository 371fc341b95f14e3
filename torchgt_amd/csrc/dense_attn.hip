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
// The bias tile is transposed through LDS so that its global reads are coalesced.
#include "common.h"

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

constexpr int kTilePad = 33;   // LDS row stride of a 32x32 fp32 tile (conflict-free transposed reads)

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

// dynamic LDS sizes (bytes)
template <int D, int NT> constexpr int fwd_lds_bytes() {
    return 2 * (rm_elems<D, NT * 32>() + tr_elems<D, NT * 32>()) + 4 * NT * 32 * kTilePad;
}
template <int D, int NT> constexpr int bwd_lds_bytes() {
    return 2 * (4 * rm_elems<D, NT * 32>() + 3 * tr_elems<D, NT * 32>()) + 4 * 2 * NT * 32 + 4 * NT * 32 * kTilePad;
}

// ---------------------------------------------------------------------------
// forward
// ---------------------------------------------------------------------------
template <typename T, int D, int NT>
__global__ __launch_bounds__(64 * NT) void k_dense_fwd(const T* __restrict__ Q, const T* __restrict__ K,
                                                       const T* __restrict__ V, const T* __restrict__ bias,
                                                       T* __restrict__ out, float* __restrict__ lse, int S,
                                                       int H, float scale) {
    constexpr int KS = D / 8;
    constexpr int SP = NT * 32;
    extern __shared__ __align__(16) char smem[];
    short* k_rm = reinterpret_cast<short*>(smem);
    short* v_tr = k_rm + rm_elems<D, SP>();
    float* bias_all = reinterpret_cast<float*>(v_tr + tr_elems<D, SP>());
    const int g = blockIdx.x / H, h = blockIdx.x % H;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int col = lane & 31, half = lane >> 5;
    float* bias_l = bias_all + wave * 32 * kTilePad;
    load_head<T, D, SP>(K, g, h, S, H, k_rm, nullptr);
    load_head<T, D, SP>(V, g, h, S, H, nullptr, v_tr);
    const int q0 = wave * 32, qi = q0 + col;
    short4_t bq[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        bq[s] = zero4();
        if (qi < S) bq[s] = ld4(Q + (((int64_t)g * S + qi) * H + h) * D + s * 8 + half * 4);
    }
    __syncthreads();
    float16_t acc[NT];
#pragma unroll
    for (int kt = 0; kt < NT; ++kt) {
        acc[kt] = zero16();
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            const short4_t a = *reinterpret_cast<const short4_t*>(&k_rm[(kt * 32 + col) * D + s * 8 + half * 4]);
            acc[kt] = mfma(a, bq[s], acc[kt]);
        }
    }
    // scale, bias (transposed through LDS), key padding
    float m = -INFINITY;
#pragma unroll
    for (int kt = 0; kt < NT; ++kt) {
        if (bias != nullptr) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = r * 2 + half, key = kt * 32 + col;
                float bv = 0.f;
                if (q0 + row < S && key < S)
                    bv = ld1(bias + (((int64_t)g * H + h) * S + q0 + row) * S + key);
                bias_l[row * kTilePad + col] = bv;
            }
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int kk = 8 * (r / 4) + 4 * half + (r % 4);
            float s = acc[kt][r] * scale;
            if (bias != nullptr) s += bias_l[col * kTilePad + kk];
            if (kt * 32 + kk >= S) s = -INFINITY;
            acc[kt][r] = s;
            m = fmaxf(m, s);
        }
        __syncthreads();
    }
    m = fmaxf(m, __shfl_xor(m, 32));
    if (m == -INFINITY) m = 0.f;
    float l = 0.f;
#pragma unroll
    for (int kt = 0; kt < NT; ++kt)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const float p = __expf(acc[kt][r] - m);
            acc[kt][r] = p;
            l += p;
        }
    l += __shfl_xor(l, 32);
    // O^T = V^T P^T
    float16_t o = zero16();
#pragma unroll
    for (int kt = 0; kt < NT; ++kt)
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            short4_t pb;
            pb.x = f2bf(acc[kt][4 * t + 0]); pb.y = f2bf(acc[kt][4 * t + 1]);
            pb.z = f2bf(acc[kt][4 * t + 2]); pb.w = f2bf(acc[kt][4 * t + 3]);
            short4_t av = zero4();
            if (col < D) av = *reinterpret_cast<const short4_t*>(&v_tr[col * (SP + 4) + kt * 32 + t * 8 + half * 4]);
            o = mfma(av, pb, o);
        }
    if (qi < S) {
        const float inv = 1.0f / l;
        T* op = out + (((int64_t)g * S + qi) * H + h) * D;
#pragma unroll
        for (int rb = 0; rb < KS; ++rb)
            st4(op + 8 * rb + 4 * half, o[4 * rb + 0] * inv, o[4 * rb + 1] * inv, o[4 * rb + 2] * inv,
                o[4 * rb + 3] * inv);
        if (half == 0) lse[((int64_t)g * H + h) * S + qi] = m + __logf(l);
    }
}

// ---------------------------------------------------------------------------
// backward
// ---------------------------------------------------------------------------
// Wave w first acts on query tile w (transposed scores, lane = query): dQ and the
// per-query D = dout . out.  Then on key tile w (direct scores, lane = key): dK, dV
// and dBias, with coalesced bias reads and dBias writes.
template <typename T, int D, int NT>
__global__ __launch_bounds__(64 * NT) void k_dense_bwd(const T* __restrict__ Q, const T* __restrict__ K,
                                                       const T* __restrict__ V, const T* __restrict__ bias,
                                                       const T* __restrict__ O, const float* __restrict__ lse,
                                                       const T* __restrict__ dO, T* __restrict__ dQ,
                                                       T* __restrict__ dK, T* __restrict__ dV,
                                                       T* __restrict__ dbias, int S, int H, float scale) {
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
    float* lse_l = reinterpret_cast<float*>(g_tr + TR);
    float* dd_l = lse_l + SP;
    const int g = blockIdx.x / H, h = blockIdx.x % H;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int col = lane & 31, half = lane >> 5;
    float* bias_l = dd_l + SP + wave * 32 * kTilePad;
    load_head<T, D, SP>(Q, g, h, S, H, q_rm, q_tr);
    load_head<T, D, SP>(K, g, h, S, H, k_rm, k_tr);
    load_head<T, D, SP>(V, g, h, S, H, v_rm, nullptr);
    load_head<T, D, SP>(dO, g, h, S, H, g_rm, g_tr);
    for (int i = threadIdx.x; i < SP; i += blockDim.x)
        lse_l[i] = i < S ? lse[((int64_t)g * H + h) * S + i] : 0.f;
    // D[q] = sum_dd dout[q,dd] out[q,dd]
    for (int i = threadIdx.x; i < SP; i += blockDim.x) {
        float dsum = 0.f;
        if (i < S) {
            const T* op = O + (((int64_t)g * S + i) * H + h) * D;
#pragma unroll
            for (int c = 0; c < D; c += 4) {
                const short4_t ov = ld4(op + c);
                const short4_t gv = ld4(dO + (((int64_t)g * S + i) * H + h) * D + c);
                dsum += bf2f(ov.x) * bf2f(gv.x) + bf2f(ov.y) * bf2f(gv.y) + bf2f(ov.z) * bf2f(gv.z) +
                        bf2f(ov.w) * bf2f(gv.w);
            }
        }
        dd_l[i] = dsum;
    }
    __syncthreads();

    // ---- query tile `wave`: dQ -------------------------------------------------
    {
        const int q0 = wave * 32, qi = q0 + col;
        short4_t bq[KS], bg[KS];
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            bq[s] = *reinterpret_cast<const short4_t*>(&q_rm[qi * D + s * 8 + half * 4]);
            bg[s] = *reinterpret_cast<const short4_t*>(&g_rm[qi * D + s * 8 + half * 4]);
        }
        const float L = lse_l[qi], Dq = dd_l[qi];
        float16_t dq = zero16();
#pragma unroll
        for (int kt = 0; kt < NT; ++kt) {
            float16_t sc = zero16(), dp = zero16();
#pragma unroll
            for (int s = 0; s < KS; ++s) {
                const short4_t ak = *reinterpret_cast<const short4_t*>(&k_rm[(kt * 32 + col) * D + s * 8 + half * 4]);
                const short4_t av = *reinterpret_cast<const short4_t*>(&v_rm[(kt * 32 + col) * D + s * 8 + half * 4]);
                sc = mfma(ak, bq[s], sc);     // S^T[key, query]
                dp = mfma(av, bg[s], dp);     // dP^T[key, query] = V dout^T
            }
            if (bias != nullptr) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int row = r * 2 + half, key = kt * 32 + col;
                    float bv = 0.f;
                    if (q0 + row < S && key < S)
                        bv = ld1(bias + (((int64_t)g * H + h) * S + q0 + row) * S + key);
                    bias_l[row * kTilePad + col] = bv;
                }
            }
            __syncthreads();
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int kk = 8 * (r / 4) + 4 * half + (r % 4);
                float s = sc[r] * scale;
                if (bias != nullptr) s += bias_l[col * kTilePad + kk];
                float p = __expf(s - L);
                if (kt * 32 + kk >= S || qi >= S) p = 0.f;
                sc[r] = p * (dp[r] - Dq);      // dS^T
            }
            __syncthreads();
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                short4_t db;
                db.x = f2bf(sc[4 * t + 0]); db.y = f2bf(sc[4 * t + 1]);
                db.z = f2bf(sc[4 * t + 2]); db.w = f2bf(sc[4 * t + 3]);
                short4_t ak = zero4();
                if (col < D) ak = *reinterpret_cast<const short4_t*>(&k_tr[col * (SP + 4) + kt * 32 + t * 8 + half * 4]);
                dq = mfma(ak, db, dq);        // dQ^T[dd, query] += K^T dS^T
            }
        }
        if (qi < S) {
            T* p = dQ + (((int64_t)g * S + qi) * H + h) * D;
#pragma unroll
            for (int rb = 0; rb < KS; ++rb)
                st4(p + 8 * rb + 4 * half, dq[4 * rb + 0] * scale, dq[4 * rb + 1] * scale, dq[4 * rb + 2] * scale,
                    dq[4 * rb + 3] * scale);
        }
    }

    // ---- key tile `wave`: dK, dV, dBias -----------------------------------------
    {
        const int k0 = wave * 32, ki = k0 + col;
        short4_t bk[KS], bv[KS];
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            bk[s] = *reinterpret_cast<const short4_t*>(&k_rm[ki * D + s * 8 + half * 4]);
            bv[s] = *reinterpret_cast<const short4_t*>(&v_rm[ki * D + s * 8 + half * 4]);
        }
        float16_t dk = zero16(), dv = zero16();
#pragma unroll
        for (int qt = 0; qt < NT; ++qt) {
            float16_t sc = zero16(), dp = zero16();
#pragma unroll
            for (int s = 0; s < KS; ++s) {
                const short4_t aq = *reinterpret_cast<const short4_t*>(&q_rm[(qt * 32 + col) * D + s * 8 + half * 4]);
                const short4_t ag = *reinterpret_cast<const short4_t*>(&g_rm[(qt * 32 + col) * D + s * 8 + half * 4]);
                sc = mfma(aq, bk[s], sc);     // S[query, key]
                dp = mfma(ag, bv[s], dp);     // dP[query, key] = dout V^T
            }
            float pr[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int qq = qt * 32 + 8 * (r / 4) + 4 * half + (r % 4);
                float s = sc[r] * scale;
                const bool ok = qq < S && ki < S;
                if (bias != nullptr && ok) s += ld1(bias + (((int64_t)g * H + h) * S + qq) * S + ki);
                float p = ok ? __expf(s - lse_l[qq]) : 0.f;
                const float ds = p * (dp[r] - dd_l[qq]);
                if (dbias != nullptr && ok) st1(dbias + (((int64_t)g * H + h) * S + qq) * S + ki, ds);
                pr[r] = p;
                sc[r] = ds;
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
        }
        if (ki < S) {
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
};

template <typename T, int D, int NT>
static int launch_dense(const DenseCall& c, bool bwd) {
    const float scale = sqrtf((float)c.d);     // the reference MULTIPLIES q by sqrt(d)
    const dim3 grid((unsigned)(c.b * c.H)), block(64 * NT);
    constexpr int lds_f = fwd_lds_bytes<D, NT>(), lds_b = bwd_lds_bytes<D, NT>();
    static_assert(lds_b <= 160 * 1024, "backward LDS image exceeds the 160 KB of a CU");
    static bool attr_done = false;     // raise the dynamic-LDS cap once per instantiation
    if (!attr_done) {
        if (lds_f > 48 * 1024)
            TGT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&k_dense_fwd<T, D, NT>),
                                              hipFuncAttributeMaxDynamicSharedMemorySize, lds_f));
        if (lds_b > 48 * 1024)
            TGT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&k_dense_bwd<T, D, NT>),
                                              hipFuncAttributeMaxDynamicSharedMemorySize, lds_b));
        attr_done = true;
    }
    if (!bwd) {
        KernelTimer t(KS_DENSE_FWD, c.st);
        hipLaunchKernelGGL((k_dense_fwd<T, D, NT>), grid, block, lds_f, c.st, (const T*)c.q, (const T*)c.k,
                           (const T*)c.v, (const T*)c.bias, (T*)c.o_out, c.o_lse, c.S, c.H, scale);
    } else {
        KernelTimer t(KS_DENSE_BWD, c.st);
        hipLaunchKernelGGL((k_dense_bwd<T, D, NT>), grid, block, lds_b, c.st, (const T*)c.q, (const T*)c.k,
                           (const T*)c.v, (const T*)c.bias, (const T*)c.out, c.lse, (const T*)c.dout, (T*)c.dq,
                           (T*)c.dk, (T*)c.dv, (T*)c.dbias, c.S, c.H, scale);
    }
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
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

static int check_dense(const void* q, const void* k, const void* v, int b, int S, int H, int d, int dtype) {
    if (!q || !k || !v) { set_error("dense attention: null q/k/v"); return TGT_ERR_INVALID_ARG; }
    if (b < 1 || S < 1 || H < 1 || d < 1) { set_error("dense attention: non-positive size"); return TGT_ERR_INVALID_ARG; }
    if (dtype != TGT_DTYPE_F32 && dtype != TGT_DTYPE_BF16) { set_error("bad dtype %d", dtype); return TGT_ERR_INVALID_ARG; }
    if ((int64_t)b * H > 0x7fffffffLL) { set_error("dense attention: b*H too large"); return TGT_ERR_INVALID_ARG; }
    return TGT_OK;
}

}  // namespace tgt

extern "C" {

int tgt_dense_attn_fwd(const void* d_q, const void* d_k, const void* d_v, const void* d_bias, int b, int S, int H,
                       int d, int dtype, void* d_out, float* d_lse, void* stream) {
    int rc = tgt::check_dense(d_q, d_k, d_v, b, S, H, d, dtype);
    if (rc) return rc;
    if (!d_out || !d_lse) { tgt::set_error("dense attention: null out or lse"); return TGT_ERR_INVALID_ARG; }
    tgt::DenseCall c{};
    c.q = d_q; c.k = d_k; c.v = d_v; c.bias = d_bias; c.o_out = d_out; c.o_lse = d_lse;
    c.b = b; c.S = S; c.H = H; c.d = d; c.st = (hipStream_t)stream;
    return dtype == TGT_DTYPE_F32 ? tgt::dispatch_d<float>(c, false) : tgt::dispatch_d<tgt::dbf16>(c, false);
}

int tgt_dense_attn_bwd(const void* d_q, const void* d_k, const void* d_v, const void* d_bias, int b, int S, int H,
                       int d, int dtype, const void* d_out, const float* d_lse, const void* d_dout, void* d_dq,
                       void* d_dk, void* d_dv, void* d_dbias, void* stream) {
    int rc = tgt::check_dense(d_q, d_k, d_v, b, S, H, d, dtype);
    if (rc) return rc;
    if (!d_out || !d_lse || !d_dout || !d_dq || !d_dk || !d_dv) {
        tgt::set_error("dense attention backward: null out/lse/dout/dq/dk/dv");
        return TGT_ERR_INVALID_ARG;
    }
    tgt::DenseCall c{};
    c.q = d_q; c.k = d_k; c.v = d_v; c.bias = d_bias; c.out = d_out; c.lse = d_lse; c.dout = d_dout;
    c.dq = d_dq; c.dk = d_dk; c.dv = d_dv; c.dbias = d_dbias;
    c.b = b; c.S = S; c.H = H; c.d = d; c.st = (hipStream_t)stream;
    return dtype == TGT_DTYPE_F32 ? tgt::dispatch_d<float>(c, true) : tgt::dispatch_d<tgt::dbf16>(c, true);
}

}  // extern "C"
