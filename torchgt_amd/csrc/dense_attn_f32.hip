// Dense biased attention in float32 arithmetic, for float32 callers.
//
// The reference's dense CoreAttention.forward (models/graphormer_graph_level.py:186-214, attn_module.py:99-127)
// computes in float32:  x = (q * sqrt(d)) k^T + attn_bias ; softmax over keys ; dropout ; x v.  The matrix-core
// kernels of dense_attn.hip round their operands to bf16, which costs 2^-8 on logits that the reference's
// q * sqrt(d) makes large; a float32 caller who has not asked for that gets these kernels instead: plain fp32
// multiply-adds on the vector units (head dims of 8 to 32 make the products 8 to 32 deep, far too thin to be
// bound by them), fp32 softmax with the accurate exponential, 1e-5 against a float64 evaluation.
//
// One workgroup per (graph, head).  Forward: K and V of the head sit in LDS, a thread owns one query row and
// walks the keys with an online softmax; every LDS read of K / V is a broadcast.  A thread that read its own
// bias row from memory would touch a different cache line in every lane, so the bias comes in strips of 32
// keys: the workgroup loads the strip [S queries][32 keys] with coalesced reads into LDS and every thread
// then takes its row from there (and, in the backward, leaves its row of dBias there for a coalesced write).
// Backward: a first walk with thread = query gives dQ and dBias, a second with thread = key gives dK and dV
// (its bias reads are coalesced over the threads as they are); both recompute the probabilities from the
// saved log-sum-exp.
#include "common.h"
#include "dense_dropout.h"

namespace tgt {

constexpr int kF32Block = 256;
constexpr int kF32Chunk = 8;        // keys between two rescalings of the online softmax
constexpr int kF32Strip = 32;       // keys of one bias strip
constexpr int kF32StripLd = 33;     // its row stride in LDS (odd: rows of consecutive queries start in different banks)

// bias[q, k0 .. k0 + 32) for the queries q0 .. q1 - 1 -> strip[q][.] (zeros past the end of a row); coalesced
__device__ __forceinline__ void load_strip(const float* __restrict__ bias_gh, int S, int q0, int q1, int k0,
                                           float* __restrict__ strip) {
    for (int i = threadIdx.x; i < (q1 - q0) * kF32Strip; i += blockDim.x) {
        const int r = q0 + i / kF32Strip, c = i % kF32Strip;
        strip[r * kF32StripLd + c] = (k0 + c < S) ? bias_gh[(int64_t)r * S + k0 + c] : 0.f;
    }
}
__device__ __forceinline__ void store_strip(float* __restrict__ dbias_gh, int S, int q0, int q1, int k0,
                                            const float* __restrict__ strip) {
    for (int i = threadIdx.x; i < (q1 - q0) * kF32Strip; i += blockDim.x) {
        const int r = q0 + i / kF32Strip, c = i % kF32Strip;
        if (k0 + c < S) dbias_gh[(int64_t)r * S + k0 + c] = strip[r * kF32StripLd + c];
    }
}

template <int D>
__device__ __forceinline__ void ld_row(const float* __restrict__ p, float (&x)[D]) {
#pragma unroll
    for (int c = 0; c < D; c += 4) {
        const float4 v = *reinterpret_cast<const float4*>(p + c);
        x[c] = v.x; x[c + 1] = v.y; x[c + 2] = v.z; x[c + 3] = v.w;
    }
}
template <int D>
__device__ __forceinline__ void st_row(float* __restrict__ p, const float (&x)[D], float f) {
#pragma unroll
    for (int c = 0; c < D; c += 4) *reinterpret_cast<float4*>(p + c) = make_float4(x[c] * f, x[c + 1] * f, x[c + 2] * f, x[c + 3] * f);
}
template <int D>
__device__ __forceinline__ float dotf(const float (&a)[D], const float* __restrict__ b) {
    float t = 0.f;
#pragma unroll
    for (int c = 0; c < D; ++c) t = fmaf(a[c], b[c], t);
    return t;
}

// X[g, :, h, :] -> LDS [S][D], optionally scaled
template <int D>
__device__ __forceinline__ void stage_head(const float* __restrict__ X, int g, int h, int S, int H, float f,
                                           float* __restrict__ dst) {
    for (int c = threadIdx.x; c < S * (D / 4); c += blockDim.x) {
        const int row = c / (D / 4), part = c % (D / 4);
        float4 v = *reinterpret_cast<const float4*>(X + (((int64_t)g * S + row) * H + h) * D + part * 4);
        v.x *= f; v.y *= f; v.z *= f; v.w *= f;
        *reinterpret_cast<float4*>(dst + row * D + part * 4) = v;
    }
}

// workgroup -> (graph, head): the H heads of a graph share every line of q/k/v, so they get workgroup ids that
// are congruent modulo 8 (same XCD, same L2) inside a window of 8 * H ids
__device__ __forceinline__ bool pair_of_block(int nb, int H, int& g, int& h) {
    const int win = blockIdx.x / (8 * H), rem = blockIdx.x % (8 * H);
    g = win * 8 + (rem & 7);
    h = rem >> 3;
    return g < nb;
}

template <int D, bool DROP>
__global__ __launch_bounds__(kF32Block) void k_dense_f32_fwd(const float* __restrict__ Q, const float* __restrict__ K,
                                                             const float* __restrict__ V, const float* __restrict__ bias,
                                                             float* __restrict__ out, float* __restrict__ lse, int S, int H,
                                                             float scale, int nb, const DropArgs da) {
    extern __shared__ __align__(16) char smem[];
    float* k_l = reinterpret_cast<float*>(smem);
    float* v_l = k_l + S * D;
    float* strip = v_l + S * D;                      // [S][kF32StripLd]
    int g, h;
    if (!pair_of_block(nb, H, g, h)) return;
    stage_head<D>(K, g, h, S, H, 1.0f, k_l);
    stage_head<D>(V, g, h, S, H, 1.0f, v_l);
    const float* bias_gh = bias ? bias + ((int64_t)g * H + h) * S * S : nullptr;
    // a thread owns query qi = threadIdx.x + 256 * pass; all threads take part in the strip loads of every pass
    for (int q0 = 0; q0 < S; q0 += blockDim.x) {
        const int qi = q0 + threadIdx.x;
        const bool qok = qi < S;
        float qs[D], o[D];
#pragma unroll
        for (int c = 0; c < D; ++c) { qs[c] = 0.f; o[c] = 0.f; }
        if (qok) ld_row<D>(Q + (((int64_t)g * S + qi) * H + h) * D, qs);
#pragma unroll
        for (int c = 0; c < D; ++c) qs[c] *= scale;      // the reference scales q before the product
        const uint32_t rh = DROP ? drop_row_hash(da, g * H + h, qi) : 0u;
        float m = -INFINITY, l = 0.f;
        for (int s0 = 0; s0 < S; s0 += kF32Strip) {
            __syncthreads();                             // K / V staged; the previous strip is consumed
            if (bias_gh) load_strip(bias_gh, S, q0, min(S, q0 + (int)blockDim.x), s0, strip);
            __syncthreads();
            if (!qok) continue;
            const float* brow = strip + qi * kF32StripLd;
#pragma unroll 1
            for (int k0 = s0; k0 < min(S, s0 + kF32Strip); k0 += kF32Chunk) {
                float sc[kF32Chunk], cm = -INFINITY;
#pragma unroll
                for (int j = 0; j < kF32Chunk; ++j) {
                    const int k = k0 + j;
                    sc[j] = -INFINITY;
                    if (k < S) sc[j] = dotf<D>(qs, k_l + k * D) + (bias_gh ? brow[k - s0] : 0.f);
                    cm = fmaxf(cm, sc[j]);
                }
                const float m_new = fmaxf(m, cm);
                const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
                const float alpha = expf(m - m_use);           // m = -inf: 0
                l *= alpha;
#pragma unroll
                for (int c = 0; c < D; ++c) o[c] *= alpha;
#pragma unroll
                for (int j = 0; j < kF32Chunk; ++j) {
                    const int k = k0 + j;
                    if (k < S) {
                        const float p = expf(sc[j] - m_use);
                        l += p;
                        const float pk = (!DROP || drop_keep(da, rh, k)) ? p : 0.f;
                        const float* vr = v_l + k * D;
#pragma unroll
                        for (int c = 0; c < D; ++c) o[c] = fmaf(pk, vr[c], o[c]);
                    }
                }
                m = m_new;
            }
        }
        if (qok) {
            st_row<D>(out + (((int64_t)g * S + qi) * H + h) * D, o, (DROP ? da.inv_keep : 1.0f) / l);
            lse[((int64_t)g * H + h) * S + qi] = (m == -INFINITY ? 0.f : m) + logf(l);
        }
    }
}

template <int D, bool DROP>
__global__ __launch_bounds__(kF32Block) void k_dense_f32_bwd(const float* __restrict__ Q, const float* __restrict__ K,
                                                             const float* __restrict__ V, const float* __restrict__ bias,
                                                             const float* __restrict__ O, const float* __restrict__ lse,
                                                             const float* __restrict__ dO, float* __restrict__ dQ,
                                                             float* __restrict__ dK, float* __restrict__ dV,
                                                             float* __restrict__ dbias, int S, int H, float scale, int nb,
                                                             const DropArgs da) {
    extern __shared__ __align__(16) char smem[];
    float* q_l = reinterpret_cast<float*>(smem);     // q * sqrt(d)
    float* k_l = q_l + S * D;
    float* v_l = k_l + S * D;
    float* g_l = v_l + S * D;                        // dout
    float* lse_l = g_l + S * D;
    float* dd_l = lse_l + S;                         // sum_c dout[q, c] out[q, c]
    float* strip = dd_l + S;                         // [S][kF32StripLd] bias in, dBias out
    int g, h;
    if (!pair_of_block(nb, H, g, h)) return;
    stage_head<D>(Q, g, h, S, H, scale, q_l);
    stage_head<D>(K, g, h, S, H, 1.0f, k_l);
    stage_head<D>(V, g, h, S, H, 1.0f, v_l);
    stage_head<D>(dO, g, h, S, H, 1.0f, g_l);
    for (int i = threadIdx.x; i < S; i += blockDim.x) {
        float ov[D], gv[D];
        ld_row<D>(O + (((int64_t)g * S + i) * H + h) * D, ov);
        ld_row<D>(dO + (((int64_t)g * S + i) * H + h) * D, gv);
        float t = 0.f;
#pragma unroll
        for (int c = 0; c < D; ++c) t = fmaf(ov[c], gv[c], t);
        dd_l[i] = t;
        lse_l[i] = lse[((int64_t)g * H + h) * S + i];
    }
    __syncthreads();
    const float* bias_gh = bias ? bias + ((int64_t)g * H + h) * S * S : nullptr;
    float* dbias_gh = dbias ? dbias + ((int64_t)g * H + h) * S * S : nullptr;
    // thread = query: dQ and the query's row of dBias, strip by strip
    for (int q0 = 0; q0 < S; q0 += blockDim.x) {
        const int qi = q0 + threadIdx.x;
        const bool qok = qi < S;
        float qs[D], gv[D], dq[D];
#pragma unroll
        for (int c = 0; c < D; ++c) { qs[c] = qok ? q_l[qi * D + c] : 0.f; gv[c] = qok ? g_l[qi * D + c] : 0.f; dq[c] = 0.f; }
        const float L = qok ? lse_l[qi] : 0.f, Dq = qok ? dd_l[qi] : 0.f;
        const uint32_t rh = DROP ? drop_row_hash(da, g * H + h, qi) : 0u;
        for (int s0 = 0; s0 < S; s0 += kF32Strip) {
            __syncthreads();                             // the previous strip is written out
            if (bias_gh) load_strip(bias_gh, S, q0, min(S, q0 + (int)blockDim.x), s0, strip);
            __syncthreads();
            if (qok) {
                float* brow = strip + qi * kF32StripLd;
                for (int k = s0; k < min(S, s0 + kF32Strip); ++k) {
                    const float b = bias_gh ? brow[k - s0] : 0.f;
                    const float p = expf(dotf<D>(qs, k_l + k * D) + b - L);
                    const float ks = !DROP ? 1.0f : (drop_keep(da, rh, k) ? da.inv_keep : 0.f);
                    const float dS = p * (dotf<D>(gv, v_l + k * D) * ks - Dq);
                    brow[k - s0] = dS;                   // this thread's own row: the strip now holds dBias
                    const float* kr = k_l + k * D;
#pragma unroll
                    for (int c = 0; c < D; ++c) dq[c] = fmaf(dS, kr[c], dq[c]);
                }
            }
            if (dbias_gh) {
                __syncthreads();
                store_strip(dbias_gh, S, q0, min(S, q0 + (int)blockDim.x), s0, strip);
            }
        }
        if (qok) st_row<D>(dQ + (((int64_t)g * S + qi) * H + h) * D, dq, scale);
    }
    __syncthreads();
    // thread = key: dK and dV (the bias element of (query, key) is read by consecutive threads for one query)
    for (int ki = threadIdx.x; ki < S; ki += blockDim.x) {
        float kv[D], vv[D], dk[D], dv[D];
#pragma unroll
        for (int c = 0; c < D; ++c) { kv[c] = k_l[ki * D + c]; vv[c] = v_l[ki * D + c]; dk[c] = 0.f; dv[c] = 0.f; }
        for (int qq = 0; qq < S; ++qq) {
            const float b = bias_gh ? bias_gh[(int64_t)qq * S + ki] : 0.f;
            const float* qr = q_l + qq * D;
            const float* gr = g_l + qq * D;
            const float p = expf(dotf<D>(kv, qr) + b - lse_l[qq]);
            const float ks = !DROP ? 1.0f : (drop_keep(da, drop_row_hash(da, g * H + h, qq), ki) ? da.inv_keep : 0.f);
            const float dS = p * (dotf<D>(vv, gr) * ks - dd_l[qq]);
            const float pk = p * ks;
#pragma unroll
            for (int c = 0; c < D; ++c) {
                dk[c] = fmaf(dS, qr[c], dk[c]);      // qr holds q * sqrt(d): d s / d k
                dv[c] = fmaf(pk, gr[c], dv[c]);
            }
        }
        st_row<D>(dK + (((int64_t)g * S + ki) * H + h) * D, dk, 1.0f);
        st_row<D>(dV + (((int64_t)g * S + ki) * H + h) * D, dv, 1.0f);
    }
}

template <int D>
static int launch_f32(const DenseF32Call& c, bool bwd) {
    const int lds_bwd = (4 * c.S * D + 2 * c.S) * 4 + c.S * kF32StripLd * 4;
    const int lds = bwd ? lds_bwd : 2 * c.S * D * 4 + c.S * kF32StripLd * 4;
    if (lds_bwd > 160 * 1024) {      // the forward refuses what its backward could not run
        set_error("dense attention (float32): S=%d with head dim %d needs %d bytes of LDS (limit %d)", c.S, D, lds_bwd, 160 * 1024);
        return TGT_ERR_UNSUPPORTED;
    }
    const float scale = sqrtf((float)D);      // the reference MULTIPLIES q by sqrt(d)
    const bool drop = c.p_drop > 0.f;
    const DropArgs da = drop_args(c.p_drop, c.seed);
    const dim3 grid((unsigned)(((c.b + 7) / 8) * 8 * c.H)), block(kF32Block);
    static bool attr_done = false;
    if (!attr_done) {
        const int cap = 160 * 1024;
        TGT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&k_dense_f32_fwd<D, false>), hipFuncAttributeMaxDynamicSharedMemorySize, cap));
        TGT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&k_dense_f32_fwd<D, true>), hipFuncAttributeMaxDynamicSharedMemorySize, cap));
        TGT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&k_dense_f32_bwd<D, false>), hipFuncAttributeMaxDynamicSharedMemorySize, cap));
        TGT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&k_dense_f32_bwd<D, true>), hipFuncAttributeMaxDynamicSharedMemorySize, cap));
        attr_done = true;
    }
    if (!bwd) {
        KernelTimer t(KS_DENSE_FWD, c.st);
        if (drop) hipLaunchKernelGGL((k_dense_f32_fwd<D, true>), grid, block, lds, c.st, c.q, c.k, c.v, c.bias, c.o_out, c.o_lse, c.S, c.H, scale, c.b, da);
        else hipLaunchKernelGGL((k_dense_f32_fwd<D, false>), grid, block, lds, c.st, c.q, c.k, c.v, c.bias, c.o_out, c.o_lse, c.S, c.H, scale, c.b, da);
    } else {
        KernelTimer t(KS_DENSE_BWD, c.st);
        if (drop) hipLaunchKernelGGL((k_dense_f32_bwd<D, true>), grid, block, lds, c.st, c.q, c.k, c.v, c.bias, c.out, c.lse, c.dout, c.dq, c.dk, c.dv, c.dbias, c.S, c.H, scale, c.b, da);
        else hipLaunchKernelGGL((k_dense_f32_bwd<D, false>), grid, block, lds, c.st, c.q, c.k, c.v, c.bias, c.out, c.lse, c.dout, c.dq, c.dk, c.dv, c.dbias, c.S, c.H, scale, c.b, da);
    }
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

int dense_attn_f32(const DenseF32Call& c, bool bwd) {
    switch (c.d) {
        case 8: return launch_f32<8>(c, bwd);
        case 16: return launch_f32<16>(c, bwd);
        case 32: return launch_f32<32>(c, bwd);
        default:
            set_error("dense attention: head dim %d not in {8, 16, 32}", c.d);
            return TGT_ERR_UNSUPPORTED;
    }
}

}  // namespace tgt
