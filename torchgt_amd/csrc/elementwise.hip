// Row-wise and elementwise pieces of the encoder layer around the attention:
// residual add + LayerNorm in one pass, and GELU.
//
// EncoderLayer.forward (models/graphormer_dist_node_level.py:296-314):
//     y = self_attention_norm(x); y = self_attention(y); x = x + y
//     y = ffn_norm(x);            y = ffn(y);            x = x + y
// FeedForwardNetwork.forward (:35-39): layer2(gelu(layer1(x))), nn.GELU() = exact erf form.
// In the reference each of these is its own ATen kernel (add, LayerNorm, GELU: three
// passes per residual block); here the residual add is folded into the LayerNorm
// that follows it: s = x + r is formed, written once and normalised from registers.
//
// Both kernels are pure streaming (HBM-bound): 16-byte accesses, a row of C features
// is held by C / (16 / sizeof) adjacent lanes and reduced with lane shuffles.
#include "common.h"
#include <algorithm>

namespace tgt {
namespace {

struct ebf16 { uint16_t x; };

template <typename T> struct Vec;      // 16 bytes of T as floats
template <> struct Vec<float> {
    static constexpr int N = 4;
    static __device__ __forceinline__ void load(const float* p, float (&f)[4]) {
        const float4 v = *reinterpret_cast<const float4*>(p);
        f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w;
    }
    static __device__ __forceinline__ void store(float* p, const float (&f)[4]) {
        *reinterpret_cast<float4*>(p) = make_float4(f[0], f[1], f[2], f[3]);
    }
};
template <> struct Vec<ebf16> {
    static constexpr int N = 8;
    static __device__ __forceinline__ void load(const ebf16* p, float (&f)[8]) {
        const uint4 u = *reinterpret_cast<const uint4*>(p);
        const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[2 * i] = __uint_as_float(w[i] << 16);
            f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
    }
    static __device__ __forceinline__ void store(ebf16* p, const float (&f)[8]) {
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const __bf16 lo = static_cast<__bf16>(f[2 * i]), hi = static_cast<__bf16>(f[2 * i + 1]);
            w[i] = (uint32_t)__builtin_bit_cast(uint16_t, lo) | ((uint32_t)__builtin_bit_cast(uint16_t, hi) << 16);
        }
        *reinterpret_cast<uint4*>(p) = make_uint4(w[0], w[1], w[2], w[3]);
    }
};

template <int LPR>
__device__ __forceinline__ float row_sum(float v) {
#pragma unroll
    for (int off = LPR / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

constexpr int kEwBlock = 256;

// s = x (+ r); y = (s - mean) * rstd * gamma + beta.  LPR lanes hold one row.
// sum_out / y / mean / rstd may be null (not wanted).
template <typename T, int LPR>
__global__ __launch_bounds__(kEwBlock) void k_add_layer_norm_fwd(const T* __restrict__ x, const T* __restrict__ r,
                                                                  const T* __restrict__ gamma, const T* __restrict__ beta,
                                                                  int64_t N, float eps, T* __restrict__ sum_out,
                                                                  T* __restrict__ y, float* __restrict__ mean_out,
                                                                  float* __restrict__ rstd_out) {
    constexpr int VE = Vec<T>::N, C = LPR * VE, RPB = kEwBlock / LPR;
    const int sub = threadIdx.x % LPR, slot = threadIdx.x / LPR;
    float g[VE], b[VE];
#pragma unroll
    for (int i = 0; i < VE; ++i) { g[i] = 1.f; b[i] = 0.f; }
    if (y) {
        Vec<T>::load(gamma + sub * VE, g);
        Vec<T>::load(beta + sub * VE, b);
    }
    for (int64_t row = (int64_t)blockIdx.x * RPB + slot; row < N; row += (int64_t)gridDim.x * RPB) {
        float s[VE];
        Vec<T>::load(x + row * C + sub * VE, s);
        if (r) {
            float t[VE];
            Vec<T>::load(r + row * C + sub * VE, t);
#pragma unroll
            for (int i = 0; i < VE; ++i) s[i] += t[i];
        }
        if (sum_out) Vec<T>::store(sum_out + row * C + sub * VE, s);
        if (!y) continue;
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < VE; ++i) acc += s[i];
        const float mean = row_sum<LPR>(acc) * (1.f / C);
        float var = 0.f;
#pragma unroll
        for (int i = 0; i < VE; ++i) var += (s[i] - mean) * (s[i] - mean);
        const float rstd = rsqrtf(row_sum<LPR>(var) * (1.f / C) + eps);
        float o[VE];
#pragma unroll
        for (int i = 0; i < VE; ++i) o[i] = (s[i] - mean) * rstd * g[i] + b[i];
        Vec<T>::store(y + row * C + sub * VE, o);
        if (sub == 0) {
            if (mean_out) mean_out[row] = mean;
            if (rstd_out) rstd_out[row] = rstd;
        }
    }
}

// ds = rstd * (g - mean(g) - xhat * mean(g * xhat)) (+ extra), g = dy * gamma, xhat = (s - mean) * rstd;
// per-workgroup partial sums of dgamma = sum_rows dy * xhat and dbeta = sum_rows dy go to
// partial[blockIdx.x][2][C].
template <typename T, int LPR>
__global__ __launch_bounds__(kEwBlock) void k_layer_norm_bwd(const T* __restrict__ s_in, const T* __restrict__ gamma,
                                                              const float* __restrict__ mean_in,
                                                              const float* __restrict__ rstd_in, const T* __restrict__ dy,
                                                              const T* __restrict__ extra, int64_t N, T* __restrict__ ds,
                                                              float* __restrict__ partial) {
    constexpr int VE = Vec<T>::N, C = LPR * VE, RPB = kEwBlock / LPR;
    __shared__ float red[2][RPB][C + 1];
    const int sub = threadIdx.x % LPR, slot = threadIdx.x / LPR;
    float g[VE], dg[VE], db[VE];
    Vec<T>::load(gamma + sub * VE, g);
#pragma unroll
    for (int i = 0; i < VE; ++i) { dg[i] = 0.f; db[i] = 0.f; }
    // two rows of the walk per step, all their loads issued before the first is used (a lane has six 16-byte loads
    // in flight instead of three); the rows enter the column sums in the order of the one-row walk: same bits
    const int64_t step = (int64_t)gridDim.x * RPB;
    for (int64_t row0 = (int64_t)blockIdx.x * RPB + slot; row0 < N; row0 += 2 * step) {
        const bool two = row0 + step < N;
        const int64_t rows[2] = {row0, two ? row0 + step : row0};
        float s[2][VE], d[2][VE], t[2][VE], mean[2], rstd[2];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            Vec<T>::load(s_in + rows[u] * C + sub * VE, s[u]);
            Vec<T>::load(dy + rows[u] * C + sub * VE, d[u]);
            mean[u] = mean_in[rows[u]]; rstd[u] = rstd_in[rows[u]];
            if (extra) Vec<T>::load(extra + rows[u] * C + sub * VE, t[u]);
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            if (u == 1 && !two) break;
            float xh[VE], gg[VE], a1 = 0.f, a2 = 0.f;
#pragma unroll
            for (int i = 0; i < VE; ++i) {
                xh[i] = (s[u][i] - mean[u]) * rstd[u];
                gg[i] = d[u][i] * g[i];
                a1 += gg[i];
                a2 += gg[i] * xh[i];
                dg[i] += d[u][i] * xh[i];
                db[i] += d[u][i];
            }
            const float m1 = row_sum<LPR>(a1) * (1.f / C), m2 = row_sum<LPR>(a2) * (1.f / C);
            float o[VE];
#pragma unroll
            for (int i = 0; i < VE; ++i) o[i] = rstd[u] * (gg[i] - m1 - xh[i] * m2);
            if (extra) {
#pragma unroll
                for (int i = 0; i < VE; ++i) o[i] += t[u][i];
            }
            Vec<T>::store(ds + rows[u] * C + sub * VE, o);
        }
    }
#pragma unroll
    for (int i = 0; i < VE; ++i) {
        red[0][slot][sub * VE + i] = dg[i];
        red[1][slot][sub * VE + i] = db[i];
    }
    __syncthreads();
    for (int c = threadIdx.x; c < 2 * C; c += kEwBlock) {
        const int which = c / C, col = c % C;
        float t = 0.f;
#pragma unroll 8
        for (int k = 0; k < RPB; ++k) t += red[which][k][col];      // slots in order
        partial[(int64_t)blockIdx.x * 2 * C + c] = t;
    }
}

// nn.GELU (exact): h = 0.5 u (1 + erf(u / sqrt 2));  dh/du = 0.5 (1 + erf(u / sqrt 2)) + u exp(-u^2 / 2) / sqrt(2 pi)
// RELU: F.relu instead (the GT layers, models/gt_dist_node_level.py:258,285): h = max(u, 0); dh/du = 1 where u > 0.
template <typename T, bool BWD, bool RELU = false>
__global__ __launch_bounds__(kEwBlock) void k_gelu(const T* __restrict__ u, const T* __restrict__ dh, int64_t nvec,
                                                   T* __restrict__ out) {
    constexpr int VE = Vec<T>::N;
    for (int64_t v = (int64_t)blockIdx.x * kEwBlock + threadIdx.x; v < nvec; v += (int64_t)gridDim.x * kEwBlock) {
        float x[VE], o[VE], d[VE];
        Vec<T>::load(u + v * VE, x);
        if (BWD) Vec<T>::load(dh + v * VE, d);
#pragma unroll
        for (int i = 0; i < VE; ++i) o[i] = BWD ? act_grad<RELU>(x[i], d[i]) : act_value<RELU>(x[i]);
        Vec<T>::store(out + v * VE, o);
    }
}

int lanes_per_row(int C, int dtype) {
    const int ve = dtype == TGT_DTYPE_F32 ? 4 : 8;
    if (C % ve) return 0;
    const int l = C / ve;
    return (l == 2 || l == 4 || l == 8 || l == 16 || l == 32 || l == 64) ? l : 0;
}

int ln_check(int64_t N, int C, int dtype, const char* who) {
    if (N < 0 || C <= 0 || (dtype != TGT_DTYPE_F32 && dtype != TGT_DTYPE_BF16)) {
        set_error("%s: bad size or dtype", who);
        return TGT_ERR_INVALID_ARG;
    }
    if (!lanes_per_row(C, dtype)) {
        set_error("%s: %d features are not supported (16-byte vectors times a power of two up to 64 lanes)", who, C);
        return TGT_ERR_UNSUPPORTED;
    }
    return TGT_OK;
}

constexpr int kLnWorkers = 512;     // workgroups (= partial sums) of the LayerNorm backward

unsigned ew_grid(int64_t items, int per_block, int cap) {
    return (unsigned)std::max<int64_t>(1, std::min<int64_t>((items + per_block - 1) / per_block, cap));
}

#define TGT_LPR_SWITCH(L, X) \
    switch (L) {             \
        case 2: X(2); break; case 4: X(4); break; case 8: X(8); break; case 16: X(16); break; \
        case 32: X(32); break; default: X(64); break;                                          \
    }

template <typename T>
void launch_ln_fwd(int lpr, const void* x, const void* r, const void* gamma, const void* beta, int64_t N, float eps,
                   void* sum, void* y, float* mean, float* rstd, hipStream_t st) {
#define X(L)                                                                                                      \
    hipLaunchKernelGGL((k_add_layer_norm_fwd<T, L>), dim3(ew_grid(N, kEwBlock / L, 8192)), dim3(kEwBlock), 0, st, \
                       (const T*)x, (const T*)r, (const T*)gamma, (const T*)beta, N, eps, (T*)sum, (T*)y, mean, rstd)
    TGT_LPR_SWITCH(lpr, X)
#undef X
}

template <typename T>
void launch_ln_bwd(int lpr, int workers, const void* s, const void* gamma, const float* mean, const float* rstd,
                   const void* dy, const void* extra, int64_t N, void* ds, float* partial, hipStream_t st) {
#define X(L)                                                                                                     \
    hipLaunchKernelGGL((k_layer_norm_bwd<T, L>), dim3(workers), dim3(kEwBlock), 0, st, (const T*)s, (const T*)gamma, \
                       mean, rstd, (const T*)dy, (const T*)extra, N, (T*)ds, partial)
    TGT_LPR_SWITCH(lpr, X)
#undef X
}

}  // namespace
}  // namespace tgt

extern "C" {

int tgt_add_layer_norm_fwd(const void* d_x, const void* d_r, const void* d_gamma, const void* d_beta, int64_t N, int C,
                           float eps, int dtype, void* d_sum, void* d_y, float* d_mean, float* d_rstd, void* stream) {
    using namespace tgt;
    const int rc = ln_check(N, C, dtype, "tgt_add_layer_norm_fwd");
    if (rc != TGT_OK) return rc;
    if (N == 0) return TGT_OK;
    if (!d_x || (!d_y && !d_sum) || (d_y && (!d_gamma || !d_beta))) {
        set_error("tgt_add_layer_norm_fwd: null pointer");
        return TGT_ERR_INVALID_ARG;
    }
    hipStream_t st = (hipStream_t)stream;
    const int lpr = lanes_per_row(C, dtype);
    KernelTimer t(KS_LAYER_NORM_FWD, st);
    if (dtype == TGT_DTYPE_F32) launch_ln_fwd<float>(lpr, d_x, d_r, d_gamma, d_beta, N, eps, d_sum, d_y, d_mean, d_rstd, st);
    else launch_ln_fwd<ebf16>(lpr, d_x, d_r, d_gamma, d_beta, N, eps, d_sum, d_y, d_mean, d_rstd, st);
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

int64_t tgt_layer_norm_bwd_workspace_bytes(int C) {
    return C > 0 ? (int64_t)sizeof(float) * tgt::kLnWorkers * 2 * C : 0;
}

static int layer_norm_bwd_entry(const void* d_s, const void* d_gamma, const float* d_mean, const float* d_rstd, const void* d_dy,
                                const void* d_ds_extra, int64_t N, int C, int dtype, void* d_ds, void* d_dgamma, void* d_dbeta,
                                void* d_workspace, int64_t workspace_bytes, void* stream, tgt_reduce_desc* defer) {
    using namespace tgt;
    const int rc = ln_check(N, C, dtype, "tgt_layer_norm_bwd");
    if (rc != TGT_OK) return rc;
    if (!d_gamma || !d_dgamma || !d_dbeta || (N > 0 && (!d_s || !d_mean || !d_rstd || !d_dy || !d_ds))) {
        set_error("tgt_layer_norm_bwd: null pointer");
        return TGT_ERR_INVALID_ARG;
    }
    if (!d_workspace || workspace_bytes < tgt_layer_norm_bwd_workspace_bytes(C) || ((uintptr_t)d_workspace & 15)) {
        set_error("tgt_layer_norm_bwd: workspace of %lld bytes (16-byte aligned) needed, got %lld",
                  (long long)tgt_layer_norm_bwd_workspace_bytes(C), (long long)workspace_bytes);
        return TGT_ERR_WORKSPACE;
    }
    hipStream_t st = (hipStream_t)stream;
    const int lpr = lanes_per_row(C, dtype);
    const int workers = (int)ew_grid(N, kEwBlock / lpr, kLnWorkers);
    float* partial = (float*)d_workspace;
    {
        KernelTimer t(KS_LAYER_NORM_BWD, st);
        if (dtype == TGT_DTYPE_F32) launch_ln_bwd<float>(lpr, workers, d_s, d_gamma, d_mean, d_rstd, d_dy, d_ds_extra, N, d_ds, partial, st);
        else launch_ln_bwd<ebf16>(lpr, workers, d_s, d_gamma, d_mean, d_rstd, d_dy, d_ds_extra, N, d_ds, partial, st);
    }
    TGT_HIP_CHECK(hipGetLastError());
    // the workgroups' column sums ([workers][2 C]: dgamma, then dbeta), added in a fixed order
    tgt_reduce_desc r{};
    r.partial = partial; r.workers = workers; r.n = 2 * C; r.n_out = 2;
    r.out[0] = d_dgamma; r.begin[0] = 0;
    r.out[1] = d_dbeta;  r.begin[1] = C;
    if (defer) { *defer = r; return TGT_OK; }
    return reduce_partials(&r, 1, dtype, st);
}

int tgt_layer_norm_bwd(const void* d_s, const void* d_gamma, const float* d_mean, const float* d_rstd, const void* d_dy,
                       const void* d_ds_extra, int64_t N, int C, int dtype, void* d_ds, void* d_dgamma, void* d_dbeta,
                       void* d_workspace, int64_t workspace_bytes, void* stream) {
    return layer_norm_bwd_entry(d_s, d_gamma, d_mean, d_rstd, d_dy, d_ds_extra, N, C, dtype, d_ds, d_dgamma, d_dbeta, d_workspace,
                                workspace_bytes, stream, nullptr);
}

int tgt_layer_norm_bwd_deferred(const void* d_s, const void* d_gamma, const float* d_mean, const float* d_rstd, const void* d_dy,
                                const void* d_ds_extra, int64_t N, int C, int dtype, void* d_ds, void* d_dgamma, void* d_dbeta,
                                void* d_workspace, int64_t workspace_bytes, void* stream, tgt_reduce_desc* desc) {
    if (!desc) { tgt::set_error("tgt_layer_norm_bwd_deferred: a descriptor is needed"); return TGT_ERR_INVALID_ARG; }
    *desc = tgt_reduce_desc{};
    return layer_norm_bwd_entry(d_s, d_gamma, d_mean, d_rstd, d_dy, d_ds_extra, N, C, dtype, d_ds, d_dgamma, d_dbeta, d_workspace,
                                workspace_bytes, stream, desc);
}

static int gelu_call(const void* d_u, const void* d_dh, int64_t n, int dtype, void* d_out, void* stream, bool bwd, bool relu = false) {
    using namespace tgt;
    if (n < 0 || (dtype != TGT_DTYPE_F32 && dtype != TGT_DTYPE_BF16)) {
        set_error("tgt_gelu: bad size or dtype");
        return TGT_ERR_INVALID_ARG;
    }
    const int ve = dtype == TGT_DTYPE_F32 ? 4 : 8;
    if (n % ve) {
        set_error("tgt_gelu: the element count must be a multiple of %d", ve);
        return TGT_ERR_UNSUPPORTED;
    }
    if (n == 0) return TGT_OK;
    if (!d_u || !d_out || (bwd && !d_dh)) { set_error("tgt_gelu: null pointer"); return TGT_ERR_INVALID_ARG; }
    hipStream_t st = (hipStream_t)stream;
    const int64_t nvec = n / ve;
    const dim3 grid(ew_grid(nvec, kEwBlock, 16384));
    KernelTimer t(KS_GELU, st);
    if (relu) {
        if (dtype == TGT_DTYPE_F32) {
            if (bwd) hipLaunchKernelGGL((k_gelu<float, true, true>), grid, dim3(kEwBlock), 0, st, (const float*)d_u, (const float*)d_dh, nvec, (float*)d_out);
            else hipLaunchKernelGGL((k_gelu<float, false, true>), grid, dim3(kEwBlock), 0, st, (const float*)d_u, (const float*)nullptr, nvec, (float*)d_out);
        } else {
            if (bwd) hipLaunchKernelGGL((k_gelu<ebf16, true, true>), grid, dim3(kEwBlock), 0, st, (const ebf16*)d_u, (const ebf16*)d_dh, nvec, (ebf16*)d_out);
            else hipLaunchKernelGGL((k_gelu<ebf16, false, true>), grid, dim3(kEwBlock), 0, st, (const ebf16*)d_u, (const ebf16*)nullptr, nvec, (ebf16*)d_out);
        }
    } else if (dtype == TGT_DTYPE_F32) {
        if (bwd) hipLaunchKernelGGL((k_gelu<float, true>), grid, dim3(kEwBlock), 0, st, (const float*)d_u, (const float*)d_dh, nvec, (float*)d_out);
        else hipLaunchKernelGGL((k_gelu<float, false>), grid, dim3(kEwBlock), 0, st, (const float*)d_u, (const float*)nullptr, nvec, (float*)d_out);
    } else {
        if (bwd) hipLaunchKernelGGL((k_gelu<ebf16, true>), grid, dim3(kEwBlock), 0, st, (const ebf16*)d_u, (const ebf16*)d_dh, nvec, (ebf16*)d_out);
        else hipLaunchKernelGGL((k_gelu<ebf16, false>), grid, dim3(kEwBlock), 0, st, (const ebf16*)d_u, (const ebf16*)nullptr, nvec, (ebf16*)d_out);
    }
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

int tgt_gelu_fwd(const void* d_u, int64_t n, int dtype, void* d_h, void* stream) {
    return gelu_call(d_u, nullptr, n, dtype, d_h, stream, false);
}

int tgt_gelu_bwd(const void* d_u, const void* d_dh, int64_t n, int dtype, void* d_du, void* stream) {
    return gelu_call(d_u, d_dh, n, dtype, d_du, stream, true);
}

int tgt_relu_fwd(const void* d_u, int64_t n, int dtype, void* d_h, void* stream) {
    return gelu_call(d_u, nullptr, n, dtype, d_h, stream, false, true);
}

int tgt_relu_bwd(const void* d_u, const void* d_dh, int64_t n, int dtype, void* d_du, void* stream) {
    return gelu_call(d_u, d_dh, n, dtype, d_du, stream, true, true);
}

}  // extern "C"
