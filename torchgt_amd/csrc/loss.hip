// F.nll_loss(log_probs, target) of the node-level training loop (main_sp_sparse_node_level.py:200, gt_sp/evaluate.py:52):
// reduction 'mean' over the rows whose target is not ignore_index.
//
//   loss = - sum_i log_probs[i, t_i] / count,   d log_probs[i, c] = - dloss / count  where c == t_i, else 0
//
// One row per lane: the forward is a gather of one value per row (N x 8 bytes of targets plus one touched line
// per row), summed per workgroup and then over the workgroups in a fixed order (no atomics: the same inputs give
// the same bits); the backward is one streaming write of [N, C].  A target outside [0, C) that is not ignore_index
// counts as ignored.
#include "common.h"

namespace tgt {
namespace {

constexpr int kLossBlock = 256;
constexpr int kLossWorkers = 1024;      // at most this many workgroups (= partial sums) in the forward

__device__ __forceinline__ float ld(const float* p) { return *p; }
__device__ __forceinline__ float ld(const uint16_t* p) { return __uint_as_float((uint32_t)*p << 16); }
__device__ __forceinline__ void st(float* p, float v) { *p = v; }
__device__ __forceinline__ void st(uint16_t* p, float v) {
    const __bf16 b = static_cast<__bf16>(v);
    *p = __builtin_bit_cast(uint16_t, b);
}

template <typename T>
__global__ __launch_bounds__(kLossBlock) void k_nll_fwd(const T* __restrict__ logp, const int64_t* __restrict__ target, int64_t N,
                                                         int C, int64_t ignore_index, float* __restrict__ partial) {
    __shared__ float red[kLossBlock / 64];
    __shared__ int cnt[kLossBlock / 64];
    float s = 0.f;
    int n = 0;      // rows counted as integers: a float count is exact only up to 2^24 rows
    for (int64_t i = (int64_t)blockIdx.x * kLossBlock + threadIdx.x; i < N; i += (int64_t)gridDim.x * kLossBlock) {
        const int64_t t = target[i];
        if (t != ignore_index && t >= 0 && t < C) { s += ld(logp + i * C + t); n += 1; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) { s += __shfl_xor(s, o); n += __shfl_xor(n, o); }
    if ((threadIdx.x & 63) == 0) { red[threadIdx.x >> 6] = s; cnt[threadIdx.x >> 6] = n; }
    __syncthreads();
    if (threadIdx.x == 0) {
        float a = 0.f;
        int b = 0;
#pragma unroll
        for (int w = 0; w < kLossBlock / 64; ++w) { a += red[w]; b += cnt[w]; }
        partial[2 * blockIdx.x] = a;
        partial[2 * blockIdx.x + 1] = __int_as_float(b);       // the count travels as its bit pattern
    }
}

// one workgroup: the partials in a fixed order; loss = -sum / count (0 / 0 = nan like torch when every row is ignored)
template <typename T>
__global__ __launch_bounds__(kLossBlock) void k_nll_finish(const float* __restrict__ partial, int workers, T* __restrict__ loss,
                                                            float* __restrict__ count) {
    __shared__ float red[kLossBlock];
    __shared__ long long cnt[kLossBlock];
    float s = 0.f;
    long long n = 0;
    for (int w = threadIdx.x; w < workers; w += kLossBlock) { s += partial[2 * w]; n += __float_as_int(partial[2 * w + 1]); }
    red[threadIdx.x] = s; cnt[threadIdx.x] = n;
    __syncthreads();
    for (int o = kLossBlock / 2; o > 0; o >>= 1) {
        if ((int)threadIdx.x < o) { red[threadIdx.x] += red[threadIdx.x + o]; cnt[threadIdx.x] += cnt[threadIdx.x + o]; }
        __syncthreads();
    }
    if (threadIdx.x == 0) { st(loss, -red[0] / (float)cnt[0]); *count = (float)cnt[0]; }
}

// VE consecutive elements of the flattened [N, C] per lane (N * C is a multiple of VE)
template <typename T, int VE>
__global__ __launch_bounds__(kLossBlock) void k_nll_bwd(const int64_t* __restrict__ target, const T* __restrict__ dloss,
                                                         const float* __restrict__ count, int64_t N, int C, int64_t ignore_index,
                                                         T* __restrict__ dlogp) {
    const float g = -ld(dloss) / *count;
    const int64_t nvec = N * C / VE;
    for (int64_t v = (int64_t)blockIdx.x * kLossBlock + threadIdx.x; v < nvec; v += (int64_t)gridDim.x * kLossBlock) {
        const int64_t e0 = v * VE;
        int64_t r = e0 / C;
        int c = (int)(e0 - r * C);
        int64_t t = target[r];
        T out[VE];
#pragma unroll
        for (int i = 0; i < VE; ++i) {
            st(&out[i], (t == c && t != ignore_index) ? g : 0.f);
            if (++c == C) { c = 0; ++r; t = r < N ? target[r] : -1; }
        }
        if constexpr (sizeof(T) * VE == 16) *reinterpret_cast<uint4*>(dlogp + e0) = *reinterpret_cast<const uint4*>(out);
        else {
#pragma unroll
            for (int i = 0; i < VE; ++i) dlogp[e0 + i] = out[i];
        }
    }
}

int loss_check(int64_t N, int C, int dtype, const char* who) {
    if (N < 0 || C < 1 || N * (int64_t)C >= ((int64_t)1 << 40)) { set_error("%s: bad shape N=%lld C=%d", who, (long long)N, C); return TGT_ERR_INVALID_ARG; }
    if (dtype != TGT_DTYPE_F32 && dtype != TGT_DTYPE_BF16) { set_error("%s: unknown dtype %d", who, dtype); return TGT_ERR_INVALID_ARG; }
    return TGT_OK;
}

int fwd_workers(int64_t N) { return (int)std::max<int64_t>(1, std::min<int64_t>((N + kLossBlock - 1) / kLossBlock, kLossWorkers)); }

}  // namespace
}  // namespace tgt

extern "C" {

int64_t tgt_nll_loss_workspace_bytes(int64_t N) { return N >= 0 ? (int64_t)sizeof(float) * 2 * tgt::fwd_workers(N) : -1; }

int tgt_nll_loss_fwd(const void* d_log_probs, const int64_t* d_target, int64_t N, int C, int dtype, int64_t ignore_index, void* d_loss,
                     float* d_count, void* d_workspace, int64_t workspace_bytes, void* stream) {
    using namespace tgt;
    const int rc = loss_check(N, C, dtype, "tgt_nll_loss_fwd");
    if (rc != TGT_OK) return rc;
    if (!d_loss || !d_count || (N > 0 && (!d_log_probs || !d_target))) { set_error("tgt_nll_loss_fwd: null pointer"); return TGT_ERR_INVALID_ARG; }
    if (!d_workspace || workspace_bytes < tgt_nll_loss_workspace_bytes(N) || ((uintptr_t)d_workspace & 3)) {
        set_error("tgt_nll_loss_fwd: workspace of %lld bytes needed, got %lld", (long long)tgt_nll_loss_workspace_bytes(N), (long long)workspace_bytes);
        return TGT_ERR_WORKSPACE;
    }
    hipStream_t st = (hipStream_t)stream;
    const int workers = fwd_workers(N);
    float* partial = (float*)d_workspace;
    KernelTimer t(KS_LOSS, st);
    if (dtype == TGT_DTYPE_F32) {
        hipLaunchKernelGGL((k_nll_fwd<float>), dim3(workers), dim3(kLossBlock), 0, st, (const float*)d_log_probs, d_target, N, C, ignore_index, partial);
        hipLaunchKernelGGL((k_nll_finish<float>), dim3(1), dim3(kLossBlock), 0, st, partial, workers, (float*)d_loss, d_count);
    } else {
        hipLaunchKernelGGL((k_nll_fwd<uint16_t>), dim3(workers), dim3(kLossBlock), 0, st, (const uint16_t*)d_log_probs, d_target, N, C, ignore_index, partial);
        hipLaunchKernelGGL((k_nll_finish<uint16_t>), dim3(1), dim3(kLossBlock), 0, st, partial, workers, (uint16_t*)d_loss, d_count);
    }
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

int tgt_nll_loss_bwd(const int64_t* d_target, const void* d_dloss, const float* d_count, int64_t N, int C, int dtype, int64_t ignore_index,
                     void* d_dlog_probs, void* stream) {
    using namespace tgt;
    const int rc = loss_check(N, C, dtype, "tgt_nll_loss_bwd");
    if (rc != TGT_OK) return rc;
    if (N == 0) return TGT_OK;
    if (!d_target || !d_dloss || !d_count || !d_dlog_probs) { set_error("tgt_nll_loss_bwd: null pointer"); return TGT_ERR_INVALID_ARG; }
    hipStream_t st = (hipStream_t)stream;
    const int64_t total = N * C;
    const int full = dtype == TGT_DTYPE_F32 ? 4 : 8;
    const bool vec = total % full == 0 && ((uintptr_t)d_dlog_probs & 15) == 0;
    const int64_t nvec = vec ? total / full : total;
    const dim3 grid((unsigned)std::max<int64_t>(1, std::min<int64_t>((nvec + kLossBlock - 1) / kLossBlock, 16384)));
    KernelTimer t(KS_LOSS, st);
#define LAUNCH(T, VE) hipLaunchKernelGGL((k_nll_bwd<T, VE>), grid, dim3(kLossBlock), 0, st, d_target, (const T*)d_dloss, d_count, N, C, ignore_index, (T*)d_dlog_probs)
    if (dtype == TGT_DTYPE_F32) { if (vec) LAUNCH(float, 4); else LAUNCH(float, 1); }
    else { if (vec) LAUNCH(uint16_t, 8); else LAUNCH(uint16_t, 1); }
#undef LAUNCH
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

}  // extern "C"
