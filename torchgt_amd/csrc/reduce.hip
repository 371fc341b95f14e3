// Sums of per-workgroup partials, several of them in one launch.
//
// The weight-gradient kernels of the projections (linear.hip) and the LayerNorm backward (elementwise.hip) leave
// one float partial per workgroup, [workers][n], and the result is their sum over the workers in a fixed order: the
// workers are cut into 16 slices, every slice is added in worker order, then the 16 slice sums in slice order - the
// same inputs give the same bits whatever the launch.  A backward pass of an encoder layer has six such sums (four
// linears, two LayerNorms), each a few microseconds of almost nothing but launch latency; tgt_reduce_partials takes
// up to eight of them in one launch (blockIdx.y picks the sum).  The arithmetic of one sum does not depend on what
// else is in the launch.
#include "common.h"

namespace tgt {
namespace {

struct ReduceBatch { tgt_reduce_desc d[8]; };

__device__ __forceinline__ void put(float* p, float v) { *p = v; }
__device__ __forceinline__ void put(uint16_t* p, float v) {
    const __bf16 b = static_cast<__bf16>(v);
    *p = __builtin_bit_cast(uint16_t, b);
}

// 64 consecutive elements x 16 slices of the workers per workgroup
template <typename T>
__global__ __launch_bounds__(1024) void k_reduce_partials(const ReduceBatch b) {
    __shared__ float part[16][64];
    const tgt_reduce_desc& d = b.d[blockIdx.y];
    if ((int)blockIdx.x * 64 >= d.n) return;               // a shorter sum than the longest of the launch
    const int el = threadIdx.x & 63, sl = threadIdx.x >> 6;
    const int e = blockIdx.x * 64 + el;
    const int n = d.n;
    const int w0 = (int)((int64_t)d.workers * sl / 16), w1 = (int)((int64_t)d.workers * (sl + 1) / 16);
    float s = 0.f;
    if (e < n) {
        const float* __restrict__ src = d.partial + e;
        int w = w0;
        for (; w + 8 <= w1; w += 8) {      // eight loads in flight, added in worker order
            float t[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) t[i] = src[(int64_t)(w + i) * n];
#pragma unroll
            for (int i = 0; i < 8; ++i) s += t[i];
        }
        for (; w < w1; ++w) s += src[(int64_t)w * n];
    }
    part[sl][el] = s;
    __syncthreads();
    if (sl == 0 && e < n) {
        float t = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) t += part[i][el];
        int seg = 0;
        for (int i = 1; i < d.n_out; ++i)
            if (e >= d.begin[i]) seg = i;
        if (d.out[seg]) put(reinterpret_cast<T*>(d.out[seg]) + (e - d.begin[seg]), t);
    }
}

}  // namespace

int reduce_partials(const tgt_reduce_desc* descs, int count, int dtype, hipStream_t st) {
    if (count < 1) return TGT_OK;
    if (count > 8 || !descs) { set_error("tgt_reduce_partials: 1 to 8 sums per call"); return TGT_ERR_INVALID_ARG; }
    if (dtype != TGT_DTYPE_F32 && dtype != TGT_DTYPE_BF16) { set_error("tgt_reduce_partials: unknown dtype %d", dtype); return TGT_ERR_INVALID_ARG; }
    ReduceBatch b{};
    int longest = 0;
    for (int i = 0; i < count; ++i) {
        const tgt_reduce_desc& d = descs[i];
        if (!d.partial || d.workers < 1 || d.n < 1 || d.n_out < 1 || d.n_out > 6 || d.begin[0] != 0) {
            set_error("tgt_reduce_partials: descriptor %d is not one a *_deferred call filled in", i);
            return TGT_ERR_INVALID_ARG;
        }
        b.d[i] = d;
        longest = d.n > longest ? d.n : longest;
    }
    KernelTimer t(KS_LINEAR_DW, st);
    const dim3 grid((unsigned)((longest + 63) / 64), (unsigned)count);
    if (dtype == TGT_DTYPE_F32) hipLaunchKernelGGL((k_reduce_partials<float>), grid, dim3(1024), 0, st, b);
    else hipLaunchKernelGGL((k_reduce_partials<uint16_t>), grid, dim3(1024), 0, st, b);
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

}  // namespace tgt

extern "C" int tgt_reduce_partials(const tgt_reduce_desc* descs, int count, int dtype, void* stream) {
    return tgt::reduce_partials(descs, count, dtype, (hipStream_t)stream);
}
