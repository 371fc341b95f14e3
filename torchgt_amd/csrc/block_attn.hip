// Block path: attention over a list of dense 16 x 16 tiles plus a remainder of
// ordinary edges, one softmax per destination.
//
// The reference's cluster reordering replaces the edges of every partition pair
// by dense bs x bs blocks of (source, destination) pairs (gt_sp/utils.py:284-299,
// create_pairs :218-220) and then feeds the expanded edge list to the same
// sparse_attention (attn_module.py:133-189).  Here a block is never expanded: a
// tile (r0, c0) stands for the 256 edges a -> b, a in [r0, r0+16), b in
// [c0, c0+16).  Its scores are one 16x16 matrix product per head on the matrix
// cores (v_mfma_f32_16x16x16_bf16_1k, K and V rows of the tile read once for 16
// destinations), and because the reference's softmax has no max subtraction the
// tile sums (sum w v, Z) simply add to the sums of the remaining edges: the tile
// kernels leave fp32 partial sums per node and the sparse kernels add them when
// they write the row (forward) or the gradient row (backward).
//
// Layouts of the matrix instruction (lane l, col = l % 16, kq = l / 16):
//   A 16x16: A[col][4kq .. 4kq+3]      B 16x16: B[4kq .. 4kq+3][col]
//   C 16x16: register r holds C[4kq + r][col]
// Scores are formed transposed (rows = sources, col = destination) so that the
// weights sit in the B layout of the next product.
#include "common.h"
#include <algorithm>
#include <vector>
#include <new>

namespace tgt {

typedef short bshort4 __attribute__((ext_vector_type(4)));
typedef float bfloat4 __attribute__((ext_vector_type(4)));
struct tbf16 { uint16_t x; };

__device__ __forceinline__ short t_f2bf(float f) {
    const __bf16 b = static_cast<__bf16>(f);
    return __builtin_bit_cast(short, b);
}
__device__ __forceinline__ bshort4 t_ld4(const tbf16* p) { return *reinterpret_cast<const bshort4*>(p); }
__device__ __forceinline__ bshort4 t_ld4(const float* p) {
    const bfloat4 f = *reinterpret_cast<const bfloat4*>(p);
    bshort4 r;
    r.x = t_f2bf(f.x); r.y = t_f2bf(f.y); r.z = t_f2bf(f.z); r.w = t_f2bf(f.w);
    return r;
}
__device__ __forceinline__ short t_ld1(const tbf16* p) { return (short)p->x; }
__device__ __forceinline__ short t_ld1(const float* p) { return t_f2bf(*p); }
__device__ __forceinline__ bshort4 t_zero4() { bshort4 z; z.x = 0; z.y = 0; z.z = 0; z.w = 0; return z; }
__device__ __forceinline__ bfloat4 t_zerof() { bfloat4 z; z.x = 0.f; z.y = 0.f; z.z = 0.f; z.w = 0.f; return z; }
// the operand of the lanes whose four elements lie beyond the head's D must be zero whatever the memory holds
// (0 x Inf would not be): an AND with 0 or ~0 instead of a load under a lane mask
__device__ __forceinline__ bshort4 t_and4(bshort4 v, int m) {
    typedef int i2 __attribute__((ext_vector_type(2)));
    i2 x = __builtin_bit_cast(i2, v);
    x.x &= m; x.y &= m;
    return __builtin_bit_cast(bshort4, x);
}
__device__ __forceinline__ bfloat4 mfma16(bshort4 a, bshort4 b, bfloat4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, b, c, 0, 0, 0);
}
// exp(clamp(s / sqrt(d), -5, 5)) (attn_module.py:160-161) from x2 = s * log2(e) / sqrt(d): one multiply, a median of
// three and the hardware's exp2 (its argument stays within +-7.3); NaN stays NaN, like torch.clamp
constexpr float kLog2e = 1.44269504088896340736f;
constexpr float kClamp2 = 5.0f * kLog2e;
__device__ __forceinline__ float t_weight(float x2) {
    const float w = __builtin_amdgcn_exp2f(__builtin_amdgcn_fmed3f(x2, -kClamp2, kClamp2));
    return x2 != x2 ? x2 : w;
}
// the clamp lets a gradient through where the score is inside [-5, 5] (inclusive, like torch.clamp's backward)
__device__ __forceinline__ bool t_inside(float x2) { return fabsf(x2) <= kClamp2; }
// four floats -> four bf16 (round to nearest even), two values per conversion instruction
__device__ __forceinline__ int t_cvt_pk(float lo, float hi) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    f32x2 x;
    x.x = lo; x.y = hi;
    return __builtin_bit_cast(int, __builtin_convertvector(x, bf16x2));
}
__device__ __forceinline__ bshort4 t_pack(const float (&x)[4]) {
    typedef int i2 __attribute__((ext_vector_type(2)));
    i2 r;
    r.x = t_cvt_pk(x[0], x[1]);
    r.y = t_cvt_pk(x[2], x[3]);
    return __builtin_bit_cast(bshort4, r);
}
constexpr int kTile = 16;
constexpr float kTileEps = 1e-6f;   // attn_module.py:187

__device__ __forceinline__ void t_st4(float* p, float a, float b, float c, float d) {
    bfloat4 r; r.x = a; r.y = b; r.z = c; r.w = d;
    *reinterpret_cast<bfloat4*>(p) = r;
}
__device__ __forceinline__ void t_st4(tbf16* p, float a, float b, float c, float d) {
    const float x[4] = {a, b, c, d};
    *reinterpret_cast<bshort4*>(p) = t_pack(x);
}

// Rows no tile covers get zeros when the tile kernels write final results (no remaining edges, or a plan of the
// remaining edges that schedules only rows with edges: then the rows without, rem_rowptr[row + 1] ==
// rem_rowptr[row]).  The rows are listed when the tile set is built; the workgroups behind the last tile group of
// a launch write them (eight lanes per row, 16-byte stores), so they cost no launch of their own.
struct BareRows {
    const int32_t* rows;
    int32_t n_rows;
    int32_t first_block;       // workgroups from here on zero rows instead of walking tiles
};
template <typename T>
__device__ __forceinline__ void zero_bare_rows(const BareRows& br, int HD, int H, T* __restrict__ a, T* __restrict__ b,
                                               float* __restrict__ Z, const int32_t* __restrict__ rem_rowptr) {
    const int per_block = blockDim.x / 8;
    const int64_t i = (int64_t)(blockIdx.x - br.first_block) * per_block + threadIdx.x / 8;
    const int part = threadIdx.x % 8;
    if (i >= br.n_rows) return;
    const int64_t row = br.rows[i];
    if (rem_rowptr && rem_rowptr[row + 1] != rem_rowptr[row]) return;      // the sparse kernels write this row
    const int bytes = HD * (int)sizeof(T);                 // a multiple of 16: HD is a multiple of 8
    const uint4 z4 = make_uint4(0u, 0u, 0u, 0u);
    for (int o = part * 16; o < bytes; o += 128) {
        if (a) *reinterpret_cast<uint4*>(reinterpret_cast<char*>(a + row * HD) + o) = z4;
        if (b) *reinterpret_cast<uint4*>(reinterpret_cast<char*>(b + row * HD) + o) = z4;
    }
    if (Z) for (int h = part; h < H; h += 8) Z[row * H + h] = 0.f;
}
// Waves per SIMD the kernels are compiled for (the register budget follows from it).  Without a bound the compiler
// budgets 512 registers, puts the matrix accumulators into AGPRs and copies them around every matrix instruction.
#ifndef TGT_TILE_FWD_OCC
#define TGT_TILE_FWD_OCC 4
#endif
#ifndef TGT_TILE_DST_OCC
#define TGT_TILE_DST_OCC 4
#endif
#ifndef TGT_TILE_SRC_OCC
#define TGT_TILE_SRC_OCC 4
#endif
template <int HDL> constexpr int fwd_occupancy() { return TGT_TILE_FWD_OCC; }
template <typename T, int HDL> constexpr int dst_occupancy() { return TGT_TILE_DST_OCC; }
// Heads one wave works on.  A group of tiles is shared out over H / heads_per_wave waves, each with its own 32
// elements of every row (four heads of 8, two of 16): half the accumulators and half the LDS per wave of what all
// eight heads took, so that twice the waves are resident - the kernels wait on chains of loads, LDS and matrix steps,
// and the number of waves in flight is what hides them.  Each wave stages just its 64-byte share of the rows.
#ifndef TGT_TILE_HDL
#define TGT_TILE_HDL 32
#endif
template <int D, int H> constexpr int heads_per_wave() { return H * D <= TGT_TILE_HDL ? H : (TGT_TILE_HDL / D > 0 ? TGT_TILE_HDL / D : 1); }
// waves (= tile groups) per workgroup of the tile kernels: as many as keep the static LDS under 64 KB
template <int HDL> constexpr int tile_waves() { return 4; }

// LDS images of a block of 16 node rows (all heads, HD = H*D elements per row, bf16 bits):
//   row-major   rm[row * (HD + 4) + e]   - the A operand "16 rows x 4 consecutive elements"
//   transposed  tr[e * 20 + row]         - the A operand "element e x 4 consecutive rows"
// The strides (HD + 4 and 20 elements) keep the 8-byte reads of 16 lanes on different banks.
template <int HD> constexpr int rm_size() { return kTile * (HD + 4); }
template <int HD> constexpr int tr_size() { return HD * 20; }

// Coalesced copy of rows row0 .. row0+15 of X ([N, HD]) into the LDS images (either may be null): every lane
// fetches 16-byte pieces of consecutive memory.  Loading and storing are separate steps so that a kernel can ask
// for the rows of all its tensors before it waits for the first of them.
// a piece in registers: eight bf16 values (float inputs are rounded as they arrive)
template <typename T, int HDL> struct RowPieces {
    static constexpr int CPR = HDL / 8;                     // 8-element pieces per row
    static constexpr int ITERS = (kTile * CPR + 63) / 64;
    uint4 p[ITERS];
};
__device__ __forceinline__ void load_piece(const tbf16* p, uint4& r) { r = *reinterpret_cast<const uint4*>(p); }
__device__ __forceinline__ void load_piece(const float* p, uint4& r) {
    const bfloat4 a = *reinterpret_cast<const bfloat4*>(p);
    const bfloat4 b = *reinterpret_cast<const bfloat4*>(p + 4);
    r.x = (uint32_t)t_cvt_pk(a.x, a.y); r.y = (uint32_t)t_cvt_pk(a.z, a.w);
    r.z = (uint32_t)t_cvt_pk(b.x, b.y); r.w = (uint32_t)t_cvt_pk(b.z, b.w);
}
__device__ __forceinline__ void unpack_piece(const uint4& u, short (&v)[8]) {
    v[0] = (short)(u.x & 0xffffu); v[1] = (short)(u.x >> 16);
    v[2] = (short)(u.y & 0xffffu); v[3] = (short)(u.y >> 16);
    v[4] = (short)(u.z & 0xffffu); v[5] = (short)(u.z >> 16);
    v[6] = (short)(u.w & 0xffffu); v[7] = (short)(u.w >> 16);
}
// elements [e_off, e_off + HDL) of rows row0 .. row0 + 15 of X ([N, HD])
template <typename T, int HD, int HDL>
__device__ __forceinline__ void load_rows(const T* __restrict__ X, int row0, int e_off, int lane, RowPieces<T, HDL>& rp) {
    constexpr int CPR = RowPieces<T, HDL>::CPR;
#pragma unroll
    for (int i = 0; i < RowPieces<T, HDL>::ITERS; ++i) {
        const int c = i * 64 + lane;
        // a scalar base (row0 and e_off are the same in all lanes) plus a 32-bit lane offset; the empty statement
        // keeps the sum from being re-associated into a 64-bit address per lane held across the tile loop
        const char* base = reinterpret_cast<const char*>(X) + ((int64_t)row0 * HD + e_off) * (int)sizeof(T);
        asm volatile("" : "+s"(base));
        if (kTile * CPR % 64 == 0 || c < kTile * CPR)
            load_piece(reinterpret_cast<const T*>(base + (uint32_t)(((c / CPR) * HD + (c % CPR) * 8) * (int)sizeof(T))), rp.p[i]);
    }
}
template <typename T, int HDL>
__device__ __forceinline__ void store_rows(const RowPieces<T, HDL>& rp, short* __restrict__ rm, short* __restrict__ tr, int lane) {
    constexpr int CPR = RowPieces<T, HDL>::CPR;
#pragma unroll
    for (int i = 0; i < RowPieces<T, HDL>::ITERS; ++i) {
        const int c = i * 64 + lane;
        if (kTile * CPR % 64 != 0 && c >= kTile * CPR) break;
        const int row = c / CPR, e0 = (c % CPR) * 8;
        short v[8];
        unpack_piece(rp.p[i], v);
        if (rm) {
            bshort4 lo, hi;
            lo.x = v[0]; lo.y = v[1]; lo.z = v[2]; lo.w = v[3];
            hi.x = v[4]; hi.y = v[5]; hi.z = v[6]; hi.w = v[7];
            *reinterpret_cast<bshort4*>(&rm[row * (HDL + 4) + e0]) = lo;
            *reinterpret_cast<bshort4*>(&rm[row * (HDL + 4) + e0 + 4]) = hi;
        }
        if (tr) {
#pragma unroll
            for (int j = 0; j < 8; ++j) tr[(e0 + j) * 20 + row] = v[j];
        }
    }
}
// Whether the next tile's rows are asked for while the current one is worked on: where the pieces in flight fit the
// registers next to the accumulators (2-byte elements)
template <typename T, int HDL> constexpr bool tile_prefetch() { return sizeof(T) == 2 && HDL <= 64; }
// Hides where a scalar came from: addresses formed from the result cannot be computed before this point.  Put
// behind a kernel's tile loop it keeps the epilogue's pointers out of the registers the loop needs.
__device__ __forceinline__ int late_scalar(int x) { asm volatile("" : "+s"(x)); return x; }
// the first lane's value as a scalar: what every lane of a wave holds alike (a group's record) steers loops and
// addresses from scalar registers
__device__ __forceinline__ int wave_uniform(int x) { return __builtin_amdgcn_readfirstlane(x); }
// A operand "rows x 4 consecutive elements": lane (col, kq) reads row `col`, elements e .. e+3
template <int HD>
__device__ __forceinline__ bshort4 a_rows(const short* __restrict__ rm, int col, int e) {
    return *reinterpret_cast<const bshort4*>(&rm[col * (HD + 4) + e]);
}
// A operand "element x 4 consecutive rows": lane reads element e of rows 4kq .. 4kq+3
__device__ __forceinline__ bshort4 a_cols(const short* __restrict__ tr, int e, int kq) {
    return *reinterpret_cast<const bshort4*>(&tr[e * 20 + 4 * kq]);
}
// in-wave ordering of LDS traffic: the images are written and read by the same wave only
__device__ __forceinline__ void wave_lds_fence() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// One wave per group of tiles that share their 16 destinations: sum w v and Z of the tiles, all
// heads at once.  The K and V rows of a tile are staged in LDS once (coalesced) and every head's
// two products take their operands from there.
// FINAL: the tiles are all there is (no remaining edges): the kernel divides by Z + eps and writes
// the output rows and Z themselves; otherwise it does so for the destinations that have no remaining edge and
// leaves fp32 sums of the others for the sparse kernel to add (which skips the former).
template <typename T, int D, int H, bool FINAL>
__global__ __launch_bounds__((64 * tile_waves<heads_per_wave<D, H>() * D>()), (fwd_occupancy<heads_per_wave<D, H>() * D>())) void k_tile_fwd(const int4* __restrict__ grp_rec,
                                                              const int32_t* __restrict__ tile_r0, int n_groups,
                                                              const T* __restrict__ Q, const T* __restrict__ K,
                                                              const T* __restrict__ V, float* __restrict__ acc,
                                                              float* __restrict__ Zp, T* __restrict__ out,
                                                              float* __restrict__ Zout,
                                                              const int32_t* __restrict__ rem_rowptr, const BareRows bare,
                                                              float inv_scale) {
    constexpr int HD = H * D;
    constexpr int HW = heads_per_wave<D, H>(), NP = H / HW, HDL = HW * D;     // this wave's heads: h0 .. h0 + HW - 1
    constexpr int kTileWaves = tile_waves<HDL>();
    constexpr bool kPrefetch = tile_prefetch<T, HDL>();
    const float scale2 = inv_scale * kLog2e;
    __shared__ short lds[kTileWaves * (rm_size<HDL>() + tr_size<HDL>())];
    if ((int)blockIdx.x >= bare.first_block) {      // uniform over the workgroup
        zero_bare_rows<T>(bare, HD, H, out, (T*)nullptr, Zout, rem_rowptr);
        return;
    }
    const int wave = wave_uniform(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int gw = blockIdx.x * kTileWaves + wave;
    const int g = gw / NP, h0 = (gw % NP) * HW;
    if (g >= n_groups) return;
    short* k_rm = lds + wave * (rm_size<HDL>() + tr_size<HDL>());
    short* v_tr = k_rm + rm_size<HDL>();
    const int col = lane & 15, kq = lane >> 4;
    const bool kval = kq * 4 < D;
    const int kmask = kval ? -1 : 0;
    // one 16-byte record per group: (first node, tile range, the first tile's other side) - a wave with one tile, the
    // usual case, needs no second look-up before it can ask for the tile's rows
    const int4 gr = grp_rec[g];
    const int c0 = wave_uniform(gr.x), t0 = wave_uniform(gr.y), t1 = wave_uniform(gr.z);
    int r0 = wave_uniform(gr.w);
    RowPieces<T, HDL> pk, pv;
    load_rows<T, HD, HDL>(K, r0, h0 * D, lane, pk);         // asked for before anything waits
    load_rows<T, HD, HDL>(V, r0, h0 * D, lane, pv);
    bshort4 bq[HW];
#pragma unroll
    for (int h = 0; h < HW; ++h) {
        bq[h] = t_zero4();
        if (kval) bq[h] = t_ld4(Q + (int64_t)(c0 + col) * HD + (h0 + h) * D + kq * 4);
    }
    // a destination without remaining edges (row pointers of the plan that holds them) is finished here as well
    bool fin = true;
    if (!FINAL) fin = rem_rowptr[c0 + col + 1] == rem_rowptr[c0 + col];
    bfloat4 o[HW];
    float z[HW];
#pragma unroll
    for (int h = 0; h < HW; ++h) { o[h] = t_zerof(); z[h] = 0.f; }
    for (int t = t0; t < t1; ++t) {
        if (!kPrefetch && t > t0) {
            r0 = wave_uniform(tile_r0[t]);
            load_rows<T, HD, HDL>(K, r0, h0 * D, lane, pk);
            load_rows<T, HD, HDL>(V, r0, h0 * D, lane, pv);
        }
        wave_lds_fence();                      // the previous tile's reads are done
        store_rows<T, HDL>(pk, k_rm, nullptr, lane);
        store_rows<T, HDL>(pv, nullptr, v_tr, lane);
        wave_lds_fence();
        if (kPrefetch && t + 1 < t1) {         // the next tile's rows travel while this one is worked on
            r0 = wave_uniform(tile_r0[t + 1]);
            load_rows<T, HD, HDL>(K, r0, h0 * D, lane, pk);
            load_rows<T, HD, HDL>(V, r0, h0 * D, lane, pv);
        }
#pragma unroll
        for (int h = 0; h < HW; ++h) {
            // every lane reads (no lane mask around the LDS reads): lanes beyond the head's D get zeros by an AND, and
            // what the rows dd >= D of the second product hold is never stored
            const bshort4 ak = t_and4(a_rows<HDL>(k_rm, col, h * D + (kq * 4) % D), kmask);
            const bfloat4 sc = mfma16(ak, bq[h], t_zerof());       // S^T[source 4kq+r][destination col]
            float w[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                w[r] = t_weight(sc[r] * scale2);
                z[h] += w[r];
            }
            const bshort4 av = a_cols(v_tr, h * D + col % D, kq);
            o[h] = mfma16(av, t_pack(w), o[h]);                    // O^T[dd 4kq+r][destination col]
        }
    }
    const int c0e = late_scalar(c0);
#pragma unroll
    for (int h = 0; h < HW; ++h) {
        float zz = z[h];
        zz += __shfl_xor(zz, 16);
        zz += __shfl_xor(zz, 32);
        if (fin) {
            const float inv = 1.0f / (zz + kTileEps);
            if (kval) t_st4(out + (int64_t)(c0e + col) * HD + (h0 + h) * D + kq * 4, o[h].x * inv, o[h].y * inv, o[h].z * inv, o[h].w * inv);
        } else if (kval) {
            *reinterpret_cast<bfloat4*>(acc + (int64_t)(c0e + col) * HD + (h0 + h) * D + kq * 4) = o[h];
        }
        if (kq == 0) (fin ? Zout : Zp)[(int64_t)(c0e + col) * H + h0 + h] = zz;
    }
}

// Same grouping: dQ of the tiles.  nd[i,h] = (1/(Z+eps), dout.out) of the FINAL output.
template <typename T, int D, int H, bool FINAL>
__global__ __launch_bounds__((64 * tile_waves<heads_per_wave<D, H>() * D>()), (dst_occupancy<T, heads_per_wave<D, H>() * D>())) void k_tile_bwd_dst(const int4* __restrict__ grp_rec,
                                                                  const int32_t* __restrict__ tile_r0, int n_groups,
                                                                  const T* __restrict__ Q, const T* __restrict__ K,
                                                                  const T* __restrict__ V, const T* __restrict__ dO,
                                                                  const float2* __restrict__ nd,
                                                                  float* __restrict__ dq_part, T* __restrict__ dq_out,
                                                                  const int32_t* __restrict__ rem_rowptr,
                                                                  const BareRows bare, float inv_scale) {
    constexpr int HD = H * D;
    constexpr int HW = heads_per_wave<D, H>(), NP = H / HW, HDL = HW * D;     // this wave's heads: h0 .. h0 + HW - 1
    constexpr int kTileWaves = tile_waves<HDL>();
    constexpr bool kPrefetch = tile_prefetch<T, HDL>();
    const float scale2 = inv_scale * kLog2e;
    constexpr int PER_WAVE = 2 * rm_size<HDL>() + tr_size<HDL>();
    __shared__ short lds[kTileWaves * PER_WAVE];
    if ((int)blockIdx.x >= bare.first_block) {
        zero_bare_rows<T>(bare, HD, H, dq_out, (T*)nullptr, (float*)nullptr, rem_rowptr);
        return;
    }
    const int wave = wave_uniform(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int gw = blockIdx.x * kTileWaves + wave;
    const int g = gw / NP, h0 = (gw % NP) * HW;
    if (g >= n_groups) return;
    short* k_rm = lds + wave * PER_WAVE;
    short* v_rm = k_rm + rm_size<HDL>();
    short* k_tr = v_rm + rm_size<HDL>();
    const int col = lane & 15, kq = lane >> 4;
    const bool kval = kq * 4 < D;
    // one 16-byte record per group: (first node, tile range, the first tile's other side) - a wave with one tile, the
    // usual case, needs no second look-up before it can ask for the tile's rows
    const int4 gr = grp_rec[g];
    const int c0 = wave_uniform(gr.x), t0 = wave_uniform(gr.y), t1 = wave_uniform(gr.z);
    int r0 = wave_uniform(gr.w);
    RowPieces<T, HDL> pk, pv;
    load_rows<T, HD, HDL>(K, r0, h0 * D, lane, pk);
    load_rows<T, HD, HDL>(V, r0, h0 * D, lane, pv);
    bool fin = true;                            // no remaining edge into this row
    if (!FINAL) fin = rem_rowptr[c0 + col + 1] == rem_rowptr[c0 + col];
    bshort4 bq[HW], bg[HW];
    float2 ndv[HW];
    bfloat4 dq[HW];
#pragma unroll
    for (int h = 0; h < HW; ++h) {
        bq[h] = t_zero4(); bg[h] = t_zero4();
        if (kval) {
            bq[h] = t_ld4(Q + (int64_t)(c0 + col) * HD + (h0 + h) * D + kq * 4);
            bg[h] = t_ld4(dO + (int64_t)(c0 + col) * HD + (h0 + h) * D + kq * 4);
        }
        ndv[h] = nd[(int64_t)(c0 + col) * H + h0 + h];
        dq[h] = t_zerof();
    }
    for (int t = t0; t < t1; ++t) {
        if (!kPrefetch && t > t0) {
            r0 = wave_uniform(tile_r0[t]);
            load_rows<T, HD, HDL>(K, r0, h0 * D, lane, pk);
            load_rows<T, HD, HDL>(V, r0, h0 * D, lane, pv);
        }
        wave_lds_fence();
        store_rows<T, HDL>(pk, k_rm, k_tr, lane);
        store_rows<T, HDL>(pv, v_rm, nullptr, lane);
        wave_lds_fence();
        if (kPrefetch && t + 1 < t1) {
            r0 = wave_uniform(tile_r0[t + 1]);
            load_rows<T, HD, HDL>(K, r0, h0 * D, lane, pk);
            load_rows<T, HD, HDL>(V, r0, h0 * D, lane, pv);
        }
#pragma unroll
        for (int h = 0; h < HW; ++h) {
            // operands of the lanes beyond the head's D: reads under a lane mask here - read by all lanes as in the
            // forward, the compiler moves more reads to the front than the registers of this occupancy hold
            bshort4 ak = t_zero4(), av = t_zero4();
            if (kval) {
                ak = a_rows<HDL>(k_rm, col, h * D + kq * 4);
                av = a_rows<HDL>(v_rm, col, h * D + kq * 4);
            }
            const bfloat4 sc = mfma16(ak, bq[h], t_zerof());       // S^T[source][destination]
            const bfloat4 dp = mfma16(av, bg[h], t_zerof());       // dP^T = V dout^T
            float md[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float x2 = sc[r] * scale2;
                const float dS = t_weight(x2) * ndv[h].x * (dp[r] - ndv[h].y);
                md[r] = t_inside(x2) ? dS : 0.f;
            }
            bshort4 akT = t_zero4();
            if (col < D) akT = a_cols(k_tr, h * D + col, kq);
            dq[h] = mfma16(akT, t_pack(md), dq[h]);                // dQ^T[dd][destination] += K^T (m dS)^T
        }
    }
    const int c0e = late_scalar(c0);
    if (kval) {
#pragma unroll
        for (int h = 0; h < HW; ++h) {
            bfloat4 o;
            o.x = dq[h].x * inv_scale; o.y = dq[h].y * inv_scale; o.z = dq[h].z * inv_scale; o.w = dq[h].w * inv_scale;
            if (fin) t_st4(dq_out + (int64_t)(c0e + col) * HD + (h0 + h) * D + kq * 4, o.x, o.y, o.z, o.w);
            else *reinterpret_cast<bfloat4*>(dq_part + (int64_t)(c0e + col) * HD + (h0 + h) * D + kq * 4) = o;
        }
    }
}

// One wave per group of tiles that share their 16 SOURCES: dK and dV of the tiles.
template <typename T, int D, int H, bool FINAL>
__global__ __launch_bounds__((64 * tile_waves<heads_per_wave<D, H>() * D>()), TGT_TILE_SRC_OCC) void k_tile_bwd_src(const int4* __restrict__ grp_rec,
                                                                  const int32_t* __restrict__ tile_c0, int n_groups,
                                                                  const T* __restrict__ Q, const T* __restrict__ K,
                                                                  const T* __restrict__ V, const T* __restrict__ dO,
                                                                  const float2* __restrict__ nd,
                                                                  float* __restrict__ dk_part,
                                                                  float* __restrict__ dv_part, T* __restrict__ dk_out,
                                                                  T* __restrict__ dv_out,
                                                                  const int32_t* __restrict__ rem_rowptr, const BareRows bare,
                                                                  float inv_scale) {
    constexpr int HD = H * D;
    constexpr int HW = heads_per_wave<D, H>(), NP = H / HW, HDL = HW * D;     // this wave's heads: h0 .. h0 + HW - 1
    constexpr int kTileWaves = tile_waves<HDL>();
    constexpr bool kPrefetch = tile_prefetch<T, HDL>();
    const float scale2 = inv_scale * kLog2e;
    constexpr int PER_WAVE = 2 * rm_size<HDL>() + 2 * tr_size<HDL>() + 4 * kTile * HW;   // + nd tile (float2 = 4 shorts)
    __shared__ __align__(16) short lds[kTileWaves * PER_WAVE];
    if ((int)blockIdx.x >= bare.first_block) {
        zero_bare_rows<T>(bare, HD, H, dk_out, dv_out, (float*)nullptr, rem_rowptr);
        return;
    }
    const int wave = wave_uniform(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int gw = blockIdx.x * kTileWaves + wave;
    const int g = gw / NP, h0 = (gw % NP) * HW;
    if (g >= n_groups) return;
    short* q_rm = lds + wave * PER_WAVE;
    short* g_rm = q_rm + rm_size<HDL>();
    short* q_tr = g_rm + rm_size<HDL>();
    short* g_tr = q_tr + tr_size<HDL>();
    float2* nd_l = reinterpret_cast<float2*>(g_tr + tr_size<HDL>());     // [16 destinations][HW]
    const int col = lane & 15, kq = lane >> 4;
    const bool kval = kq * 4 < D;
    const int4 gr = grp_rec[g];
    const int r0 = wave_uniform(gr.x), t0 = wave_uniform(gr.y), t1 = wave_uniform(gr.z);
    int c0 = wave_uniform(gr.w);
    RowPieces<T, HDL> pq, pg;
    load_rows<T, HD, HDL>(Q, c0, h0 * D, lane, pq);
    load_rows<T, HD, HDL>(dO, c0, h0 * D, lane, pg);
    constexpr int ND_ITERS = (kTile * HW + 63) / 64;
    float2 ndr[ND_ITERS];
    // entry e of the [16][HW] tile: destination c0 + e / HW, head h0 + e % HW
    auto load_nd = [&](const int cc) {
#pragma unroll
        for (int i = 0; i < ND_ITERS; ++i) {
            const int e = i * 64 + lane;
            if (kTile * HW % 64 == 0 || e < kTile * HW) ndr[i] = nd[(int64_t)(cc + e / HW) * H + h0 + e % HW];
        }
    };
    load_nd(c0);
    bool fin = true;                            // no remaining edge out of this row
    if (!FINAL) fin = rem_rowptr[r0 + col + 1] == rem_rowptr[r0 + col];
    bshort4 bk[HW], bv[HW];
    bfloat4 dk[HW], dv[HW];
#pragma unroll
    for (int h = 0; h < HW; ++h) {
        bk[h] = t_zero4(); bv[h] = t_zero4();
        if (kval) {
            bk[h] = t_ld4(K + (int64_t)(r0 + col) * HD + (h0 + h) * D + kq * 4);
            bv[h] = t_ld4(V + (int64_t)(r0 + col) * HD + (h0 + h) * D + kq * 4);
        }
        dk[h] = t_zerof(); dv[h] = t_zerof();
    }
    for (int t = t0; t < t1; ++t) {
        if (!kPrefetch && t > t0) {
            c0 = wave_uniform(tile_c0[t]);
            load_rows<T, HD, HDL>(Q, c0, h0 * D, lane, pq);
            load_rows<T, HD, HDL>(dO, c0, h0 * D, lane, pg);
            load_nd(c0);
        }
        wave_lds_fence();
        store_rows<T, HDL>(pq, q_rm, q_tr, lane);
        store_rows<T, HDL>(pg, g_rm, g_tr, lane);
#pragma unroll
        for (int i = 0; i < ND_ITERS; ++i)
            if (kTile * HW % 64 == 0 || i * 64 + lane < kTile * HW) nd_l[i * 64 + lane] = ndr[i];
        wave_lds_fence();
        if (kPrefetch && t + 1 < t1) {
            c0 = wave_uniform(tile_c0[t + 1]);
            load_rows<T, HD, HDL>(Q, c0, h0 * D, lane, pq);
            load_rows<T, HD, HDL>(dO, c0, h0 * D, lane, pg);
            load_nd(c0);
        }
#pragma unroll
        for (int h = 0; h < HW; ++h) {
            bshort4 aq = t_zero4(), ag = t_zero4();
            if (kval) {
                aq = a_rows<HDL>(q_rm, col, h * D + kq * 4);
                ag = a_rows<HDL>(g_rm, col, h * D + kq * 4);
            }
            const bfloat4 sc = mfma16(aq, bk[h], t_zerof());       // S[destination 4kq+r][source col]
            const bfloat4 dp = mfma16(ag, bv[h], t_zerof());       // dP = dout V^T
            float pw[4], md[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float2 ndv = nd_l[(4 * kq + r) * HW + h];
                const float x2 = sc[r] * scale2;
                const float p = t_weight(x2) * ndv.x;
                const float dS = p * (dp[r] - ndv.y);
                pw[r] = p;
                md[r] = t_inside(x2) ? dS : 0.f;
            }
            bshort4 agT = t_zero4(), aqT = t_zero4();
            if (col < D) {
                agT = a_cols(g_tr, h * D + col, kq);
                aqT = a_cols(q_tr, h * D + col, kq);
            }
            dv[h] = mfma16(agT, t_pack(pw), dv[h]);                // dV^T[dd][source] += dout^T p
            dk[h] = mfma16(aqT, t_pack(md), dk[h]);                // dK^T[dd][source] += Q^T (m dS)
        }
    }
    const int r0e = late_scalar(r0);
    if (kval) {
#pragma unroll
        for (int h = 0; h < HW; ++h) {
            bfloat4 o;
            o.x = dk[h].x * inv_scale; o.y = dk[h].y * inv_scale; o.z = dk[h].z * inv_scale; o.w = dk[h].w * inv_scale;
            if (fin) {
                t_st4(dk_out + (int64_t)(r0e + col) * HD + (h0 + h) * D + kq * 4, o.x, o.y, o.z, o.w);
                t_st4(dv_out + (int64_t)(r0e + col) * HD + (h0 + h) * D + kq * 4, dv[h].x, dv[h].y, dv[h].z, dv[h].w);
            } else {
                *reinterpret_cast<bfloat4*>(dk_part + (int64_t)(r0e + col) * HD + (h0 + h) * D + kq * 4) = o;
                *reinterpret_cast<bfloat4*>(dv_part + (int64_t)(r0e + col) * HD + (h0 + h) * D + kq * 4) = dv[h];
            }
        }
    }
}

}  // namespace tgt

// Tiles grouped by destination block and by source block.
struct tgt_tiles {
    int64_t N = 0, T = 0;
    int32_t n_dst_groups = 0, n_src_groups = 0;
    tgt::DevBuf dst_c0, dst_off, dst_r0;     // [G], [G+1], [T]
    tgt::DevBuf dst_rec, src_rec;            // [G] / [Gs] int4 (group's first node, off[g], off[g + 1], first tile's other side)
    tgt::DevBuf src_r0, src_off, src_c0;     // [Gs], [Gs+1], [T]
    tgt::DevBuf cover_dst, cover_src;        // [N] bytes
    tgt::DevBuf bare_dst, bare_src;          // the rows cover_* marks 0
    int64_t n_bare_dst = 0, n_bare_src = 0;
};

namespace tgt {

static inline int64_t a256(int64_t x) { return (x + 255) & ~(int64_t)255; }

struct BlockWs { int64_t acc, Z, dq, dk, dv, sparse, total; };
static BlockWs block_ws(const tgt_tiles* tl, const tgt_plan* plan, int H, int d) {
    const int64_t nhd = a256(tl->N * H * d * 4), nh = a256(tl->N * H * 4);
    BlockWs w;
    w.acc = 0;
    w.Z = w.acc + nhd;
    w.dq = w.Z + nh;
    w.dk = w.dq + nhd;
    w.dv = w.dk + nhd;
    w.sparse = w.dv + nhd;
    w.total = w.sparse + tgt_sparse_attn_workspace_bytes(plan, H, d);
    return w;
}

// group (key, other) pairs by key; keys of different groups must be >= 16 apart
static int group_tiles(const std::vector<std::pair<int32_t, int32_t>>& pairs, int64_t N, const char* what,
                       std::vector<int32_t>& keys, std::vector<int32_t>& off, std::vector<int32_t>& others,
                       std::vector<uint8_t>& cover) {
    std::vector<std::pair<int32_t, int32_t>> s(pairs);
    std::stable_sort(s.begin(), s.end(), [](const auto& a, const auto& b) { return a.first < b.first; });
    cover.assign((size_t)N, 0);
    for (size_t i = 0; i < s.size(); ++i) {
        if (i == 0 || s[i].first != s[i - 1].first) {
            if (i > 0 && s[i].first - s[i - 1].first < kTile) {
                set_error("tiles: %s blocks starting at %d and %d overlap partially", what, s[i - 1].first, s[i].first);
                return TGT_ERR_INVALID_ARG;
            }
            keys.push_back(s[i].first);
            off.push_back((int32_t)i);
            for (int j = 0; j < kTile; ++j) cover[(size_t)s[i].first + j] = 1;
        }
        others.push_back(s[i].second);
    }
    off.push_back((int32_t)s.size());
    return TGT_OK;
}

template <typename X>
static int upload(DevBuf& b, const std::vector<X>& v, hipStream_t st) {
    TGT_HIP_CHECK(b.alloc(sizeof(X) * (v.size() + 1)));
    if (!v.empty()) TGT_HIP_CHECK(hipMemcpyAsync(b.p, v.data(), sizeof(X) * v.size(), hipMemcpyHostToDevice, st));
    return TGT_OK;
}

// `final_out` non-null: the tiles are all there is; the kernels write final results (and zeros on
// rows without tiles) and the sparse kernels are not run.
template <typename T, int D, int H>
static int tile_fwd_launch_s(const tgt_tiles* tl, const void* q, const void* k, const void* v, float* acc, float* Zp,
                             void* final_out, void* out, float* Zout, const int32_t* rem_rowptr, bool zero_rows, hipStream_t st) {
    constexpr int NP = H / heads_per_wave<D, H>();          // waves per group
    constexpr int W = tile_waves<heads_per_wave<D, H>() * D>();
    const float inv_scale = 1.0f / sqrtf((float)D);
    KernelTimer t(KS_TILE_FWD, st);
    const int gblocks = (tl->n_dst_groups * NP + W - 1) / W;
    const dim3 block(64 * W);
    // the rows without tiles are zeroed by workgroups appended to the same launch: all of them when the tiles are all
    // there is, else (zero_rows: the plan of the remaining edges schedules only rows with edges) those without edges
    const int per = 64 * W / 8, zblocks = final_out || zero_rows ? (int)((tl->n_bare_dst + per - 1) / per) : 0;
    const BareRows bare{tl->bare_dst.as<int32_t>(), (int32_t)tl->n_bare_dst, zblocks ? gblocks : 0x7fffffff};
    if (gblocks + zblocks == 0) return TGT_OK;
    if (final_out) {
        hipLaunchKernelGGL((k_tile_fwd<T, D, H, true>), dim3(gblocks + zblocks), block, 0, st, tl->dst_rec.as<int4>(), tl->dst_r0.as<int32_t>(), tl->n_dst_groups, (const T*)q,
                           (const T*)k, (const T*)v, acc, Zp, (T*)final_out, Zp, (const int32_t*)nullptr, bare, inv_scale);
    } else {
        hipLaunchKernelGGL((k_tile_fwd<T, D, H, false>), dim3(gblocks + zblocks), block, 0, st, tl->dst_rec.as<int4>(), tl->dst_r0.as<int32_t>(), tl->n_dst_groups, (const T*)q,
                           (const T*)k, (const T*)v, acc, Zp, (T*)out, Zout, rem_rowptr, bare, inv_scale);
    }
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

template <typename T, int D, int H>
static int tile_bwd_launch_s(const tgt_tiles* tl, const void* q, const void* k, const void* v, const void* dout,
                             const float2* nd, float* dq, float* dk, float* dv, void* f_dq, void* f_dk, void* f_dv,
                             void* o_dq, void* o_dk, void* o_dv, const int32_t* rem_dst, const int32_t* rem_src,
                             bool zero_rows, hipStream_t st) {
    constexpr int NP = H / heads_per_wave<D, H>();          // waves per group
    constexpr int W = tile_waves<heads_per_wave<D, H>() * D>();
    const float inv_scale = 1.0f / sqrtf((float)D);
    KernelTimer t(KS_TILE_BWD, st);
    const int gdb = (tl->n_dst_groups * NP + W - 1) / W, gsb = (tl->n_src_groups * NP + W - 1) / W;
    const dim3 block(64 * W);
    const bool zr = f_dq || zero_rows;
    const int per = 64 * W / 8;
    const int zd = zr ? (int)((tl->n_bare_dst + per - 1) / per) : 0, zs = zr ? (int)((tl->n_bare_src + per - 1) / per) : 0;
    const BareRows bare_d{tl->bare_dst.as<int32_t>(), (int32_t)tl->n_bare_dst, zd ? gdb : 0x7fffffff};
    const BareRows bare_s{tl->bare_src.as<int32_t>(), (int32_t)tl->n_bare_src, zs ? gsb : 0x7fffffff};
    if (f_dq) {
        if (gdb + zd > 0)
            hipLaunchKernelGGL((k_tile_bwd_dst<T, D, H, true>), dim3(gdb + zd), block, 0, st, tl->dst_rec.as<int4>(), tl->dst_r0.as<int32_t>(), tl->n_dst_groups, (const T*)q,
                               (const T*)k, (const T*)v, (const T*)dout, nd, dq, (T*)f_dq, (const int32_t*)nullptr, bare_d,
                               inv_scale);
        if (gsb + zs > 0)
            hipLaunchKernelGGL((k_tile_bwd_src<T, D, H, true>), dim3(gsb + zs), block, 0, st, tl->src_rec.as<int4>(), tl->src_c0.as<int32_t>(), tl->n_src_groups, (const T*)q,
                               (const T*)k, (const T*)v, (const T*)dout, nd, dk, dv, (T*)f_dk, (T*)f_dv,
                               (const int32_t*)nullptr, bare_s, inv_scale);
    } else {
        if (gdb + zd > 0)
            hipLaunchKernelGGL((k_tile_bwd_dst<T, D, H, false>), dim3(gdb + zd), block, 0, st, tl->dst_rec.as<int4>(), tl->dst_r0.as<int32_t>(), tl->n_dst_groups, (const T*)q,
                               (const T*)k, (const T*)v, (const T*)dout, nd, dq, (T*)o_dq, rem_dst, bare_d, inv_scale);
        if (gsb + zs > 0)
            hipLaunchKernelGGL((k_tile_bwd_src<T, D, H, false>), dim3(gsb + zs), block, 0, st, tl->src_rec.as<int4>(), tl->src_c0.as<int32_t>(), tl->n_src_groups, (const T*)q,
                               (const T*)k, (const T*)v, (const T*)dout, nd, dk, dv, (T*)o_dk, (T*)o_dv, rem_src, bare_s,
                               inv_scale);
    }
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

// the (d, H) shapes the tile kernels are compiled for (the same ones the sparse kernels' tile-sum hook has)
#define TGT_TILE_SHAPES(X) X(8, 8) X(16, 4) X(16, 8) X(8, 2)

template <typename T>
static int tile_fwd_launch(const tgt_tiles* tl, const void* q, const void* k, const void* v, float* acc, float* Zp,
                           void* final_out, void* out, float* Zout, const int32_t* rem_rowptr, bool zero_rows, int H, int d,
                           hipStream_t st) {
#define X(D_, H_) \
    if (d == D_ && H == H_) return tile_fwd_launch_s<T, D_, H_>(tl, q, k, v, acc, Zp, final_out, out, Zout, rem_rowptr, zero_rows, st);
    TGT_TILE_SHAPES(X)
#undef X
    set_error("block attention: no tile kernel for H=%d, d=%d", H, d);
    return TGT_ERR_UNSUPPORTED;
}

template <typename T>
static int tile_bwd_launch(const tgt_tiles* tl, const void* q, const void* k, const void* v, const void* dout,
                           const float2* nd, float* dq, float* dk, float* dv, void* f_dq, void* f_dk, void* f_dv,
                           void* o_dq, void* o_dk, void* o_dv, const int32_t* rem_dst, const int32_t* rem_src, bool zero_rows,
                           int H, int d, hipStream_t st) {
#define X(D_, H_)                                                                                                        \
    if (d == D_ && H == H_)                                                                                              \
        return tile_bwd_launch_s<T, D_, H_>(tl, q, k, v, dout, nd, dq, dk, dv, f_dq, f_dk, f_dv, o_dq, o_dk, o_dv, rem_dst, \
                                            rem_src, zero_rows, st);
    TGT_TILE_SHAPES(X)
#undef X
    set_error("block attention: no tile kernel for H=%d, d=%d", H, d);
    return TGT_ERR_UNSUPPORTED;
}

static int check_block(const tgt_tiles* tl, const tgt_plan* plan, int H, int d, int dtype, const void* ws,
                       int64_t ws_bytes) {
    if (!tl || !plan) { set_error("block attention: null tiles or plan"); return TGT_ERR_INVALID_ARG; }
    if (tl->N != plan->N) { set_error("block attention: tiles and plan disagree on N"); return TGT_ERR_INVALID_ARG; }
    if (d != 8 && d != 16) { set_error("block attention: head dim %d not in {8, 16}", d); return TGT_ERR_UNSUPPORTED; }
    if (dtype != TGT_DTYPE_F32 && dtype != TGT_DTYPE_BF16) { set_error("bad dtype %d", dtype); return TGT_ERR_INVALID_ARG; }
    if (H < 1) { set_error("H must be positive"); return TGT_ERR_INVALID_ARG; }
    const int64_t need = block_ws(tl, plan, H, d).total;
    if (!ws || ws_bytes < need || (reinterpret_cast<uintptr_t>(ws) & 255u)) {
        set_error("block attention workspace: need %lld bytes, 256-byte aligned; got %lld", (long long)need,
                  (long long)ws_bytes);
        return TGT_ERR_WORKSPACE;
    }
    return TGT_OK;
}

}  // namespace tgt

extern "C" {

int tgt_tiles_create(const int32_t* h_tiles, int64_t T, int block_size, int64_t N, void* stream,
                     tgt_tiles_t** out) {
    if (!out || T < 0 || N < 1 || (T > 0 && !h_tiles)) {
        tgt::set_error("tgt_tiles_create: bad argument");
        return TGT_ERR_INVALID_ARG;
    }
    if (block_size != tgt::kTile) {
        tgt::set_error("tgt_tiles_create: only 16 x 16 tiles (the reference's block size) have a kernel");
        return TGT_ERR_UNSUPPORTED;
    }
    std::vector<std::pair<int32_t, int32_t>> by_dst, by_src;
    for (int64_t t = 0; t < T; ++t) {
        const int32_t r0 = h_tiles[2 * t], c0 = h_tiles[2 * t + 1];
        if (r0 < 0 || c0 < 0 || (int64_t)r0 + tgt::kTile > N || (int64_t)c0 + tgt::kTile > N) {
            tgt::set_error("tgt_tiles_create: tile %lld = (%d, %d) leaves [0, %lld)", (long long)t, r0, c0, (long long)N);
            return TGT_ERR_INDEX_RANGE;
        }
        by_dst.emplace_back(c0, r0);
        by_src.emplace_back(r0, c0);
    }
    tgt_tiles* tl = new (std::nothrow) tgt_tiles();
    if (!tl) return TGT_ERR_INVALID_ARG;
    tl->N = N;
    tl->T = T;
    hipStream_t st = (hipStream_t)stream;
    std::vector<int32_t> kd, od, xd, ks, os, xs;
    std::vector<uint8_t> cd, cs;
    int rc = tgt::group_tiles(by_dst, N, "destination", kd, od, xd, cd);
    if (!rc) rc = tgt::group_tiles(by_src, N, "source", ks, os, xs, cs);
    if (!rc) rc = tgt::upload(tl->dst_c0, kd, st);
    if (!rc) rc = tgt::upload(tl->dst_off, od, st);
    if (!rc) rc = tgt::upload(tl->dst_r0, xd, st);
    if (!rc) rc = tgt::upload(tl->src_r0, ks, st);
    if (!rc) rc = tgt::upload(tl->src_off, os, st);
    if (!rc) rc = tgt::upload(tl->src_c0, xs, st);
    {
        std::vector<int4> rd(kd.size()), rs(ks.size());
        for (size_t g = 0; g < kd.size(); ++g) rd[g] = make_int4(kd[g], od[g], od[g + 1], xd[od[g]]);
        for (size_t g = 0; g < ks.size(); ++g) rs[g] = make_int4(ks[g], os[g], os[g + 1], xs[os[g]]);
        if (!rc && !rd.empty()) rc = tgt::upload(tl->dst_rec, rd, st);
        if (!rc && !rs.empty()) rc = tgt::upload(tl->src_rec, rs, st);
    }
    if (!rc) rc = tgt::upload(tl->cover_dst, cd, st);
    if (!rc) rc = tgt::upload(tl->cover_src, cs, st);
    std::vector<int32_t> bd, bs;
    if (!rc) {
        for (int64_t i = 0; i < N; ++i) {
            if (i >= (int64_t)cd.size() || !cd[i]) bd.push_back((int32_t)i);
            if (i >= (int64_t)cs.size() || !cs[i]) bs.push_back((int32_t)i);
        }
    }
    tl->n_bare_dst = (int64_t)bd.size();
    tl->n_bare_src = (int64_t)bs.size();
    if (!rc && !bd.empty()) rc = tgt::upload(tl->bare_dst, bd, st);
    if (!rc && !bs.empty()) rc = tgt::upload(tl->bare_src, bs, st);
    if (!rc && hipStreamSynchronize(st) != hipSuccess) rc = TGT_ERR_HIP;
    if (rc) { delete tl; return rc; }
    tl->n_dst_groups = (int32_t)kd.size();
    tl->n_src_groups = (int32_t)ks.size();
    *out = tl;
    return TGT_OK;
}

int tgt_tiles_destroy(tgt_tiles_t* tiles) {
    delete tiles;
    return TGT_OK;
}

int64_t tgt_block_attn_workspace_bytes(const tgt_tiles_t* tiles, const tgt_plan_t* plan, int H, int d) {
    if (!tiles || !plan || H < 1 || d < 1) return -1;
    return tgt::block_ws(tiles, plan, H, d).total;
}

int tgt_block_attn_fwd(const tgt_tiles_t* tiles, const tgt_plan_t* plan, const void* d_q, const void* d_k,
                       const void* d_v, const void* d_bias, int bias_mode, int H, int d, int dtype, void* d_out,
                       float* d_Z, void* d_workspace, int64_t workspace_bytes, void* stream) {
    int rc = tgt::check_block(tiles, plan, H, d, dtype, d_workspace, workspace_bytes);
    if (rc) return rc;
    if (!d_q || !d_k || !d_v || !d_out || !d_Z) { tgt::set_error("block attention: null q/k/v/out/Z"); return TGT_ERR_INVALID_ARG; }
    const tgt::BlockWs L = tgt::block_ws(tiles, plan, H, d);
    char* ws = static_cast<char*>(d_workspace);
    float* acc = reinterpret_cast<float*>(ws + L.acc);
    float* Zp = reinterpret_cast<float*>(ws + L.Z);
    hipStream_t st = (hipStream_t)stream;
    // no remaining edges: the tile kernels write out and Z themselves and nothing else runs
    const bool tiles_only = plan->E == 0;
    void* fin = tiles_only ? d_out : nullptr;
    float* Zdst = tiles_only ? d_Z : Zp;
    // with remaining edges: the tile kernels still finish the rows that have none (the sparse kernels skip them)
    const int32_t* rem = plan->dst.rowptr;
    // a plan that schedules only rows with edges leaves the rows without edges and without tiles to the tile launch
    const bool zr = plan->rows_with_edges_only;
    rc = dtype == TGT_DTYPE_F32 ? tgt::tile_fwd_launch<float>(tiles, d_q, d_k, d_v, acc, Zdst, fin, d_out, d_Z, rem, zr, H, d, st)
                                : tgt::tile_fwd_launch<tgt::tbf16>(tiles, d_q, d_k, d_v, acc, Zdst, fin, d_out, d_Z, rem, zr, H, d, st);
    if (rc || tiles_only) return rc;
    tgt::TileInit init{};
    init.acc = acc; init.Z = Zp; init.cover_dst = tiles->cover_dst.as<uint8_t>();
    return tgt::sparse_attn_fwd_impl(plan, d_q, d_k, d_v, d_bias, bias_mode, H, d, dtype, d_out, d_Z, ws + L.sparse,
                                     workspace_bytes - L.sparse, stream, &init);
}

int tgt_block_attn_bwd(const tgt_tiles_t* tiles, const tgt_plan_t* plan, const void* d_q, const void* d_k,
                       const void* d_v, const void* d_bias, int bias_mode, int H, int d, int dtype,
                       const void* d_out, const float* d_Z, const void* d_dout, void* d_dq, void* d_dk, void* d_dv,
                       void* d_dbias, void* d_workspace, int64_t workspace_bytes, void* stream) {
    int rc = tgt::check_block(tiles, plan, H, d, dtype, d_workspace, workspace_bytes);
    if (rc) return rc;
    if (!d_q || !d_k || !d_v || !d_out || !d_Z || !d_dout || !d_dq || !d_dk || !d_dv) {
        tgt::set_error("block attention backward: null pointer");
        return TGT_ERR_INVALID_ARG;
    }
    const tgt::BlockWs L = tgt::block_ws(tiles, plan, H, d);
    char* ws = static_cast<char*>(d_workspace);
    hipStream_t st = (hipStream_t)stream;
    rc = tgt::sparse_attn_node_side(plan, H, d, dtype, d_out, d_Z, d_dout, ws + L.sparse, stream);
    if (rc) return rc;
    const float2* nd = tgt::sparse_attn_nd_ptr(ws + L.sparse);
    float* dq = reinterpret_cast<float*>(ws + L.dq);
    float* dk = reinterpret_cast<float*>(ws + L.dk);
    float* dv = reinterpret_cast<float*>(ws + L.dv);
    const bool tiles_only = plan->E == 0;
    void* f_dq = tiles_only ? d_dq : nullptr;
    void* f_dk = tiles_only ? d_dk : nullptr;
    void* f_dv = tiles_only ? d_dv : nullptr;
    rc = dtype == TGT_DTYPE_F32
             ? tgt::tile_bwd_launch<float>(tiles, d_q, d_k, d_v, d_dout, nd, dq, dk, dv, f_dq, f_dk, f_dv, d_dq, d_dk, d_dv,
                                           plan->dst.rowptr, plan->src.rowptr, plan->rows_with_edges_only, H, d, st)
             : tgt::tile_bwd_launch<tgt::tbf16>(tiles, d_q, d_k, d_v, d_dout, nd, dq, dk, dv, f_dq, f_dk, f_dv, d_dq, d_dk,
                                                d_dv, plan->dst.rowptr, plan->src.rowptr, plan->rows_with_edges_only, H, d, st);
    if (rc || tiles_only) return rc;     // (no edges: there is no per-edge bias gradient to write either)
    tgt::TileInit init{};
    init.dq = dq; init.dk = dk; init.dv = dv;
    init.cover_dst = tiles->cover_dst.as<uint8_t>();
    init.cover_src = tiles->cover_src.as<uint8_t>();
    return tgt::sparse_attn_bwd_impl(plan, d_q, d_k, d_v, d_bias, bias_mode, H, d, dtype, d_out, d_Z, d_dout, d_dq,
                                     d_dk, d_dv, d_dbias, ws + L.sparse, workspace_bytes - L.sparse, stream, &init,
                                     true);
}

}  // extern "C"
