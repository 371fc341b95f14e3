// Edge construction and ordering on the GPU: the integer side of the reference's
// batch preparation.
//
//   tgt_fix_edge_index      gt_sp/utils.py:34-50   (global node 0, edges to and from it)
//   tgt_sub_edge_index      gt_sp/utils.py:202-215 (edges among the nodes of a batch, renamed)
//   tgt_reformat_*          gt_sp/utils.py:319-359 (relabel by partition, cluster
//                           "blockize" of gt_sp/utils.py:223-305, stable sort by source)
//
// The reference does this with Python lists and per-edge appends (minutes at
// 18 M edges).  Here the per-edge work runs in kernels; the only host work is
// the k x k table of partition pairs and the block coordinates, which the
// reference draws from numpy's legacy MT19937 stream (np.random.seed(n) then
// np.random.randint) - restated below so the blocks are the same ones.
#include "common.h"
#include <vector>
#include <new>

namespace tgt {

// ---------------------------------------------------------------------------
// numpy legacy RandomState: MT19937 seeded with init_genrand, randint(0, high)
// by masked rejection on 32-bit outputs.
// ---------------------------------------------------------------------------
class LegacyMT {
public:
    explicit LegacyMT(uint32_t seed) {
        mt_[0] = seed;
        for (int i = 1; i < 624; ++i) mt_[i] = 1812433253u * (mt_[i - 1] ^ (mt_[i - 1] >> 30)) + (uint32_t)i;
        pos_ = 624;
    }
    uint32_t next() {
        if (pos_ == 624) refill();
        uint32_t y = mt_[pos_++];
        y ^= y >> 11;
        y ^= (y << 7) & 0x9d2c5680u;
        y ^= (y << 15) & 0xefc60000u;
        y ^= y >> 18;
        return y;
    }
    // randint(0, high), high >= 1 and high - 1 < 2^32 - 1
    int64_t randint(int64_t high) {
        const uint64_t rng = (uint64_t)(high - 1);
        if (rng == 0) return 0;                       // no draw is consumed
        uint64_t mask = rng;
        mask |= mask >> 1; mask |= mask >> 2; mask |= mask >> 4; mask |= mask >> 8; mask |= mask >> 16;
        uint32_t v;
        do { v = next() & (uint32_t)mask; } while (v > rng);
        return (int64_t)v;
    }
private:
    void refill() {
        const uint32_t UP = 0x80000000u, LO = 0x7fffffffu, MAG = 0x9908b0dfu;
        int i = 0;
        for (; i < 624 - 397; ++i) {
            uint32_t y = (mt_[i] & UP) | (mt_[i + 1] & LO);
            mt_[i] = mt_[i + 397] ^ (y >> 1) ^ ((y & 1u) ? MAG : 0u);
        }
        for (; i < 623; ++i) {
            uint32_t y = (mt_[i] & UP) | (mt_[i + 1] & LO);
            mt_[i] = mt_[i + (397 - 624)] ^ (y >> 1) ^ ((y & 1u) ? MAG : 0u);
        }
        uint32_t y = (mt_[623] & UP) | (mt_[0] & LO);
        mt_[623] = mt_[396] ^ (y >> 1) ^ ((y & 1u) ? MAG : 0u);
        pos_ = 0;
    }
    uint32_t mt_[624];
    int pos_;
};

// ---------------------------------------------------------------------------
// kernels
// ---------------------------------------------------------------------------
__global__ void k_fix_edge_index(const int64_t* __restrict__ in, int64_t E0, int64_t n,
                                 int64_t* __restrict__ out) {
    const int64_t Eo = E0 + 2 * n;
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= Eo) return;
    int64_t s, d;
    if (i < E0) { s = in[i] + 1; d = in[E0 + i] + 1; }
    else if (i < E0 + n) { s = i - E0 + 1; d = 0; }     // real node -> global node
    else { s = 0; d = i - E0 - n + 1; }                  // global node -> real node
    out[i] = s;
    out[Eo + i] = d;
}

__global__ void k_check_partition(const int64_t* __restrict__ part, int64_t N, int k, uint32_t* __restrict__ p32,
                                  int* __restrict__ flag) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= N) return;
    int64_t p = part[i];
    if (p < 0 || p >= k) { flag[0] = 1; p = 0; }
    p32[i] = (uint32_t)p;
}

__global__ void k_check_edges(const int64_t* __restrict__ src, const int64_t* __restrict__ dst, int64_t E,
                              int64_t N, int* __restrict__ flag) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= E) return;
    const int64_t s = src[i], d = dst[i];
    if ((s < 0) | (s >= N) | (d < 0) | (d >= N)) flag[0] = 1;
}

// mapping[old] = new position; sorted[new] = old (as int64 for the caller)
__global__ void k_invert(const uint32_t* __restrict__ sorted_old, int64_t N, uint32_t* __restrict__ mapping,
                         int64_t* __restrict__ sorted_out) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= N) return;
    const uint32_t o = sorted_old[i];
    mapping[o] = (uint32_t)i;
    sorted_out[i] = (int64_t)o;
}

// Histogram of keys in [0, nbins).  The bins are few (k or k*k partition pairs) and neighbouring
// keys are often equal, so equal keys of a wave are first merged with ballots (one LDS add per
// distinct key and wave), workgroups count in LDS, and only non-empty bins reach global memory.
// Integer counts: the order of the additions does not matter.
constexpr int kCountLdsBins = 4096;
__global__ __launch_bounds__(256) void k_count(const uint32_t* __restrict__ keys, int64_t n, int nbins, int key_bits,
                                               unsigned long long* __restrict__ cnt) {
    __shared__ uint32_t h[kCountLdsBins];
    const bool lds = nbins <= kCountLdsBins;
    if (lds) {
        for (int b = threadIdx.x; b < nbins; b += blockDim.x) h[b] = 0;
        __syncthreads();
    }
    const int lane = threadIdx.x & 63;
    const uint64_t lower = lane == 0 ? 0ull : (~0ull >> (64 - lane));
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    const int64_t rounds = (n + stride - 1) / stride;          // the same for every thread: ballots need whole waves
    for (int64_t t = 0; t < rounds; ++t) {
        const int64_t i = t * stride + (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
        const bool valid = i < n;
        const uint32_t key = valid ? keys[i] : 0u;
        uint64_t same = __ballot(valid);
        for (int b = 0; b < key_bits; ++b) {
            const bool bit = (key >> b) & 1u;
            const uint64_t bal = __ballot(bit);
            same &= bit ? bal : ~bal;
        }
        if (valid && (same & lower) == 0) {                    // lowest lane of its group of equal keys
            const uint32_t c = (uint32_t)__popcll(same);
            if (lds) atomicAdd(&h[key], c);
            else atomicAdd(&cnt[key], (unsigned long long)c);
        }
    }
    if (lds) {
        __syncthreads();
        for (int b = threadIdx.x; b < nbins; b += blockDim.x)
            if (h[b]) atomicAdd(&cnt[b], (unsigned long long)h[b]);
    }
}

// per-edge keys: pair = part[src]*k + part[dst], s32 = src, d32 = dst
__global__ void k_edge_keys(const int64_t* __restrict__ src, const int64_t* __restrict__ dst, int64_t E,
                            const uint32_t* __restrict__ p32, int k, uint32_t* __restrict__ pair,
                            uint32_t* __restrict__ s32, uint32_t* __restrict__ d32) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= E) return;
    const uint32_t s = (uint32_t)src[i], d = (uint32_t)dst[i];
    s32[i] = s;
    d32[i] = d;
    pair[i] = p32[s] * (uint32_t)k + p32[d];
}

// out[i] = table[idx[i]]
__global__ void k_gather_u32(const uint32_t* __restrict__ table, const uint32_t* __restrict__ idx, int64_t n,
                             uint32_t* __restrict__ out) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = table[idx[i]];
}

// relabelled endpoints of the edges order[lo + t], t < cnt, written at out_off + t
__global__ void k_emit_raw(const uint32_t* __restrict__ order, int64_t lo, int64_t cnt,
                           const uint32_t* __restrict__ s32, const uint32_t* __restrict__ d32,
                           const uint32_t* __restrict__ mapping, int64_t out_off, uint32_t* __restrict__ ns,
                           uint32_t* __restrict__ nd) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= cnt) return;
    const uint32_t e = order ? order[lo + t] : (uint32_t)(lo + t);
    ns[out_off + t] = mapping[s32[e]];
    nd[out_off + t] = mapping[d32[e]];
}

// dense bs x bs block, pairs (a, b) row-major (gt_sp/utils.py:218-220); one workgroup per block
__global__ void k_emit_blocks(const int64_t* __restrict__ blk_off, const uint32_t* __restrict__ blk_r0,
                              const uint32_t* __restrict__ blk_c0, int bs, uint32_t* __restrict__ ns,
                              uint32_t* __restrict__ nd) {
    const int64_t off = blk_off[blockIdx.x];
    const uint32_t r0 = blk_r0[blockIdx.x], c0 = blk_c0[blockIdx.x];
    for (int p = threadIdx.x; p < bs * bs; p += blockDim.x) {
        ns[off + p] = r0 + (uint32_t)(p / bs);
        nd[off + p] = c0 + (uint32_t)(p % bs);
    }
}

__global__ void k_write_raw(const uint32_t* __restrict__ ns, const uint32_t* __restrict__ nd, int64_t off,
                            int64_t cnt, int64_t dst_off, int64_t E_raw, int64_t* __restrict__ out) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= cnt) return;
    out[dst_off + i] = (int64_t)ns[off + i];
    out[E_raw + dst_off + i] = (int64_t)nd[off + i];
}

__global__ void k_write_sorted(const uint32_t* __restrict__ keys_sorted, const uint32_t* __restrict__ order,
                               const uint32_t* __restrict__ nd, int64_t n, int64_t* __restrict__ out) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    out[i] = (int64_t)keys_sorted[i];
    out[n + i] = (int64_t)nd[order[i]];
}

static inline unsigned nblk(int64_t n, int t = 256) { return (unsigned)((n + t - 1) / t); }

}  // namespace tgt

struct tgt_reformat {
    int64_t N = 0, E_out = 0;
    tgt::DevBuf edge_index;       // int64 [2, E_out], stably sorted by source
    tgt::DevBuf sorted_indices;   // int64 [N], new id -> old id
    std::vector<int32_t> tiles;   // (first source, first destination) of every emitted block, emission order
    int64_t E_raw = 0;            // edges kept as they are (the sparsity > p branch, or everything if !blockize)
    tgt::DevBuf raw;              // int64 [2, E_raw], relabelled, emission order
};

namespace tgt {

static int reformat_impl(const int64_t* d_src, const int64_t* d_dst, int64_t E, int64_t N,
                         const int64_t* d_part, int k, int bs, int blockize, hipStream_t st, tgt_reformat* R) {
    R->N = N;
    DevBuf flag, p32, mapping, sorted_old;
    TGT_HIP_CHECK(flag.alloc(sizeof(int)));
    TGT_HIP_CHECK(p32.alloc(sizeof(uint32_t) * N));
    TGT_HIP_CHECK(mapping.alloc(sizeof(uint32_t) * N));
    TGT_HIP_CHECK(R->sorted_indices.alloc(sizeof(int64_t) * N));
    TGT_HIP_CHECK(hipMemsetAsync(flag.p, 0, sizeof(int), st));
    hipLaunchKernelGGL(k_check_partition, dim3(nblk(N)), dim3(256), 0, st, d_part, N, k, p32.as<uint32_t>(),
                       flag.as<int>());
    if (E > 0)
        hipLaunchKernelGGL(k_check_edges, dim3(nblk(E)), dim3(256), 0, st, d_src, d_dst, E, N, flag.as<int>());
    int h_flag = 0;
    TGT_HIP_CHECK(hipMemcpyAsync(&h_flag, flag.p, sizeof(int), hipMemcpyDeviceToHost, st));
    TGT_HIP_CHECK(hipStreamSynchronize(st));
    if (h_flag) {
        set_error("partition id outside [0, %d) or edge endpoint outside [0, %lld)", k, (long long)N);
        return TGT_ERR_INDEX_RANGE;
    }
    // relabel: parts in order, members in ascending old id (gt_sp/utils.py:329-335) = stable sort by part
    RadixSorter node_sorter;
    int rc = node_sorter.init(N);
    if (rc) return rc;
    const uint32_t *ks = nullptr, *vs = nullptr;
    rc = node_sorter.sort(p32.as<uint32_t>(), nullptr, N, bits_for(k), st, &ks, &vs);
    if (rc) return rc;
    hipLaunchKernelGGL(k_invert, dim3(nblk(N)), dim3(256), 0, st, vs, N, mapping.as<uint32_t>(),
                       R->sorted_indices.as<int64_t>());
    // node count per part
    DevBuf cnt_nodes, cnt_pairs;
    TGT_HIP_CHECK(cnt_nodes.alloc(sizeof(unsigned long long) * k));
    TGT_HIP_CHECK(cnt_pairs.alloc(sizeof(unsigned long long) * k * k));
    TGT_HIP_CHECK(hipMemsetAsync(cnt_nodes.p, 0, sizeof(unsigned long long) * k, st));
    TGT_HIP_CHECK(hipMemsetAsync(cnt_pairs.p, 0, sizeof(unsigned long long) * k * k, st));
    const auto count_grid = [](int64_t n) { return dim3((unsigned)std::min<int64_t>(256, (n + 255) / 256)); };
    hipLaunchKernelGGL(k_count, count_grid(N), dim3(256), 0, st, p32.as<uint32_t>(), N, k, bits_for(k),
                       cnt_nodes.as<unsigned long long>());
    DevBuf pair, s32, d32;
    const size_t eb = sizeof(uint32_t) * (size_t)(E ? E : 1);
    TGT_HIP_CHECK(pair.alloc(eb));
    TGT_HIP_CHECK(s32.alloc(eb));
    TGT_HIP_CHECK(d32.alloc(eb));
    if (E > 0) {
        hipLaunchKernelGGL(k_edge_keys, dim3(nblk(E)), dim3(256), 0, st, d_src, d_dst, E, p32.as<uint32_t>(), k,
                           pair.as<uint32_t>(), s32.as<uint32_t>(), d32.as<uint32_t>());
        hipLaunchKernelGGL(k_count, count_grid(E), dim3(256), 0, st, pair.as<uint32_t>(), E, k * k,
                           bits_for((int64_t)k * k), cnt_pairs.as<unsigned long long>());
    }
    std::vector<unsigned long long> h_nodes(k), h_pairs((size_t)k * k);
    TGT_HIP_CHECK(hipMemcpyAsync(h_nodes.data(), cnt_nodes.p, sizeof(unsigned long long) * k,
                                 hipMemcpyDeviceToHost, st));
    TGT_HIP_CHECK(hipMemcpyAsync(h_pairs.data(), cnt_pairs.p, sizeof(unsigned long long) * k * k,
                                 hipMemcpyDeviceToHost, st));
    TGT_HIP_CHECK(hipStreamSynchronize(st));

    // ---- what to emit, in the reference's order ------------------------------
    struct RawSlice { int64_t lo, cnt, out_off; };
    std::vector<RawSlice> raws;
    std::vector<int64_t> blk_off;
    std::vector<uint32_t> blk_r0, blk_c0;
    int64_t E_out = 0;
    if (!blockize) {
        E_out = E;
    } else {
        // run lengths of equal (part_src, part_dst) in sorted order, stored COMPACTLY in the order
        // of the non-empty pairs and read back as [i*k+j] (gt_sp/utils.py:237-246,270)
        std::vector<int64_t> counts((size_t)k * k, 0), cum((size_t)k * k + 1, 0), offs(k, 0);
        size_t w = 0;
        for (size_t pq = 0; pq < (size_t)k * k; ++pq)
            if (h_pairs[pq]) counts[w++] = (int64_t)h_pairs[pq];
        for (size_t pq = 0; pq < (size_t)k * k; ++pq) cum[pq + 1] = cum[pq] + counts[pq];
        for (int i = 1; i < k; ++i) offs[i] = offs[i - 1] + (int64_t)h_nodes[i - 1];
        int64_t keep_cnt = 0;
        const double per_block = (double)bs * (double)bs;
        for (int i = 0; i < k; ++i) {
            for (int j = 0; j < k; ++j) {
                const int64_t ni = (int64_t)h_nodes[i], nj = (int64_t)h_nodes[j];
                const int64_t total = ni * nj;
                if (total == 0) {
                    set_error("partition %d or %d is empty (the reference divides by zero here)", i, j);
                    return TGT_ERR_INVALID_ARG;
                }
                const int64_t c = counts[(size_t)i * k + j];
                const double sparsity = (double)c / (double)total;
                if (sparsity > 1.0) {                       // p is hard-wired to 1 (gt_sp/utils.py:344)
                    raws.push_back(RawSlice{cum[(size_t)i * k + j], c, E_out});
                    E_out += c;
                } else {
                    const int nb = (int)(sparsity * (double)total / per_block) + 1;
                    LegacyMT rng((uint32_t)keep_cnt);        // np.random.seed(keep_cnt)
                    if (ni >= bs && nj >= bs) {
                        for (int b = 0; b < nb; ++b) {
                            const int64_t br = rng.randint(ni / bs);
                            const int64_t bc = rng.randint(nj / bs);
                            ++keep_cnt;
                            blk_off.push_back(E_out);
                            blk_r0.push_back((uint32_t)(br * bs + offs[i]));
                            blk_c0.push_back((uint32_t)(bc * bs + offs[j]));
                            E_out += (int64_t)bs * bs;
                        }
                    }
                }
            }
        }
    }
    if (E_out > 0x7fff0000LL) { set_error("reordered edge list does not fit 31 bits"); return TGT_ERR_INVALID_ARG; }
    R->E_out = E_out;
    TGT_HIP_CHECK(R->edge_index.alloc(sizeof(int64_t) * 2 * (size_t)(E_out ? E_out : 1)));
    DevBuf ns, nd;
    TGT_HIP_CHECK(ns.alloc(sizeof(uint32_t) * (size_t)(E_out ? E_out : 1)));
    TGT_HIP_CHECK(nd.alloc(sizeof(uint32_t) * (size_t)(E_out ? E_out : 1)));
    RadixSorter sorter;
    rc = sorter.init(E_out > E ? E_out : E);
    if (rc) return rc;

    if (!blockize) {
        if (E > 0)
            hipLaunchKernelGGL(k_emit_raw, dim3(nblk(E)), dim3(256), 0, st, (const uint32_t*)nullptr, (int64_t)0, E,
                               s32.as<uint32_t>(), d32.as<uint32_t>(), mapping.as<uint32_t>(), (int64_t)0,
                               ns.as<uint32_t>(), nd.as<uint32_t>());
    } else {
        if (!raws.empty()) {
            // edges sorted by ((part_src, part_dst), (src, dst)) (gt_sp/utils.py:230-235): LSD over
            // dst, src, pair with the stable sort
            DevBuf tmp, order;
            TGT_HIP_CHECK(tmp.alloc(eb));
            TGT_HIP_CHECK(order.alloc(eb));
            const uint32_t *ko = nullptr, *vo = nullptr;
            rc = sorter.sort(d32.as<uint32_t>(), nullptr, E, bits_for(N), st, &ko, &vo);
            if (rc) return rc;
            hipLaunchKernelGGL(k_gather_u32, dim3(nblk(E)), dim3(256), 0, st, s32.as<uint32_t>(), vo, E,
                               tmp.as<uint32_t>());
            TGT_HIP_CHECK(hipMemcpyAsync(order.p, vo, eb, hipMemcpyDeviceToDevice, st));
            rc = sorter.sort(tmp.as<uint32_t>(), order.as<uint32_t>(), E, bits_for(N), st, &ko, &vo);
            if (rc) return rc;
            hipLaunchKernelGGL(k_gather_u32, dim3(nblk(E)), dim3(256), 0, st, pair.as<uint32_t>(), vo, E,
                               tmp.as<uint32_t>());
            TGT_HIP_CHECK(hipMemcpyAsync(order.p, vo, eb, hipMemcpyDeviceToDevice, st));
            rc = sorter.sort(tmp.as<uint32_t>(), order.as<uint32_t>(), E, bits_for((int64_t)k * k), st, &ko, &vo);
            if (rc) return rc;
            for (const RawSlice& r : raws)
                if (r.cnt > 0)
                    hipLaunchKernelGGL(k_emit_raw, dim3(nblk(r.cnt)), dim3(256), 0, st, vo, r.lo, r.cnt,
                                       s32.as<uint32_t>(), d32.as<uint32_t>(), mapping.as<uint32_t>(), r.out_off,
                                       ns.as<uint32_t>(), nd.as<uint32_t>());
            TGT_HIP_CHECK(hipStreamSynchronize(st));   // tmp / order die here
        }
        if (!blk_off.empty()) {
            DevBuf d_off, d_r0, d_c0;
            const size_t nb = blk_off.size();
            TGT_HIP_CHECK(d_off.alloc(sizeof(int64_t) * nb));
            TGT_HIP_CHECK(d_r0.alloc(sizeof(uint32_t) * nb));
            TGT_HIP_CHECK(d_c0.alloc(sizeof(uint32_t) * nb));
            TGT_HIP_CHECK(hipMemcpyAsync(d_off.p, blk_off.data(), sizeof(int64_t) * nb, hipMemcpyHostToDevice, st));
            TGT_HIP_CHECK(hipMemcpyAsync(d_r0.p, blk_r0.data(), sizeof(uint32_t) * nb, hipMemcpyHostToDevice, st));
            TGT_HIP_CHECK(hipMemcpyAsync(d_c0.p, blk_c0.data(), sizeof(uint32_t) * nb, hipMemcpyHostToDevice, st));
            hipLaunchKernelGGL(k_emit_blocks, dim3((unsigned)nb), dim3(256), 0, st, d_off.as<int64_t>(),
                               d_r0.as<uint32_t>(), d_c0.as<uint32_t>(), bs, ns.as<uint32_t>(), nd.as<uint32_t>());
            TGT_HIP_CHECK(hipStreamSynchronize(st));   // the descriptor buffers die here
        }
    }
    // the blocks as a tile list and the edges kept as they are, for the block attention path
    for (size_t i = 0; i < blk_r0.size(); ++i) {
        R->tiles.push_back((int32_t)blk_r0[i]);
        R->tiles.push_back((int32_t)blk_c0[i]);
    }
    {
        int64_t e_raw = blockize ? 0 : E;
        for (const RawSlice& r : raws) e_raw += r.cnt;
        R->E_raw = e_raw;
        TGT_HIP_CHECK(R->raw.alloc(sizeof(int64_t) * 2 * (size_t)(e_raw ? e_raw : 1)));
        if (!blockize) {
            if (E > 0)
                hipLaunchKernelGGL(k_write_raw, dim3(nblk(E)), dim3(256), 0, st, ns.as<uint32_t>(), nd.as<uint32_t>(),
                                   (int64_t)0, E, (int64_t)0, e_raw, R->raw.as<int64_t>());
        } else {
            int64_t pos = 0;
            for (const RawSlice& r : raws) {
                if (r.cnt > 0)
                    hipLaunchKernelGGL(k_write_raw, dim3(nblk(r.cnt)), dim3(256), 0, st, ns.as<uint32_t>(),
                                       nd.as<uint32_t>(), r.out_off, r.cnt, pos, e_raw, R->raw.as<int64_t>());
                pos += r.cnt;
            }
        }
    }
    // stable sort by new source (gt_sp/utils.py:354-356)
    if (E_out > 0) {
        const uint32_t *ko = nullptr, *vo = nullptr;
        rc = sorter.sort(ns.as<uint32_t>(), nullptr, E_out, bits_for(N), st, &ko, &vo);
        if (rc) return rc;
        hipLaunchKernelGGL(k_write_sorted, dim3(nblk(E_out)), dim3(256), 0, st, ko, vo, nd.as<uint32_t>(), E_out,
                           R->edge_index.as<int64_t>());
    }
    TGT_HIP_CHECK(hipGetLastError());
    TGT_HIP_CHECK(hipStreamSynchronize(st));
    return TGT_OK;
}

// ---------------------------------------------------------------------------
// Sub-graph of a node batch (gen_sub_edge_index, gt_sp/utils.py:202-215): the
// sequence of torch_geometric 2.0.0 calls
//   remove_self_loops(edge_index)              keep edges with src != dst, in order
//   add_self_loops(.., num_nodes=N)            append (i, i) for i = 0..N-1
//   subgraph(idx_batch, .., relabel_nodes=True, num_nodes=N)
//                                              keep edges with both ends in the batch, in
//                                              order, and rename node idx_batch[p] to p
// as one order-preserving compaction over the E edges followed by the N
// self-loops.  A node that occurs more than once in idx_batch takes its LAST
// position (what the sequential index assignment n_idx[subset] = arange gives).
// ---------------------------------------------------------------------------
constexpr int kSubItems = 1024;     // items per workgroup of the compaction (4 rounds of 256)

__global__ void k_sub_fill(int32_t* __restrict__ pos, int64_t N) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < N) pos[i] = -1;
}

__global__ void k_sub_positions(const int64_t* __restrict__ idx, int64_t S, int64_t N, int32_t* __restrict__ pos,
                                int* __restrict__ bad) {
    const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= S) return;
    const int64_t v = idx[p];
    if (v < 0 || v >= N) { atomicOr(bad, 1); return; }
    atomicMax(&pos[v], (int32_t)p);
}

// item i < E: edge i; item E + v: self-loop of node v.  Returns the renamed endpoints.
__device__ __forceinline__ bool sub_item(const int64_t* __restrict__ ei, int64_t E, int64_t N,
                                         const int32_t* __restrict__ pos, int64_t i, int32_t& a, int32_t& b,
                                         int* __restrict__ bad) {
    if (i < E) {
        const int64_t s = ei[i], d = ei[E + i];
        if (s < 0 || s >= N || d < 0 || d >= N) { atomicOr(bad, 2); return false; }
        if (s == d) return false;
        a = pos[s]; b = pos[d];
        return a >= 0 && b >= 0;
    }
    a = b = pos[i - E];
    return a >= 0;
}

// pass 0 counts the kept items of every workgroup; pass 1 writes them behind the
// workgroup's offset, in item order (ballot ranks inside a wave, wave totals in LDS).
template <int PASS>
__global__ __launch_bounds__(256) void k_sub_compact(const int64_t* __restrict__ ei, int64_t E, int64_t N,
                                                     const int32_t* __restrict__ pos, uint32_t* __restrict__ counts,
                                                     uint64_t* __restrict__ keep_bits, int64_t* __restrict__ out,
                                                     int64_t capacity, int* __restrict__ bad) {
    __shared__ uint32_t wave_n[4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t total = E + N;
    uint32_t run = PASS ? counts[blockIdx.x] : 0u;          // pass 1: exclusive prefix of this workgroup
    for (int round = 0; round < kSubItems / 256; ++round) {
        const int64_t i = (int64_t)blockIdx.x * kSubItems + round * 256 + threadIdx.x;
        int32_t a = 0, b = 0;
        // one keep bit per item, a 64-bit word per wave and round: the writing pass reads the words and
        // looks at the endpoints of the kept items only (a few per cent of the edge list)
        const int64_t word = ((int64_t)blockIdx.x * (kSubItems / 256) + round) * 4 + wave;
        bool keep;
        uint64_t m;
        if (PASS == 0) {
            keep = i < total && sub_item(ei, E, N, pos, i, a, b, bad);
            m = __ballot(keep);
            if (lane == 0) keep_bits[word] = m;
        } else {
            m = keep_bits[word];
            keep = (m >> lane) & 1ull;
            if (keep) (void)sub_item(ei, E, N, pos, i, a, b, bad);
        }
        if (lane == 0) wave_n[wave] = (uint32_t)__popcll(m);
        __syncthreads();
        uint32_t before = 0, all = 0;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            if (w < wave) before += wave_n[w];
            all += wave_n[w];
        }
        if (PASS && keep) {
            const int64_t o = (int64_t)run + before + __popcll(m & ((1ull << lane) - 1ull));
            out[o] = a;
            out[capacity + o] = b;
        }
        run += all;
        __syncthreads();
    }
    if (!PASS && threadIdx.x == 0) counts[blockIdx.x] = run;
}

// exclusive prefix of the workgroup counts in place (one workgroup), total to counts[n]
__global__ __launch_bounds__(256) void k_sub_scan(uint32_t* __restrict__ counts, int n) {
    __shared__ uint32_t part[256];
    const int tid = threadIdx.x;
    const int chunk = (n + 255) / 256;
    const int b = min(tid * chunk, n), e = min(b + chunk, n);
    uint32_t sum = 0;
    for (int i = b; i < e; ++i) sum += counts[i];
    part[tid] = sum;
    __syncthreads();
    for (int off = 1; off < 256; off <<= 1) {
        const uint32_t x = tid >= off ? part[tid - off] : 0u;
        __syncthreads();
        part[tid] += x;
        __syncthreads();
    }
    uint32_t run = tid ? part[tid - 1] : 0u;
    for (int i = b; i < e; ++i) {
        const uint32_t x = counts[i];
        counts[i] = run;
        run += x;
    }
    if (tid == 255) counts[n] = part[255];
}

static int sub_edge_index_impl(const int64_t* d_ei, int64_t E, int64_t N, const int64_t* d_idx, int64_t S,
                               int64_t* d_out, int64_t capacity, int64_t* h_num, hipStream_t st) {
    const int64_t total = E + N;
    const int nblocks = (int)((total + kSubItems - 1) / kSubItems);
    DevBuf pos, counts, bad, bits;
    TGT_HIP_CHECK(pos.alloc(sizeof(int32_t) * (size_t)N));
    TGT_HIP_CHECK(counts.alloc(sizeof(uint32_t) * (size_t)(nblocks + 1)));
    TGT_HIP_CHECK(bits.alloc(sizeof(uint64_t) * (size_t)nblocks * (kSubItems / 64)));
    TGT_HIP_CHECK(bad.alloc(sizeof(int)));
    TGT_HIP_CHECK(hipMemsetAsync(bad.p, 0, sizeof(int), st));
    hipLaunchKernelGGL(k_sub_fill, dim3(nblk(N)), dim3(256), 0, st, pos.as<int32_t>(), N);
    if (S > 0)
        hipLaunchKernelGGL(k_sub_positions, dim3(nblk(S)), dim3(256), 0, st, d_idx, S, N, pos.as<int32_t>(),
                           bad.as<int>());
    hipLaunchKernelGGL((k_sub_compact<0>), dim3(nblocks), dim3(256), 0, st, d_ei, E, N, pos.as<int32_t>(),
                       counts.as<uint32_t>(), bits.as<uint64_t>(), (int64_t*)nullptr, (int64_t)0, bad.as<int>());
    hipLaunchKernelGGL(k_sub_scan, dim3(1), dim3(256), 0, st, counts.as<uint32_t>(), nblocks);
    TGT_HIP_CHECK(hipGetLastError());
    uint32_t n_keep = 0;
    int h_bad = 0;
    TGT_HIP_CHECK(hipMemcpyAsync(&n_keep, counts.as<uint32_t>() + nblocks, sizeof(uint32_t), hipMemcpyDeviceToHost, st));
    TGT_HIP_CHECK(hipMemcpyAsync(&h_bad, bad.p, sizeof(int), hipMemcpyDeviceToHost, st));
    TGT_HIP_CHECK(hipStreamSynchronize(st));
    if (h_bad) {
        set_error("tgt_sub_edge_index: %s outside [0, %lld)", (h_bad & 1) ? "a batch node id is" : "an edge endpoint is",
                  (long long)N);
        return TGT_ERR_INDEX_RANGE;
    }
    *h_num = (int64_t)n_keep;
    if ((int64_t)n_keep > capacity) {
        set_error("tgt_sub_edge_index: %lld edges kept, room for %lld", (long long)n_keep, (long long)capacity);
        return TGT_ERR_WORKSPACE;
    }
    if (n_keep > 0) {
        hipLaunchKernelGGL((k_sub_compact<1>), dim3(nblocks), dim3(256), 0, st, d_ei, E, N, pos.as<int32_t>(),
                           counts.as<uint32_t>(), bits.as<uint64_t>(), d_out, capacity, bad.as<int>());
        TGT_HIP_CHECK(hipGetLastError());
        TGT_HIP_CHECK(hipStreamSynchronize(st));      // the scratch buffers are freed on return
    }
    return TGT_OK;
}

}  // namespace tgt

extern "C" {

int tgt_fix_edge_index(const int64_t* d_edge_index, int64_t E0, int64_t num_node, int64_t* d_out, void* stream) {
    if (E0 < 0 || num_node < 0 || !d_out || (E0 > 0 && !d_edge_index)) {
        tgt::set_error("tgt_fix_edge_index: null pointer or negative size");
        return TGT_ERR_INVALID_ARG;
    }
    const int64_t Eo = E0 + 2 * num_node;
    if (Eo == 0) return TGT_OK;
    hipLaunchKernelGGL(tgt::k_fix_edge_index, dim3(tgt::nblk(Eo)), dim3(256), 0, (hipStream_t)stream, d_edge_index,
                       E0, num_node, d_out);
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

int tgt_sub_edge_index(const int64_t* d_edge_index, int64_t E, int64_t N, const int64_t* d_idx_batch, int64_t S,
                       int64_t* d_out, int64_t capacity, int64_t* h_num_edges, void* stream) {
    if (E < 0 || N < 1 || S < 0 || capacity < 0 || !h_num_edges || (E > 0 && !d_edge_index) || (S > 0 && !d_idx_batch) ||
        (capacity > 0 && !d_out)) {
        tgt::set_error("tgt_sub_edge_index: null pointer or bad size");
        return TGT_ERR_INVALID_ARG;
    }
    if (E > 0x7fff0000LL || N > 0x7fff0000LL || S > 0x7fff0000LL) {
        tgt::set_error("tgt_sub_edge_index: E, N and the batch size must fit 31 bits");
        return TGT_ERR_INVALID_ARG;
    }
    return tgt::sub_edge_index_impl(d_edge_index, E, N, d_idx_batch, S, d_out, capacity, h_num_edges,
                                    (hipStream_t)stream);
}

int tgt_np_legacy_randint(uint32_t seed, const int64_t* h_highs, int n, int64_t* h_out) {
    if (n < 0 || (n > 0 && (!h_highs || !h_out))) return TGT_ERR_INVALID_ARG;
    tgt::LegacyMT rng(seed);
    for (int i = 0; i < n; ++i) {
        if (h_highs[i] < 1 || h_highs[i] > 0xffffffffLL) return TGT_ERR_INVALID_ARG;
        h_out[i] = rng.randint(h_highs[i]);
    }
    return TGT_OK;
}

int tgt_reformat_create(const int64_t* d_src, const int64_t* d_dst, int64_t E, int64_t N,
                        const int64_t* d_partition_ids, int k, int block_size, int blockize, void* stream,
                        tgt_reformat_t** out) {
    if (!out || E < 0 || N < 1 || k < 1 || k > 4096 || block_size < 1 || !d_partition_ids ||
        (E > 0 && (!d_src || !d_dst))) {
        tgt::set_error("tgt_reformat_create: bad argument");
        return TGT_ERR_INVALID_ARG;
    }
    if (E > 0x7fff0000LL || N > 0x7fff0000LL) {
        tgt::set_error("tgt_reformat_create: E and N must fit 31 bits");
        return TGT_ERR_INVALID_ARG;
    }
    tgt_reformat* R = new (std::nothrow) tgt_reformat();
    if (!R) return TGT_ERR_INVALID_ARG;
    const int rc = tgt::reformat_impl(d_src, d_dst, E, N, d_partition_ids, k, block_size, blockize,
                                      (hipStream_t)stream, R);
    if (rc != TGT_OK) { delete R; return rc; }
    *out = R;
    return TGT_OK;
}

int64_t tgt_reformat_num_edges(const tgt_reformat_t* r) { return r ? r->E_out : -1; }

int tgt_reformat_export(const tgt_reformat_t* r, int64_t* d_edge_index, int64_t* d_sorted_indices, void* stream) {
    if (!r || !d_sorted_indices || (r->E_out > 0 && !d_edge_index)) {
        tgt::set_error("tgt_reformat_export: null pointer");
        return TGT_ERR_INVALID_ARG;
    }
    hipStream_t st = (hipStream_t)stream;
    if (r->E_out > 0)
        TGT_HIP_CHECK(hipMemcpyAsync(d_edge_index, r->edge_index.p, sizeof(int64_t) * 2 * r->E_out,
                                     hipMemcpyDeviceToDevice, st));
    TGT_HIP_CHECK(hipMemcpyAsync(d_sorted_indices, r->sorted_indices.p, sizeof(int64_t) * r->N,
                                 hipMemcpyDeviceToDevice, st));
    return TGT_OK;
}

int64_t tgt_reformat_num_tiles(const tgt_reformat_t* r) { return r ? (int64_t)(r->tiles.size() / 2) : -1; }
int64_t tgt_reformat_num_raw_edges(const tgt_reformat_t* r) { return r ? r->E_raw : -1; }

int tgt_reformat_export_tiles(const tgt_reformat_t* r, int32_t* h_tiles, int64_t* d_raw_edge_index, void* stream) {
    if (!r || (!r->tiles.empty() && !h_tiles) || (r->E_raw > 0 && !d_raw_edge_index)) {
        tgt::set_error("tgt_reformat_export_tiles: null pointer");
        return TGT_ERR_INVALID_ARG;
    }
    for (size_t i = 0; i < r->tiles.size(); ++i) h_tiles[i] = r->tiles[i];
    if (r->E_raw > 0)
        TGT_HIP_CHECK(hipMemcpyAsync(d_raw_edge_index, r->raw.p, sizeof(int64_t) * 2 * r->E_raw,
                                     hipMemcpyDeviceToDevice, (hipStream_t)stream));
    return TGT_OK;
}

int tgt_reformat_destroy(tgt_reformat_t* r) {
    delete r;
    return TGT_OK;
}

}  // extern "C"
