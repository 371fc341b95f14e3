// Stable LSD radix sort of (uint32 key, uint32 value) pairs, 8-bit digits.
//
// The ranking is position-based (ballots and prefix counts), so the output is
// the stable order - what numpy's argsort(kind='stable') gives - and is
// bit-reproducible: integer LDS counters only count, they never decide an order.
// Used for the CSR/CSC build (keys = destination / source node) and for the
// graph reordering (keys = partition id, new source id).
#include "common.h"
#include <mutex>
#include <unordered_map>
#include <utility>

namespace tgt {

constexpr int RS_THREADS = 256;
constexpr int RS_ITEMS = 16;
constexpr int RS_TILE = RS_THREADS * RS_ITEMS;   // 4096 keys per workgroup
constexpr int RS_WAVE_SPAN = kWave * RS_ITEMS;   // 1024 consecutive keys per wave

// Per-workgroup digit histogram, stored digit-major: hist[digit * nblocks + block].
__global__ __launch_bounds__(RS_THREADS) void k_rs_hist(const uint32_t* __restrict__ keys, int64_t n,
                                                        int shift, uint32_t* __restrict__ hist,
                                                        int nblocks) {
    __shared__ uint32_t h[256];
    const int tid = threadIdx.x;
    h[tid] = 0;
    __syncthreads();
    const int64_t base = (int64_t)blockIdx.x * RS_TILE;
#pragma unroll
    for (int i = 0; i < RS_ITEMS; ++i) {
        int64_t idx = base + i * RS_THREADS + tid;
        if (idx < n) atomicAdd(&h[(keys[idx] >> shift) & 255u], 1u);   // integer count: order-free
    }
    __syncthreads();
    hist[(int64_t)tid * nblocks + blockIdx.x] = h[tid];
}

// Workgroup `digit` turns its row of per-block counts into exclusive offsets and
// records the row total.
__global__ __launch_bounds__(256) void k_rs_scan_rows(uint32_t* __restrict__ hist, int nblocks,
                                                      uint32_t* __restrict__ totals) {
    __shared__ uint32_t part[256];
    const int tid = threadIdx.x;
    uint32_t* row = hist + (int64_t)blockIdx.x * nblocks;
    const int chunk = (nblocks + 255) / 256;
    const int b = tid * chunk;
    const int e = min(b + chunk, nblocks);
    uint32_t s = 0;
    for (int i = b; i < e; ++i) s += row[i];
    part[tid] = s;
    __syncthreads();
    for (int off = 1; off < 256; off <<= 1) {
        uint32_t x = tid >= off ? part[tid - off] : 0u;
        __syncthreads();
        part[tid] += x;
        __syncthreads();
    }
    uint32_t run = tid ? part[tid - 1] : 0u;
    for (int i = b; i < e; ++i) {
        uint32_t x = row[i];
        row[i] = run;
        run += x;
    }
    if (tid == 255) totals[blockIdx.x] = part[255];
}

// Stable scatter of one radix pass.  Each wave owns 1024 consecutive keys of the
// tile and ranks them in 16 rounds of 64; the rank of a key among equal digits is
// (count in earlier rounds) + (number of lower lanes with the same digit).  The tile
// is then put in digit order in LDS (stable), so that the writes to global memory go
// out as runs of consecutive addresses, one run per digit, instead of one scattered
// 4-byte store per key.
__global__ __launch_bounds__(RS_THREADS) void k_rs_scatter(
    const uint32_t* __restrict__ keys_in, const uint32_t* __restrict__ vals_in,
    uint32_t* __restrict__ keys_out, uint32_t* __restrict__ vals_out, int64_t n, int shift,
    const uint32_t* __restrict__ hist, const uint32_t* __restrict__ totals, int nblocks) {
    __shared__ uint32_t cnt[4][256];
    __shared__ uint32_t base[256];        // first output position of this tile's keys of a digit
    __shared__ uint32_t scan[256];        // scan of the global digit totals
    __shared__ uint32_t tstart[256];      // scan of the tile's digit counts: first LDS slot of a digit
    __shared__ uint32_t lkey[RS_TILE];
    __shared__ uint32_t lval[RS_TILE];
    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    for (int i = tid; i < 4 * 256; i += RS_THREADS) (&cnt[0][0])[i] = 0;
    scan[tid] = totals[tid];
    __syncthreads();

    volatile uint32_t* wcnt = &cnt[wave][0];
    uint32_t key[RS_ITEMS], rank[RS_ITEMS];
    const int64_t tbase = (int64_t)blockIdx.x * RS_TILE;
    const int64_t wbase = tbase + (int64_t)wave * RS_WAVE_SPAN;
    const uint64_t lower_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
#pragma unroll
    for (int r = 0; r < RS_ITEMS; ++r) {
        const int64_t idx = wbase + r * kWave + lane;
        const bool valid = idx < n;
        const uint32_t kk = valid ? keys_in[idx] : 0u;
        key[r] = kk;
        const uint32_t dg = (kk >> shift) & 255u;
        uint64_t same = __ballot(valid);
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            const bool bit = (dg >> b) & 1u;
            const uint64_t bal = __ballot(bit);
            same &= bit ? bal : ~bal;
        }
        uint32_t prior = 0;
        if (valid) prior = wcnt[dg];
        const uint32_t lower = (uint32_t)__popcll(same & lower_mask);
        rank[r] = prior + lower;
        if (valid && lower == 0) wcnt[dg] = prior + (uint32_t)__popcll(same);
    }
    __syncthreads();
    // exclusive prefix over the 4 waves (thread = digit); the tile's count of the digit
    {
        const uint32_t c0 = cnt[0][tid], c1 = cnt[1][tid], c2 = cnt[2][tid], c3 = cnt[3][tid];
        cnt[0][tid] = 0;
        cnt[1][tid] = c0;
        cnt[2][tid] = c0 + c1;
        cnt[3][tid] = c0 + c1 + c2;
        tstart[tid] = c0 + c1 + c2 + c3;
    }
    __syncthreads();
    // inclusive scans over the 256 digits: global totals and tile counts
    for (int off = 1; off < 256; off <<= 1) {
        const uint32_t x = tid >= off ? scan[tid - off] : 0u;
        const uint32_t y = tid >= off ? tstart[tid - off] : 0u;
        __syncthreads();
        scan[tid] += x;
        tstart[tid] += y;
        __syncthreads();
    }
    const uint32_t my_tstart = tid ? tstart[tid - 1] : 0u;
    base[tid] = (tid ? scan[tid - 1] : 0u) + hist[(int64_t)tid * nblocks + blockIdx.x];
    __syncthreads();
    tstart[tid] = my_tstart;              // now exclusive
    __syncthreads();
    // the tile in digit order (stable) in LDS
#pragma unroll
    for (int r = 0; r < RS_ITEMS; ++r) {
        const int64_t idx = wbase + r * kWave + lane;
        if (idx < n) {
            const uint32_t dg = (key[r] >> shift) & 255u;
            const uint32_t slot = tstart[dg] + cnt[wave][dg] + rank[r];
            lkey[slot] = key[r];
            lval[slot] = vals_in ? vals_in[idx] : (uint32_t)idx;
        }
    }
    __syncthreads();
    const int tile_n = (int)min((int64_t)RS_TILE, n - tbase);
    for (int i = tid; i < tile_n; i += RS_THREADS) {
        const uint32_t kk = lkey[i];
        const uint32_t dg = (kk >> shift) & 255u;
        const uint32_t pos = base[dg] + ((uint32_t)i - tstart[dg]);
        keys_out[pos] = kk;
        vals_out[pos] = lval[i];
    }
}


// allocator hooks (tgt_set_allocator); read on every call, set before the first plan is made
static tgt_alloc_fn g_alloc = nullptr;
static tgt_free_fn g_free = nullptr;
static void* g_alloc_user = nullptr;
// what the hook handed out and has not taken back: memory goes back to where it came from even if the
// hooks were set or cleared in between
static std::mutex g_hooked_mutex;
static std::unordered_map<void*, std::pair<tgt_free_fn, void*>> g_hooked;

hipError_t dev_alloc(void** p, size_t bytes, hipStream_t st) {
    if (bytes == 0) bytes = 4;
    const tgt_alloc_fn alloc = g_alloc;
    if (alloc) {
        *p = alloc(bytes, (void*)st, g_alloc_user);
        if (!*p) return hipErrorOutOfMemory;
        std::lock_guard<std::mutex> lock(g_hooked_mutex);
        g_hooked[*p] = std::make_pair(g_free, g_alloc_user);
        return hipSuccess;
    }
    return hipMalloc(p, bytes);
}
void dev_free(void* p) {
    if (!p) return;
    std::pair<tgt_free_fn, void*> how(nullptr, nullptr);
    {
        std::lock_guard<std::mutex> lock(g_hooked_mutex);
        auto it = g_hooked.find(p);
        if (it != g_hooked.end()) { how = it->second; g_hooked.erase(it); }
    }
    if (how.first) how.first(p, how.second);
    else (void)hipFree(p);
}

hipError_t DevBuf::alloc(size_t bytes, hipStream_t st) {
    if (p) { dev_free(p); p = nullptr; }
    return dev_alloc(&p, bytes, st);
}
DevBuf::~DevBuf() { dev_free(p); }

int bits_for(int64_t n) {
    int bits = 1;
    while (bits < 32 && ((int64_t)1 << bits) < n) ++bits;
    return bits;
}

int RadixSorter::init(int64_t n, hipStream_t st) {
    cap_ = n > 0 ? n : 1;
    nblocks_ = (int)((cap_ + RS_TILE - 1) / RS_TILE);
    const size_t eb = sizeof(uint32_t) * (size_t)cap_;
    TGT_HIP_CHECK(keysA_.alloc(eb, st));
    TGT_HIP_CHECK(keysB_.alloc(eb, st));
    TGT_HIP_CHECK(valsA_.alloc(eb, st));
    TGT_HIP_CHECK(valsB_.alloc(eb, st));
    TGT_HIP_CHECK(hist_.alloc(sizeof(uint32_t) * 256 * (size_t)nblocks_, st));
    TGT_HIP_CHECK(totals_.alloc(sizeof(uint32_t) * 256, st));
    return TGT_OK;
}

int RadixSorter::sort(const uint32_t* keys_in, const uint32_t* vals_in, int64_t n, int bits, hipStream_t st,
                      const uint32_t** keys_out, const uint32_t** vals_out) {
    if (n > cap_) { set_error("RadixSorter: n exceeds capacity"); return TGT_ERR_INVALID_ARG; }
    const int passes = (bits + 7) / 8 > 0 ? (bits + 7) / 8 : 1;
    const int nblocks = (int)((n + RS_TILE - 1) / RS_TILE);
    const uint32_t* kin = keys_in;
    const uint32_t* vin = vals_in;
    uint32_t* kout = keysA_.as<uint32_t>();
    uint32_t* vout = valsA_.as<uint32_t>();
    for (int p = 0; p < passes && n > 0; ++p) {
        const int shift = 8 * p;
        hipLaunchKernelGGL(k_rs_hist, dim3(nblocks), dim3(RS_THREADS), 0, st, kin, n, shift,
                           hist_.as<uint32_t>(), nblocks);
        hipLaunchKernelGGL(k_rs_scan_rows, dim3(256), dim3(256), 0, st, hist_.as<uint32_t>(), nblocks,
                           totals_.as<uint32_t>());
        hipLaunchKernelGGL(k_rs_scatter, dim3(nblocks), dim3(RS_THREADS), 0, st, kin, vin, kout, vout, n,
                           shift, hist_.as<uint32_t>(), totals_.as<uint32_t>(), nblocks);
        kin = kout;
        vin = vout;
        const bool toB = (kout == keysA_.as<uint32_t>());
        kout = toB ? keysB_.as<uint32_t>() : keysA_.as<uint32_t>();
        vout = toB ? valsB_.as<uint32_t>() : valsA_.as<uint32_t>();
    }
    TGT_HIP_CHECK(hipGetLastError());
    *keys_out = kin;
    *vals_out = vin;
    return TGT_OK;
}

}  // namespace tgt

extern "C" int tgt_set_allocator(tgt_alloc_fn alloc, tgt_free_fn free_fn, void* user) {
    if ((alloc == nullptr) != (free_fn == nullptr)) {
        tgt::set_error("tgt_set_allocator: give both functions or neither");
        return TGT_ERR_INVALID_ARG;
    }
    tgt::g_alloc = alloc;
    tgt::g_free = free_fn;
    tgt::g_alloc_user = user;
    return TGT_OK;
}
