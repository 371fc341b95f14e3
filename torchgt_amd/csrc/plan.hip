// Graph plan: stable CSR-by-destination / CSC-by-source build and the
// degree-binned row schedule.
//
// Replaces, once per edge_index, what the reference redoes on every attention
// call: the per-edge gathers k[edge_index[0]], q[edge_index[1]] and the atomic
// scatter-adds over edge_index[1] (attn_module.py:146-147,180,185).  The sorted
// order is the stable one (ties keep the caller's edge order), the contract of
// the reference's edge sort (gt_sp/utils.py:354-356).
//
// The sort is a hand-written LSD radix sort (8-bit digits) whose ranking is
// position-based, so the result is bit-reproducible: integer LDS counters only
// count, they never decide an order.
#include "common.h"
#include <vector>
#include <new>
#include <stdlib.h>

namespace tgt {

static thread_local char g_err[512] = "";
void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}
const char* last_error() { return g_err; }

// ---------------------------------------------------------------------------
// kernels
// ---------------------------------------------------------------------------
// int64 endpoints -> uint32, with a range check (flag[0] = 1 on a bad index).
__global__ void k_convert_validate(const int64_t* __restrict__ src, const int64_t* __restrict__ dst,
                                   int64_t E, int64_t N, uint32_t* __restrict__ s32,
                                   uint32_t* __restrict__ d32, int* __restrict__ flag) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= E) return;
    int64_t s = src[i], d = dst[i];
    bool bad = (s < 0) | (s >= N) | (d < 0) | (d >= N);
    if (bad) { flag[0] = 1; s = 0; d = 0; }
    s32[i] = (uint32_t)s;
    d32[i] = (uint32_t)d;
}

// rowptr[r] = first sorted position whose key is >= r (r = 0 .. N): one thread per row, binary
// search in the sorted keys (a thread per position walking the gap to the next key would leave
// all the work to one thread when the keys are few or far apart).
__global__ void k_fill_rowptr(const uint32_t* __restrict__ keys, int64_t E, int64_t N,
                              int32_t* __restrict__ rowptr) {
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (r > N) return;
    int64_t lo = 0, hi = E;            // answer in [lo, hi]
    while (lo < hi) {
        const int64_t mid = (lo + hi) >> 1;
        if ((int64_t)keys[mid] < r) lo = mid + 1;
        else hi = mid;
    }
    rowptr[r] = (int32_t)lo;
}

__global__ void k_gather_col(const uint32_t* __restrict__ eid, const uint32_t* __restrict__ other,
                             int64_t E, int32_t* __restrict__ col, int32_t* __restrict__ eid_out) {
    int64_t pos = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (pos >= E) return;
    uint32_t e = eid[pos];
    col[pos] = (int32_t)other[e];
    eid_out[pos] = (int32_t)e;
}

// ---------------------------------------------------------------------------
// schedule kernels: rows are binned on the device, window by window; only per-window counts and the
// few long rows visit the host
// ---------------------------------------------------------------------------
constexpr int kSchedCats = kNumClass + 1;   // the wave classes, then "longer than a wave row"
constexpr int kSchedMaxWaves = 16;          // a window is one workgroup of up to 1024 threads, one per row

__device__ __forceinline__ int sched_category(int len, int wave_row_max) {
    if (len > wave_row_max) return kNumClass;
    if (len > 32) return 0;
    if (len > 16) return 1;
    if (len > 8) return 2;
    if (len > 4) return 3;
    return 4;
}

// counts[window * kSchedCats + cat] = rows of that category among the window's rows (blockDim.x rows)
__global__ void k_sched_count(const int32_t* __restrict__ rowptr, int64_t N, int wave_row_max,
                              uint32_t* __restrict__ counts) {
    __shared__ uint32_t c[kSchedCats];
    if (threadIdx.x < kSchedCats) c[threadIdx.x] = 0;
    __syncthreads();
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int cat = r < N ? sched_category(rowptr[r + 1] - rowptr[r], wave_row_max) : -1;
#pragma unroll
    for (int k = 0; k < kSchedCats; ++k) {
        const uint64_t b = __ballot(cat == k);
        if ((threadIdx.x & 63) == 0 && b) atomicAdd(&c[k], (uint32_t)__popcll(b));   // integer count: order-free
    }
    __syncthreads();
    if (threadIdx.x < kSchedCats) counts[(int64_t)blockIdx.x * kSchedCats + threadIdx.x] = c[threadIdx.x];
}

// Rows keep their order inside a (window, category): position = offs[window, cat] + rank among the
// window's rows.  Wave-class rows become schedule items at items[base + position]; long rows are
// listed (row, first edge, length) for the host.
__global__ void k_sched_fill(const int32_t* __restrict__ rowptr, int64_t N, int wave_row_max,
                             const uint32_t* __restrict__ offs, int64_t base, Item* __restrict__ items,
                             int32_t* __restrict__ long_rows) {
    __shared__ uint32_t wave_cnt[kSchedMaxWaves][kSchedCats];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int start = 0, len = 0, cat = -1;
    if (r < N) {
        start = rowptr[r];
        len = rowptr[r + 1] - start;
        cat = sched_category(len, wave_row_max);
    }
    const uint64_t lower = lane == 0 ? 0ull : (~0ull >> (64 - lane));
    uint32_t rank = 0;
#pragma unroll
    for (int k = 0; k < kSchedCats; ++k) {
        const uint64_t b = __ballot(cat == k);
        if (cat == k) rank = (uint32_t)__popcll(b & lower);
        if (lane == 0) wave_cnt[wave][k] = (uint32_t)__popcll(b);
    }
    __syncthreads();
    if (cat < 0) return;
    uint32_t pos = offs[(int64_t)blockIdx.x * kSchedCats + cat] + rank;
    for (int w = 0; w < wave; ++w) pos += wave_cnt[w][cat];
    if (cat < kNumClass) {
        if (items) items[base + pos] = Item{(int32_t)r, start, len, -1};
    } else if (long_rows) {
        long_rows[3 * (int64_t)pos + 0] = (int32_t)r;
        long_rows[3 * (int64_t)pos + 1] = start;
        long_rows[3 * (int64_t)pos + 2] = len;
    }
}

// out[i] = col[idx[i]]
__global__ void k_gather_i32(const int32_t* __restrict__ col, const int32_t* __restrict__ idx, int n,
                             int32_t* __restrict__ out) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = col[idx[i]];
}

// One workgroup of 64 threads writes one wave record from its descriptor (layout: WaveRec in common.h).
__global__ __launch_bounds__(64) void k_build_records(const WaveDesc* __restrict__ desc, const Item* __restrict__ items_d,
                                                      const Item* __restrict__ items_s, const int32_t* __restrict__ col_d,
                                                      const int32_t* __restrict__ eid_d, const int32_t* __restrict__ col_s,
                                                      const int32_t* __restrict__ eid_s, WaveRecLayout L, int lpe,
                                                      int32_t* __restrict__ recs) {
    const WaveDesc d = desc[blockIdx.x];
    int32_t* out = recs + (int64_t)blockIdx.x * L.stride;
    const int t = threadIdx.x;
    const uint32_t kind = d.code & 7u;
    const bool src = (d.code & kDescSrcSide) != 0;
    const int count = (int)(d.code >> 8);
    const Item* items = src ? items_s : items_d;
    const int32_t* col = src ? col_s : col_d;
    const int32_t* eid = src ? eid_s : eid_d;
    if (t == 0) out[0] = (int32_t)d.code;
    if (kind == kDescNone) return;
    if (kind == kDescBlock) {
        if (t == 0) {
            const Item it = items[d.first];
            out[4] = it.row; out[5] = it.start; out[6] = it.len; out[7] = it.part;
        }
        return;
    }
    if (t < count) {
        const Item it = items[d.first + t];
        out[L.off_row + t] = it.row;
        out[L.off_start + t] = it.start;
        out[L.off_len + t] = it.len;
    }
    if (!class_inline(lpe, (int)kind)) return;
    const int S = slots_for_class(lpe, (int)kind);
    const int groups = kWave / lpe;
    if (t < groups) {
        const int i = t / S, sl = t % S;
        if (i < count) {
            const Item it = items[d.first + i];
            for (int u = 0; u < 4; ++u) {
                const int e = sl + u * S;
                const int ec = e < it.len ? e : it.len - 1;
                out[L.off_col + 4 * t + u] = it.len > 0 ? col[it.start + ec] : 0;
                out[L.off_eid + 4 * t + u] = it.len > 0 ? eid[it.start + ec] : 0;
            }
        }
    }
}

// ---------------------------------------------------------------------------
// host helpers
// ---------------------------------------------------------------------------
// Sort edge ids by `keys32` (stable) and fill one Side's rowptr / col / eid.
static int build_side(const uint32_t* keys32, const uint32_t* other32, int64_t E, int64_t N,
                      RadixSorter& sorter, Side& side, hipStream_t st) {
    const uint32_t* kin = keys32;
    const uint32_t* vin = nullptr;
    if (E > 0) {
        int rc = sorter.sort(keys32, nullptr, E, bits_for(N), st, &kin, &vin);
        if (rc) return rc;
    }
    const int T = 256;
    hipLaunchKernelGGL(k_fill_rowptr, dim3((unsigned)((N + 1 + T - 1) / T)), dim3(T), 0, st, kin, E, N,
                       side.rowptr);
    if (E > 0)
        hipLaunchKernelGGL(k_gather_col, dim3((unsigned)((E + T - 1) / T)), dim3(T), 0, st, vin, other32,
                           E, side.col, side.eid);
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

static int env_int(const char* name, int dflt) {
    const char* v = getenv(name);
    if (!v || !*v) return dflt;
    const int x = atoi(v);
    return x > 0 ? x : dflt;
}

static int window_rows() {
    int w = env_int("TGT_WINDOW_ROWS", tgt::kWindowRows);
    w = (w + 63) / 64 * 64;
    return w > 64 * kSchedMaxWaves ? 64 * kSchedMaxWaves : w;
}

// Row schedule.  Rows are taken window by window (a window = window_rows() consecutive node ids).
// A row of up to kWaveRowMax edges is one wave item; the wave items of a window are grouped by length
// class (longest first) and keep row order inside a class, so the lanes of a wave see uniform lengths.
// A longer row is walked by whole workgroups: balanced segments, each a workgroup item that is
// scheduled with the window most of its other endpoints lie in (so that the rows a segment gathers
// are the ones the window's own rows load); if there is more than one segment their partial sums
// meet in the workspace.
static int build_schedule(int64_t N, Side& side, hipStream_t st) {
    // tuning overrides (experiments only; the defaults are the measured best)
    const int kWaveRowMax = env_int("TGT_WAVE_ROW_MAX", tgt::kWaveRowMax);
    const int kBlockSeg = env_int("TGT_BLOCK_SEG", tgt::kBlockSeg);
    const int kSpreadSeg = env_int("TGT_SPREAD_SEG", tgt::kSpreadSeg);
    const int W = window_rows();
    const int nwin = (int)((N + W - 1) / W);
    side.n_windows = nwin;
    DevBuf counts, long_d;
    const size_t ncnt = (size_t)kSchedCats * nwin;
    TGT_HIP_CHECK(counts.alloc(sizeof(uint32_t) * ncnt));
    hipLaunchKernelGGL(k_sched_count, dim3(nwin), dim3(W), 0, st, side.rowptr, N, kWaveRowMax, counts.as<uint32_t>());
    TGT_HIP_CHECK(hipGetLastError());
    std::vector<uint32_t> cnt(ncnt), offs(ncnt);
    TGT_HIP_CHECK(hipMemcpyAsync(cnt.data(), counts.p, sizeof(uint32_t) * ncnt, hipMemcpyDeviceToHost, st));
    TGT_HIP_CHECK(hipStreamSynchronize(st));
    // positions: wave items run over (window, class); long rows over windows
    uint32_t n_wave = 0, n_long = 0;
    for (int w = 0; w < nwin; ++w) {
        for (int c = 0; c < kNumClass; ++c) { offs[(size_t)w * kSchedCats + c] = n_wave; n_wave += cnt[(size_t)w * kSchedCats + c]; }
        offs[(size_t)w * kSchedCats + kNumClass] = n_long;
        n_long += cnt[(size_t)w * kSchedCats + kNumClass];
    }
    side.win_class_off = offs;
    side.win_class_cnt = cnt;
    TGT_HIP_CHECK(hipMemcpyAsync(counts.p, offs.data(), sizeof(uint32_t) * ncnt, hipMemcpyHostToDevice, st));
    // the long rows (few) come to the host, which cuts them into workgroup items
    std::vector<int32_t> longs((size_t)3 * n_long);
    if (n_long > 0) {
        TGT_HIP_CHECK(long_d.alloc(sizeof(int32_t) * (size_t)3 * n_long));
        hipLaunchKernelGGL(k_sched_fill, dim3(nwin), dim3(W), 0, st, side.rowptr, N, kWaveRowMax, counts.as<uint32_t>(),
                           (int64_t)0, (Item*)nullptr, long_d.as<int32_t>());
        TGT_HIP_CHECK(hipGetLastError());
        TGT_HIP_CHECK(hipMemcpyAsync(longs.data(), long_d.p, sizeof(int32_t) * longs.size(), hipMemcpyDeviceToHost, st));
        TGT_HIP_CHECK(hipStreamSynchronize(st));
    }
    std::vector<Item> items;
    std::vector<int32_t> split_row, split_off, part2split, split_grp, mid;
    int32_t n_groups = 0;
    int32_t n_parts = 0;
    for (int64_t i = 0; i < (int64_t)n_long; ++i) {
        const int32_t r = longs[3 * i], b = longs[3 * i + 1], len = longs[3 * i + 2];
        int nseg = (len + kBlockSeg - 1) / kBlockSeg;
        // a row with many segments (a global node) gets short ones: each is scheduled next to the rows it gathers
        const bool spread = nseg > kSpreadSegs;
        if (spread) nseg = (len + kSpreadSeg - 1) / kSpreadSeg;
        if (nseg == 1) {
            items.push_back(Item{r, b, len, -1});
            mid.push_back(b + len / 2);
            side.block_spread.push_back(0);
            continue;
        }
        const int seg = (len + nseg - 1) / nseg;
        split_off.push_back(n_parts);
        for (int s = 0; s < nseg; ++s) {
            const int o = s * seg;
            const int l = (o + seg <= len) ? seg : (len - o);
            part2split.push_back((int32_t)split_row.size());
            items.push_back(Item{r, b + o, l, n_parts++});
            mid.push_back(b + o + l / 2);
            side.block_spread.push_back(spread ? 1 : 0);
        }
        split_row.push_back(r);
        split_grp.push_back(n_groups);
        if (nseg > kCombineFan) n_groups += (nseg + kCombineFan - 1) / kCombineFan;
    }
    split_off.push_back(n_parts);
    split_grp.push_back(n_groups);
    side.n_groups = n_groups;
    side.n_block_items = (int32_t)items.size();
    side.n_items = (int32_t)(items.size() + n_wave);
    side.n_split = (int32_t)split_row.size();
    side.n_parts = n_parts;
    side.block_len.resize(items.size());
    side.block_home.assign(items.size(), 0);
    for (size_t i = 0; i < items.size(); ++i) side.block_len[i] = items[i].len;
    TGT_HIP_CHECK(hipMalloc((void**)&side.items, sizeof(Item) * ((size_t)side.n_items + 1)));
    TGT_HIP_CHECK(hipMalloc((void**)&side.split_row, sizeof(int32_t) * (split_row.size() + 1)));
    TGT_HIP_CHECK(hipMalloc((void**)&side.split_off, sizeof(int32_t) * split_off.size()));
    TGT_HIP_CHECK(hipMalloc((void**)&side.part2split, sizeof(int32_t) * (part2split.size() + 1)));
    TGT_HIP_CHECK(hipMalloc((void**)&side.split_grp, sizeof(int32_t) * split_grp.size()));
    TGT_HIP_CHECK(hipMemcpyAsync(side.split_grp, split_grp.data(), sizeof(int32_t) * split_grp.size(), hipMemcpyHostToDevice, st));
    DevBuf mid_d, home_d;
    if (!items.empty()) {
        TGT_HIP_CHECK(hipMemcpyAsync(side.items, items.data(), sizeof(Item) * items.size(), hipMemcpyHostToDevice, st));
        // home window of a workgroup item: the window of the other endpoint in the middle of its edges
        const int nb = (int)items.size();
        TGT_HIP_CHECK(mid_d.alloc(sizeof(int32_t) * nb));
        TGT_HIP_CHECK(home_d.alloc(sizeof(int32_t) * nb));
        TGT_HIP_CHECK(hipMemcpyAsync(mid_d.p, mid.data(), sizeof(int32_t) * nb, hipMemcpyHostToDevice, st));
        hipLaunchKernelGGL(k_gather_i32, dim3((nb + 255) / 256), dim3(256), 0, st, side.col, mid_d.as<int32_t>(), nb,
                           home_d.as<int32_t>());
        TGT_HIP_CHECK(hipGetLastError());
        TGT_HIP_CHECK(hipMemcpyAsync(side.block_home.data(), home_d.p, sizeof(int32_t) * nb, hipMemcpyDeviceToHost, st));
    }
    if (!split_row.empty()) {
        TGT_HIP_CHECK(hipMemcpyAsync(side.split_row, split_row.data(), sizeof(int32_t) * split_row.size(),
                                     hipMemcpyHostToDevice, st));
        TGT_HIP_CHECK(hipMemcpyAsync(side.part2split, part2split.data(), sizeof(int32_t) * part2split.size(),
                                     hipMemcpyHostToDevice, st));
    }
    TGT_HIP_CHECK(hipMemcpyAsync(side.split_off, split_off.data(), sizeof(int32_t) * split_off.size(),
                                 hipMemcpyHostToDevice, st));
    // the wave items (the bulk) are written by the device
    hipLaunchKernelGGL(k_sched_fill, dim3(nwin), dim3(W), 0, st, side.rowptr, N, kWaveRowMax, counts.as<uint32_t>(),
                       (int64_t)side.n_block_items, side.items, (int32_t*)nullptr);
    TGT_HIP_CHECK(hipGetLastError());
    TGT_HIP_CHECK(hipStreamSynchronize(st));   // the host vectors and the scratch buffers die at return
    for (int32_t& h : side.block_home) h = h / W;   // node id -> window
    return TGT_OK;
}

// ---------------------------------------------------------------------------
// launch descriptors
// ---------------------------------------------------------------------------
// Workgroups reach the 8 XCDs round-robin (workgroup id mod 8) and every XCD has its own L2.  The
// windows are cut into 8 contiguous ranges of about equal work, XCD x walks range x in window order,
// and inside a window the workgroup items homed there come first, then the waves of its rows, longest
// class first - for the backward both views of the window side by side.  What the rows of a window
// load (their own q/k/v/dout rows, the rows of their self-loops, the window's share of a global node's
// segment) then meets in one L2 at about the same time.
namespace {
// Workgroup items homed at window w_items and wave descriptors of window w of one view (either may be -1:
// none), appended to `waves`; `cost` grows by a rough measure of the work.  part 0: the heavy share (segments of ordinary long rows and the rows of the longest class, which
// run for many steps and whose edges have no tie to the window), part 1: the rest (segments of a row that
// spans the graph, which gather exactly the window's rows, and the short rows).
void append_side(std::vector<WaveDesc>& waves, float& cost, const Side& s, int w, int w_items, int lpe, bool src_side,
                 const std::vector<std::vector<int32_t>>& homed, int part) {
    if (w_items >= 0) {
        for (int32_t it : homed[w_items]) {
            if ((s.block_spread[it] != 0) != (part == 1)) continue;
            // close a partly filled workgroup first: a workgroup item takes all four waves
            while (waves.size() % 4) waves.push_back(WaveDesc{0, kDescNone});
            for (int k = 0; k < 4; ++k) waves.push_back(WaveDesc{it, desc_code(kDescBlock, src_side, 0)});
            cost += 1.0f + s.block_len[it] / 128.0f;
        }
    }
    if (w < 0) return;
    for (int c = (part == 0 ? 0 : 1); c < (part == 0 ? 1 : kNumClass); ++c) {
        const uint32_t n = s.win_class_cnt[(size_t)w * (kNumClass + 1) + c];
        const uint32_t first = s.n_block_items + s.win_class_off[(size_t)w * (kNumClass + 1) + c];
        const uint32_t ipw = (uint32_t)rows_per_wave(lpe, c);
        for (uint32_t i = 0; i < n; i += ipw) {
            waves.push_back(WaveDesc{(int32_t)(first + i), desc_code((uint32_t)c, src_side, n - i < ipw ? n - i : ipw)});
            cost += c == 0 ? 0.75f : 0.25f;
        }
    }
}

// descriptors of all windows -> block order.  XCD x gets a contiguous range of windows; it first walks the
// heavy share of all its windows (long work first keeps the end of the launch short), then window by window.
int place(const std::vector<const Side*>& sides, int lpe, void** d_out, int32_t* n_blocks, hipStream_t st) {
    const int nwin = sides[0]->n_windows;
    const bool heavy_first = env_int("TGT_HEAVY_FIRST", 1) == 1;
    std::vector<std::vector<std::vector<int32_t>>> homed(sides.size());
    for (size_t k = 0; k < sides.size(); ++k) {
        homed[k].resize(nwin > 0 ? nwin : 1);
        for (int32_t i = 0; i < sides[k]->n_block_items; ++i) {
            int h = sides[k]->block_home[i];
            h = h < 0 ? 0 : (h >= nwin ? nwin - 1 : h);
            homed[k][h].push_back(i);
        }
    }
    // 8 contiguous window ranges with about equal numbers of edges and rows
    int bound[9];
    bound[0] = 0;
    {
        std::vector<double> cost(nwin + 1, 0.0);
        for (int w = 0; w < nwin; ++w) {
            double c = 0.0;
            for (const Side* sd : sides) {
                for (int32_t it : homed[sd == sides[0] ? 0 : 1][w]) c += 1.0 + sd->block_len[it] / 128.0;
                for (int k = 0; k < kNumClass; ++k)
                    c += (k == 0 ? 0.75 : 0.25) * ((sd->win_class_cnt[(size_t)w * (kNumClass + 1) + k] + rows_per_wave(lpe, k) - 1) /
                                                   rows_per_wave(lpe, k));
            }
            cost[w + 1] = cost[w] + c;
        }
        int x = 1;
        for (int w = 0; w < nwin && x < 8; ++w)
            while (x < 8 && cost[w + 1] * 8 >= cost[nwin] * x) bound[x++] = w + 1;
        while (x <= 8) bound[x++] = nwin;
    }
    // Per XCD and part: runs of whole workgroups.  Part 0 (heavy share) of all windows of the range first.  In
    // part 1 the segments homed at a window run `lead` windows ahead of the window's rows: close enough in
    // time for the rows to meet in the L2, and the last windows of a range end with short rows only - the
    // chain of a split row (partial slot, arrival, sums of the group and of the row) is not left for the end.
    const int lead = env_int("TGT_SEGMENT_LEAD", 6);
    std::vector<WaveDesc> xw[8];
    for (int x = 0; x < 8; ++x) {
        float c = 0.f;
        std::vector<WaveDesc>& wv = xw[x];
        const int w0 = bound[x], w1 = bound[x + 1];
        if (heavy_first) {
            // one view after the other: the long rows of the destination view gather k and v rows, those of the source
            // view q, dout and the per-node scalars; side by side the two sets compete for the L2 (870 K nodes with
            // 50 edges per row: 3 % faster one after the other; no difference where long rows are few)
            for (size_t k = 0; k < sides.size(); ++k)
                for (int w = w0; w < w1; ++w) append_side(wv, c, *sides[k], w, w, lpe, k == 1, homed[k], 0);
            while (wv.size() % 4) wv.push_back(WaveDesc{0, kDescNone});
        }
        // the segments of the last half of the range go first: when the launch ends no split row is still
        // being added up (those windows give up meeting their segment in the L2)
        const int w_early = w1 - (w1 - w0) / env_int("TGT_EARLY_SHARE", 2);
        for (int w = w_early; w < w1; ++w)
            for (size_t k = 0; k < sides.size(); ++k) append_side(wv, c, *sides[k], -1, w, lpe, k == 1, homed[k], 1);
        for (int w = w0 - lead; w < w1; ++w) {
            const int wi = w + lead < w_early ? w + lead : -1;        // segments of the window `lead` ahead
            for (size_t k = 0; k < sides.size(); ++k) {
                if (!heavy_first) append_side(wv, c, *sides[k], w >= w0 ? w : -1, w >= w0 ? w : -1, lpe, k == 1, homed[k], 0);
                append_side(wv, c, *sides[k], w >= w0 ? w : -1, wi >= w0 ? wi : -1, lpe, k == 1, homed[k], 1);
            }
            while (wv.size() % 4) wv.push_back(WaveDesc{0, kDescNone});
        }
    }
    size_t per = 0;
    for (int x = 0; x < 8; ++x) per = std::max(per, xw[x].size() / 4);
    const size_t nb = per * 8;
    std::vector<WaveDesc> placed(nb * 4 + 4, WaveDesc{0, kDescNone});
    for (int x = 0; x < 8; ++x)
        for (size_t b = 0; b < xw[x].size() / 4; ++b)
            for (int k = 0; k < 4; ++k) placed[(b * 8 + x) * 4 + k] = xw[x][b * 4 + k];
    // descriptors -> records, on the device (the edge lists never visit the host)
    const WaveRecLayout L(lpe);
    const size_t n_rec = nb * 4;
    *n_blocks = (int32_t)nb;
    if (n_rec == 0) return TGT_OK;
    DevBuf desc_d;
    TGT_HIP_CHECK(desc_d.alloc(sizeof(WaveDesc) * n_rec));
    TGT_HIP_CHECK(hipMemcpyAsync(desc_d.p, placed.data(), sizeof(WaveDesc) * n_rec, hipMemcpyHostToDevice, st));
    const size_t bytes = n_rec * (size_t)L.stride * sizeof(int32_t);
    TGT_HIP_CHECK(hipMalloc(d_out, bytes));
    TGT_HIP_CHECK(hipMemsetAsync(*d_out, 0, bytes, st));
    const Side* sd = sides[0];
    const Side* ss = sides.size() > 1 ? sides[1] : sides[0];
    hipLaunchKernelGGL(k_build_records, dim3((unsigned)n_rec), dim3(64), 0, st, desc_d.as<WaveDesc>(), sd->items, ss->items,
                       sd->col, sd->eid, ss->col, ss->eid, L, lpe, static_cast<int32_t*>(*d_out));
    TGT_HIP_CHECK(hipGetLastError());
    TGT_HIP_CHECK(hipStreamSynchronize(st));    // the descriptors are freed on return
    return TGT_OK;
}
}  // namespace

const Schedule* plan_schedule_if_ready(const tgt_plan* plan, int lpe) {
    for (int idx = 0; idx < kNumLpe; ++idx)
        if ((1 << idx) == lpe) return plan->sched[idx].ready ? &plan->sched[idx] : nullptr;
    return nullptr;
}

const Schedule* plan_schedule(const tgt_plan* plan_c, int lpe, hipStream_t st) {
    int idx = 0;
    while (idx < kNumLpe && (1 << idx) != lpe) ++idx;
    if (idx == kNumLpe) { set_error("no schedule for %d lanes per edge", lpe); return nullptr; }
    tgt_plan* plan = const_cast<tgt_plan*>(plan_c);
    Schedule& sc = plan->sched[idx];
    if (sc.ready) return &sc;
    if (place({&plan->dst}, lpe, &sc.fwd, &sc.fwd_blocks, st) != TGT_OK) return nullptr;
    if (place({&plan->dst, &plan->src}, lpe, &sc.bwd, &sc.bwd_blocks, st) != TGT_OK) return nullptr;
    sc.ready = true;
    return &sc;
}

// inv[eid[c]] = c, then pos[p] = inv[eid_src[p]]: where each edge of the source-sorted order sits in the
// destination-sorted order
__global__ void k_invert_perm(const int32_t* __restrict__ eid, int64_t E, int32_t* __restrict__ inv) {
    const int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (c < E) inv[eid[c]] = (int32_t)c;
}
__global__ void k_compose_perm(const int32_t* __restrict__ eid, const int32_t* __restrict__ inv, int64_t E,
                               int32_t* __restrict__ pos) {
    const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (p < E) pos[p] = inv[eid[p]];
}

__global__ void k_widen(const int32_t* __restrict__ in, int64_t n, int64_t* __restrict__ out) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = in[i];
}

// rows of nv vectors: out[i] = in[eid[i]] (inverse: out[eid[i]] = in[i])
template <typename V>
__global__ void k_permute_rows(const V* __restrict__ in, const int32_t* __restrict__ eid, int64_t E, int nv,
                               V* __restrict__ out, bool inverse) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= E * nv) return;
    const int64_t i = t / nv;
    const int v = (int)(t % nv);
    const int64_t j = eid[i];
    if (!inverse) out[i * nv + v] = in[j * nv + v];
    else out[j * nv + v] = in[i * nv + v];
}

static void free_side(Side& s) {
    if (s.rowptr) (void)hipFree(s.rowptr);
    if (s.col) (void)hipFree(s.col);
    if (s.eid) (void)hipFree(s.eid);
    if (s.pos) (void)hipFree(s.pos);
    if (s.items) (void)hipFree(s.items);
    if (s.split_row) (void)hipFree(s.split_row);
    if (s.split_off) (void)hipFree(s.split_off);
    if (s.part2split) (void)hipFree(s.part2split);
    if (s.split_grp) (void)hipFree(s.split_grp);
    s = Side();
}

static void free_schedules(tgt_plan* plan) {
    for (Schedule& sc : plan->sched) {
        if (sc.fwd) (void)hipFree(sc.fwd);
        if (sc.bwd) (void)hipFree(sc.bwd);
        sc = Schedule();
    }
}

static int create_impl(const int64_t* d_src, const int64_t* d_dst, int64_t E, int64_t N, hipStream_t st,
                       tgt_plan* plan) {
    plan->N = N;
    plan->E = E;
    TGT_HIP_CHECK(hipGetDevice(&plan->device));
    for (Side* s : {&plan->dst, &plan->src}) {
        TGT_HIP_CHECK(hipMalloc((void**)&s->rowptr, sizeof(int32_t) * (N + 1)));
        TGT_HIP_CHECK(hipMalloc((void**)&s->col, sizeof(int32_t) * (E ? E : 1)));
        TGT_HIP_CHECK(hipMalloc((void**)&s->eid, sizeof(int32_t) * (E ? E : 1)));
    }
    DevBuf s32, d32, flag;
    RadixSorter sorter;
    const size_t eb = sizeof(uint32_t) * (size_t)(E ? E : 1);
    TGT_HIP_CHECK(s32.alloc(eb));
    TGT_HIP_CHECK(d32.alloc(eb));
    TGT_HIP_CHECK(flag.alloc(sizeof(int)));
    {
        int rc0 = sorter.init(E);
        if (rc0) return rc0;
    }
    TGT_HIP_CHECK(hipMemsetAsync(flag.p, 0, sizeof(int), st));
    if (E > 0) {
        const int T = 256;
        hipLaunchKernelGGL(k_convert_validate, dim3((unsigned)((E + T - 1) / T)), dim3(T), 0, st, d_src,
                           d_dst, E, N, s32.as<uint32_t>(), d32.as<uint32_t>(), flag.as<int>());
        TGT_HIP_CHECK(hipGetLastError());
    }
    int h_flag = 0;
    TGT_HIP_CHECK(hipMemcpyAsync(&h_flag, flag.p, sizeof(int), hipMemcpyDeviceToHost, st));
    TGT_HIP_CHECK(hipStreamSynchronize(st));
    if (h_flag) {
        set_error("edge_index holds a node id outside [0, %lld)", (long long)N);
        return TGT_ERR_INDEX_RANGE;
    }
    int rc = build_side(d32.as<uint32_t>(), s32.as<uint32_t>(), E, N, sorter, plan->dst, st);
    if (rc) return rc;
    rc = build_side(s32.as<uint32_t>(), d32.as<uint32_t>(), E, N, sorter, plan->src, st);
    if (rc) return rc;
    rc = build_schedule(N, plan->dst, st);
    if (rc) return rc;
    rc = build_schedule(N, plan->src, st);
    if (rc) return rc;
    // the shape of the reference's node-level models (hidden 64: 8 heads of 8, or 4 of 16); other shapes on first use
    return plan_schedule(plan, 8, st) ? TGT_OK : TGT_ERR_HIP;
}

}  // namespace tgt

// ---------------------------------------------------------------------------
// C ABI
// ---------------------------------------------------------------------------
extern "C" {

int tgt_version(void) { return 1; }

int tgt_plan_enable_bias_order(tgt_plan_t* plan, void* stream) {
    if (!plan) { tgt::set_error("tgt_plan_enable_bias_order: null plan"); return TGT_ERR_INVALID_ARG; }
    if (plan->src.pos) return TGT_OK;
    const int64_t E = plan->E;
    hipStream_t st = (hipStream_t)stream;
    TGT_HIP_CHECK(hipMalloc((void**)&plan->src.pos, sizeof(int32_t) * (size_t)(E ? E : 1)));
    if (E == 0) return TGT_OK;
    tgt::DevBuf inv;
    TGT_HIP_CHECK(inv.alloc(sizeof(int32_t) * (size_t)E));
    const unsigned grid = (unsigned)((E + 255) / 256);
    hipLaunchKernelGGL(tgt::k_invert_perm, dim3(grid), dim3(256), 0, st, plan->dst.eid, E, inv.as<int32_t>());
    hipLaunchKernelGGL(tgt::k_compose_perm, dim3(grid), dim3(256), 0, st, plan->src.eid, inv.as<int32_t>(), E,
                       plan->src.pos);
    TGT_HIP_CHECK(hipGetLastError());
    TGT_HIP_CHECK(hipStreamSynchronize(st));      // the scratch buffer is freed on return
    return TGT_OK;
}

const char* tgt_error_string(int code) {
    switch (code) {
        case TGT_OK: return "ok";
        case TGT_ERR_INVALID_ARG: return "invalid argument";
        case TGT_ERR_INDEX_RANGE: return "edge endpoint out of range";
        case TGT_ERR_UNSUPPORTED: return "unsupported (H, d, dtype) combination";
        case TGT_ERR_HIP: return "HIP runtime error";
        case TGT_ERR_WORKSPACE: return "workspace too small or misaligned";
        default: return "unknown error";
    }
}

const char* tgt_last_error(void) { return tgt::last_error(); }

int tgt_plan_create(const int64_t* d_src, const int64_t* d_dst, int64_t E, int64_t N, void* stream,
                    tgt_plan_t** out_plan) {
    if (!out_plan || E < 0 || N < 1 || (E > 0 && (!d_src || !d_dst))) {
        tgt::set_error("tgt_plan_create: null pointer, E < 0 or N < 1");
        return TGT_ERR_INVALID_ARG;
    }
    if (E > 0x7fff0000LL || N > 0x7fff0000LL) {
        tgt::set_error("tgt_plan_create: E and N must fit 31 bits");
        return TGT_ERR_INVALID_ARG;
    }
    tgt_plan* plan = new (std::nothrow) tgt_plan();
    if (!plan) return TGT_ERR_INVALID_ARG;
    int rc = tgt::create_impl(d_src, d_dst, E, N, (hipStream_t)stream, plan);
    if (rc != TGT_OK) {
        tgt::free_side(plan->dst);
        tgt::free_side(plan->src);
        tgt::free_schedules(plan);
        delete plan;
        return rc;
    }
    *out_plan = plan;
    return TGT_OK;
}

int tgt_plan_destroy(tgt_plan_t* plan) {
    if (!plan) return TGT_OK;
    tgt::free_side(plan->dst);
    tgt::free_side(plan->src);
    tgt::free_schedules(plan);
    delete plan;
    return TGT_OK;
}

int tgt_plan_info(const tgt_plan_t* plan, int64_t info[16]) {
    if (!plan || !info) return TGT_ERR_INVALID_ARG;
    for (int i = 0; i < 16; ++i) info[i] = 0;
    info[0] = plan->N;
    info[1] = plan->E;
    info[2] = plan->dst.n_items;
    info[3] = plan->dst.n_split;
    info[4] = plan->dst.n_parts;
    info[5] = plan->src.n_items;
    info[6] = plan->src.n_split;
    info[7] = plan->src.n_parts;
    info[8] = tgt::kBlockSeg;
    info[9] = tgt::kWaveRowMax;
    info[10] = plan->dst.n_block_items;
    info[11] = plan->src.n_block_items;
    return TGT_OK;
}

int64_t tgt_plan_array_len(const tgt_plan_t* plan, int which) {
    if (!plan) return -1;
    switch (which) {
        case TGT_PLAN_ROWPTR_DST: case TGT_PLAN_ROWPTR_SRC: return plan->N + 1;
        case TGT_PLAN_COL_DST: case TGT_PLAN_EID_DST:
        case TGT_PLAN_COL_SRC: case TGT_PLAN_EID_SRC: return plan->E;
        case TGT_PLAN_POS_SRC: return plan->src.pos ? plan->E : 0;
        case TGT_PLAN_ITEMS_DST: return 4 * (int64_t)plan->dst.n_items;
        case TGT_PLAN_ITEMS_SRC: return 4 * (int64_t)plan->src.n_items;
        default: return -1;
    }
}

int tgt_plan_export(const tgt_plan_t* plan, int which, int32_t* h_out, int64_t capacity) {
    const int64_t n = tgt_plan_array_len(plan, which);
    if (n < 0 || !h_out || capacity < n) {
        tgt::set_error("tgt_plan_export: bad array id or capacity");
        return TGT_ERR_INVALID_ARG;
    }
    const void* p = nullptr;
    switch (which) {
        case TGT_PLAN_ROWPTR_DST: p = plan->dst.rowptr; break;
        case TGT_PLAN_COL_DST: p = plan->dst.col; break;
        case TGT_PLAN_EID_DST: p = plan->dst.eid; break;
        case TGT_PLAN_ROWPTR_SRC: p = plan->src.rowptr; break;
        case TGT_PLAN_COL_SRC: p = plan->src.col; break;
        case TGT_PLAN_EID_SRC: p = plan->src.eid; break;
        case TGT_PLAN_POS_SRC: p = plan->src.pos; break;
        case TGT_PLAN_ITEMS_DST: p = plan->dst.items; break;
        case TGT_PLAN_ITEMS_SRC: p = plan->src.items; break;
    }
    if (n == 0) return TGT_OK;
    TGT_HIP_CHECK(hipMemcpy(h_out, p, sizeof(int32_t) * n, hipMemcpyDeviceToHost));
    return TGT_OK;
}

int tgt_plan_sort_rows(const tgt_plan_t* plan, const void* d_in, int row_bytes, void* d_out, int direction, void* stream) {
    if (!plan || row_bytes < 1 || direction < 0 || direction > 2 || (plan->E > 0 && (!d_in || !d_out))) {
        tgt::set_error("tgt_plan_sort_rows: null pointer or bad row size");
        return TGT_ERR_INVALID_ARG;
    }
    if (plan->E == 0) return TGT_OK;
    hipStream_t st = (hipStream_t)stream;
    const int64_t E = plan->E;
    const int32_t* eid = direction == 2 ? plan->src.eid : plan->dst.eid;
    const bool inv = direction == 1;
#define TGT_LAUNCH_PERMUTE(V)                                                                                  \
    do {                                                                                                       \
        const int nv = row_bytes / (int)sizeof(V);                                                             \
        const int64_t total = E * nv;                                                                          \
        hipLaunchKernelGGL((tgt::k_permute_rows<V>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st,  \
                           (const V*)d_in, eid, E, nv, (V*)d_out, inv);                                        \
    } while (0)
    const uintptr_t al = (uintptr_t)d_in | (uintptr_t)d_out | (uintptr_t)row_bytes;
    if (al % 16 == 0) TGT_LAUNCH_PERMUTE(uint4);
    else if (al % 8 == 0) TGT_LAUNCH_PERMUTE(uint2);
    else if (al % 4 == 0) TGT_LAUNCH_PERMUTE(uint32_t);
    else if (al % 2 == 0) TGT_LAUNCH_PERMUTE(uint16_t);
    else TGT_LAUNCH_PERMUTE(uint8_t);
#undef TGT_LAUNCH_PERMUTE
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

int tgt_plan_edge_order_src(const tgt_plan_t* plan, int64_t* d_out, void* stream) {
    if (!plan || (plan->E > 0 && !d_out)) { tgt::set_error("tgt_plan_edge_order_src: null pointer"); return TGT_ERR_INVALID_ARG; }
    if (plan->E == 0) return TGT_OK;
    hipLaunchKernelGGL(tgt::k_widen, dim3((unsigned)((plan->E + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       plan->src.eid, plan->E, d_out);
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

int tgt_plan_edge_order(const tgt_plan_t* plan, int64_t* d_out, void* stream) {
    if (!plan || (plan->E > 0 && !d_out)) { tgt::set_error("tgt_plan_edge_order: null pointer"); return TGT_ERR_INVALID_ARG; }
    if (plan->E == 0) return TGT_OK;
    hipLaunchKernelGGL(tgt::k_widen, dim3((unsigned)((plan->E + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       plan->dst.eid, plan->E, d_out);
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

}  // extern "C"
