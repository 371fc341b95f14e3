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
#include <mutex>
#include <utility>
#include <algorithm>
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

// skip_empty: rows without edges get no place in the schedule (-1)
__device__ __forceinline__ int sched_category(int len, int wave_row_max, bool skip_empty) {
    if (skip_empty && len == 0) return -1;
    if (len > wave_row_max) return kNumClass;
    if (len > 32) return 0;
    if (len > 16) return 1;
    if (len > 8) return 2;
    if (len > 4) return 3;
    return 4;
}

// counts[window * kSchedCats + cat] = rows of that category among the window's rows (blockDim.x rows)
__global__ void k_sched_count(const int32_t* __restrict__ rowptr, int64_t N, int wave_row_max, bool skip_empty,
                              uint32_t* __restrict__ counts) {
    __shared__ uint32_t c[kSchedCats];
    if (threadIdx.x < kSchedCats) c[threadIdx.x] = 0;
    __syncthreads();
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int cat = r < N ? sched_category(rowptr[r + 1] - rowptr[r], wave_row_max, skip_empty) : -1;
#pragma unroll
    for (int k = 0; k < kSchedCats; ++k) {
        const uint64_t b = __ballot(cat == k);
        if ((threadIdx.x & 63) == 0 && b) atomicAdd(&c[k], (uint32_t)__popcll(b));   // integer count: order-free
    }
    __syncthreads();
    if (threadIdx.x < kSchedCats) counts[(int64_t)blockIdx.x * kSchedCats + threadIdx.x] = c[threadIdx.x];
}

// Per side, written by the device and read back once: how many of everything the schedule holds.
struct SchedHeader { int32_t n_wave, n_long, n_block, n_split, n_parts, n_groups, pad0, pad1; };

// offs[window, cat]: first position of the window's rows of a category - wave classes count through
// (window, class) in that order, long rows through the windows - and the two totals.  One workgroup.
__global__ __launch_bounds__(1024) void k_sched_scan(const uint32_t* __restrict__ counts, int nwin,
                                                     uint32_t* __restrict__ offs, SchedHeader* __restrict__ hdr) {
    __shared__ uint32_t sw[1024], sl[1024];
    const int tid = threadIdx.x;
    const int chunk = (nwin + 1023) / 1024;
    const int b = min(tid * chunk, nwin), e = min(b + chunk, nwin);
    uint32_t ws = 0, ls = 0;
    for (int w = b; w < e; ++w) {
        for (int c = 0; c < kNumClass; ++c) ws += counts[(int64_t)w * kSchedCats + c];
        ls += counts[(int64_t)w * kSchedCats + kNumClass];
    }
    sw[tid] = ws; sl[tid] = ls;
    __syncthreads();
    for (int off = 1; off < 1024; off <<= 1) {
        const uint32_t x = tid >= off ? sw[tid - off] : 0u, y = tid >= off ? sl[tid - off] : 0u;
        __syncthreads();
        sw[tid] += x; sl[tid] += y;
        __syncthreads();
    }
    uint32_t rw = tid ? sw[tid - 1] : 0u, rl = tid ? sl[tid - 1] : 0u;
    for (int w = b; w < e; ++w) {
        for (int c = 0; c < kNumClass; ++c) { offs[(int64_t)w * kSchedCats + c] = rw; rw += counts[(int64_t)w * kSchedCats + c]; }
        offs[(int64_t)w * kSchedCats + kNumClass] = rl;
        rl += counts[(int64_t)w * kSchedCats + kNumClass];
    }
    if (tid == 1023) { hdr->n_wave = (int32_t)sw[1023]; hdr->n_long = (int32_t)sl[1023]; }
}

// Rows keep their order inside a (window, category): position = offs[window, cat] + rank among the
// window's rows.  Wave-class rows become wave items at items[position]; long rows are listed (row, first
// edge, length) for the kernels that cut them into workgroup items.
__global__ void k_sched_fill(const int32_t* __restrict__ rowptr, int64_t N, int wave_row_max, bool skip_empty,
                             const uint32_t* __restrict__ offs, Item* __restrict__ items,
                             int32_t* __restrict__ long_rows, int64_t cap_long) {
    __shared__ uint32_t wave_cnt[kSchedMaxWaves][kSchedCats];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int start = 0, len = 0, cat = -1;
    if (r < N) {
        start = rowptr[r];
        len = rowptr[r + 1] - start;
        cat = sched_category(len, wave_row_max, skip_empty);
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
        items[pos] = Item{(int32_t)r, start, len, -1};
    } else if ((int64_t)pos < cap_long) {
        long_rows[3 * (int64_t)pos + 0] = (int32_t)r;
        long_rows[3 * (int64_t)pos + 1] = start;
        long_rows[3 * (int64_t)pos + 2] = len;
    }
}

// How a long row is cut (the same arithmetic on the device and wherever it is checked): balanced segments
// of at most block_seg edges; a row with more than spread_segs of those (a global node) gets segments of
// spread_seg edges instead, each scheduled next to the rows it gathers.
struct CutParams { int block_seg, spread_segs, spread_seg, combine_fan, window; };
__host__ __device__ inline void cut_row(const CutParams& cp, int len, int& nseg, int& seg, bool& spread) {
    nseg = (len + cp.block_seg - 1) / cp.block_seg;
    spread = nseg > cp.spread_segs;
    if (spread) nseg = (len + cp.spread_seg - 1) / cp.spread_seg;
    seg = (len + nseg - 1) / nseg;
}

// Long rows -> where their workgroup items, partial slots and combine groups start.  One workgroup: every
// thread takes a run of consecutive rows of the list (it is short: rows of more than a wave row's edges), the
// runs' totals are scanned in LDS, then every thread writes its rows.
__global__ __launch_bounds__(1024) void k_cut_rows(const int32_t* __restrict__ long_rows, SchedHeader* __restrict__ hdr,
                                                   CutParams cp, int32_t* __restrict__ row_item_off,
                                                   int32_t* __restrict__ row_split_idx, int32_t* __restrict__ row_part_off,
                                                   int32_t* __restrict__ split_row, int32_t* __restrict__ split_off,
                                                   int32_t* __restrict__ split_grp) {
    __shared__ uint32_t sh[4][1024];
    const int n_long = hdr->n_long;
    const int tid = threadIdx.x;
    const int chunk = (n_long + 1023) / 1024;
    const int b = min(tid * chunk, n_long), e = min(b + chunk, n_long);
    uint32_t items = 0, splits = 0, parts = 0, groups = 0;
    for (int i = b; i < e; ++i) {
        int nseg, seg;
        bool spread;
        cut_row(cp, long_rows[3 * i + 2], nseg, seg, spread);
        items += (uint32_t)nseg;
        if (nseg > 1) { splits += 1; parts += (uint32_t)nseg; }
        if (nseg > cp.combine_fan) groups += (uint32_t)((nseg + cp.combine_fan - 1) / cp.combine_fan);
    }
    sh[0][tid] = items; sh[1][tid] = splits; sh[2][tid] = parts; sh[3][tid] = groups;
    __syncthreads();
    for (int off = 1; off < 1024; off <<= 1) {
        uint32_t x[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) x[k] = tid >= off ? sh[k][tid - off] : 0u;
        __syncthreads();
#pragma unroll
        for (int k = 0; k < 4; ++k) sh[k][tid] += x[k];
        __syncthreads();
    }
    // running totals in front of this thread's rows
    items = tid ? sh[0][tid - 1] : 0u; splits = tid ? sh[1][tid - 1] : 0u;
    parts = tid ? sh[2][tid - 1] : 0u; groups = tid ? sh[3][tid - 1] : 0u;
    for (int i = b; i < e; ++i) {
        int nseg, seg;
        bool spread;
        cut_row(cp, long_rows[3 * i + 2], nseg, seg, spread);
        const bool is_split = nseg > 1;
        row_item_off[i] = (int32_t)items;
        row_split_idx[i] = is_split ? (int32_t)splits : -1;
        row_part_off[i] = (int32_t)parts;
        if (is_split) {
            split_row[splits] = long_rows[3 * i];
            split_off[splits] = (int32_t)parts;
            split_grp[splits] = (int32_t)groups;
            splits += 1; parts += (uint32_t)nseg;
        }
        items += (uint32_t)nseg;
        if (nseg > cp.combine_fan) groups += (uint32_t)((nseg + cp.combine_fan - 1) / cp.combine_fan);
    }
    if (tid == 1023) {
        row_item_off[n_long] = (int32_t)sh[0][1023];
        split_off[sh[1][1023]] = (int32_t)sh[2][1023];
        split_grp[sh[1][1023]] = (int32_t)sh[3][1023];
        hdr->n_block = (int32_t)sh[0][1023];
        hdr->n_split = (int32_t)sh[1][1023];
        hdr->n_parts = (int32_t)sh[2][1023];
        hdr->n_groups = (int32_t)sh[3][1023];
    }
}

// What the host needs to know of a workgroup item to place it: the window it is scheduled with (the one
// of the other endpoint in the middle of its edges), its edges, whether it is a short segment of a row
// that spans the graph.
struct BlockMeta { int32_t home, len, spread; };

// One thread per workgroup item: finds its row in the offsets and writes the item.
__global__ void k_emit_items(const int32_t* __restrict__ long_rows, const SchedHeader* __restrict__ hdr, CutParams cp,
                             const int32_t* __restrict__ row_item_off, const int32_t* __restrict__ row_split_idx,
                             const int32_t* __restrict__ row_part_off, const int32_t* __restrict__ col,
                             Item* __restrict__ block_items, BlockMeta* __restrict__ meta,
                             int32_t* __restrict__ part2split) {
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= hdr->n_block) return;
    int lo = 0, hi = hdr->n_long - 1;               // last row whose first item is <= j
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (row_item_off[mid] <= j) lo = mid;
        else hi = mid - 1;
    }
    const int i = lo, sgm = j - row_item_off[i];
    const int r = long_rows[3 * i], b = long_rows[3 * i + 1], len = long_rows[3 * i + 2];
    int nseg, seg;
    bool spread;
    cut_row(cp, len, nseg, seg, spread);
    const int o = sgm * seg;
    const int l = (o + seg <= len) ? seg : (len - o);
    const int sidx = row_split_idx[i];
    const int part = sidx >= 0 ? row_part_off[i] + sgm : -1;
    block_items[j] = Item{r, b + o, l, part};
    meta[j] = BlockMeta{col[b + o + l / 2] / cp.window, l, spread ? 1 : 0};
    if (part >= 0) part2split[part] = sidx;
}

// A run: `waves` consecutive waves of the list of XCD `xcd` that do the same kind of thing.
//   rows:       the wave items [first, first + n) of one (window, class), rows_per_wave of them per wave
//   block item: workgroup item `first`; its four waves carry the same record
//   nothing:    padding to whole workgroups, and behind the end of a list
struct Run { int32_t wave0, waves, first, n; uint32_t code; int32_t xcd; int32_t pad[2]; };

// One workgroup per run; its waves write the run's wave records in turn (layout: WaveRec in common.h).  Wave lw of
// XCD x's list is wave lw % 4 of that XCD's (lw / 4)-th workgroup, and workgroup b of the launch runs on XCD b mod 8:
// record ((lw / 4) * 8 + x) * 4 + lw % 4.  Everything a kernel uses of a record is written: no clearing pass.
__global__ __launch_bounds__(256) void k_build_records(const Run* __restrict__ runs, const Item* __restrict__ items_d,
                                                       const Item* __restrict__ items_s, const Item* __restrict__ bitems_d,
                                                       const Item* __restrict__ bitems_s, const int32_t* __restrict__ col_d,
                                                       const int32_t* __restrict__ eid_d, const int32_t* __restrict__ col_s,
                                                       const int32_t* __restrict__ eid_s, WaveRecLayout L, int lpe,
                                                       int32_t* __restrict__ recs) {
    const Run run = runs[blockIdx.x];
    const int t = threadIdx.x & 63;
    const uint32_t kind = run.code & 7u;
    const bool src = (run.code & kDescSrcSide) != 0;
    const Item* items = src ? items_s : items_d;
    const int32_t* col = src ? col_s : col_d;
    const int32_t* eid = src ? eid_s : eid_d;
    const int ipw = kind < (uint32_t)kNumClass ? rows_per_wave(lpe, (int)kind) : 1;
    const int S = kind < (uint32_t)kNumClass ? slots_for_class(lpe, (int)kind) : 1;
    const bool inl = kind < (uint32_t)kNumClass && class_inline(lpe, (int)kind);
    const int groups = kWave / lpe;
    for (int w = threadIdx.x >> 6; w < run.waves; w += 4) {
        const int lw = run.wave0 + w;
        int32_t* out = recs + (((int64_t)(lw >> 2) * 8 + run.xcd) * 4 + (lw & 3)) * L.stride;
        if (kind == kDescNone) {
            if (t == 0) out[0] = (int32_t)kDescNone;
            continue;
        }
        if (kind == kDescBlock) {
            if (t == 0) {
                const Item it = (src ? bitems_s : bitems_d)[run.first];
                out[0] = (int32_t)run.code;
                out[4] = it.row; out[5] = it.start; out[6] = it.len; out[7] = it.part;
            }
            continue;
        }
        const int first = run.first + w * ipw;
        const int count = min(ipw, run.n - w * ipw);
        if (t == 0) out[0] = (int32_t)desc_code(kind, src, (uint32_t)count);
        if (t < groups) {                               // every lane group's entries, zeros behind the last row
            const int i = t / S, sl = t % S;
            Item it{0, 0, 0, -1};
            if (i < count) it = items[first + i];
            out[L.off_row + t] = it.row;                // per lane group: a lane finds its row without knowing the class
            out[L.off_start + t] = it.start;
            out[L.off_len + t] = it.len;
            if (inl) for (int u = 0; u < 4; ++u) {
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
// meet in the workspace.  All of it is made on the device; the host reads back the counts (one copy for
// both views, together with the range-check flag) and, if there are long rows, what it needs to place
// their workgroup items.
struct SideScratch {
    DevBuf long_rows, row_item_off, row_split_idx, row_part_off, meta;
    int64_t cap_long = 0, cap_block = 0;
    CutParams cp{};
    int wave_row_max = 0, W = 0, nwin = 0;
};

// ints of the report in front of the per-window counts: two headers, the flag, padding
constexpr int kReportHead = 32;
constexpr int kReportFlag = 16;

static int schedule_device(int64_t N, int64_t E, Side& side, SideScratch& sc, int32_t* report, int side_idx,
                           bool skip_empty, hipStream_t st) {
    // tuning overrides (experiments only; the defaults are the measured best)
    sc.wave_row_max = env_int("TGT_WAVE_ROW_MAX", tgt::kWaveRowMax);
    sc.cp.block_seg = env_int("TGT_BLOCK_SEG", tgt::kBlockSeg);
    sc.cp.spread_seg = env_int("TGT_SPREAD_SEG", tgt::kSpreadSeg);
    sc.cp.spread_segs = kSpreadSegs;
    sc.cp.combine_fan = kCombineFan;
    sc.W = window_rows();
    sc.cp.window = sc.W;
    sc.nwin = (int)((N + sc.W - 1) / sc.W);
    side.n_windows = sc.nwin;
    const size_t ncnt = (size_t)kSchedCats * sc.nwin;
    SchedHeader* hdr = reinterpret_cast<SchedHeader*>(report) + side_idx;
    uint32_t* counts = reinterpret_cast<uint32_t*>(report) + kReportHead + (size_t)side_idx * 2 * ncnt;
    uint32_t* offs = counts + ncnt;
    // bounds known before anything is counted: a long row has more than wave_row_max edges, a row of len edges
    // is cut into at most len / min(block_seg, spread_seg) + 1 segments
    sc.cap_long = std::min<int64_t>(N, E / (sc.wave_row_max + 1)) + 1;
    const int min_seg = std::max(1, std::min(sc.cp.block_seg, sc.cp.spread_seg));
    sc.cap_block = E / min_seg + sc.cap_long + 1;
    TGT_HIP_CHECK(dev_alloc((void**)&side.items, sizeof(Item) * (size_t)(N + 1), st));
    TGT_HIP_CHECK(dev_alloc((void**)&side.block_items, sizeof(Item) * (size_t)sc.cap_block, st));
    TGT_HIP_CHECK(dev_alloc((void**)&side.split_row, sizeof(int32_t) * (size_t)(sc.cap_long + 1), st));
    TGT_HIP_CHECK(dev_alloc((void**)&side.split_off, sizeof(int32_t) * (size_t)(sc.cap_long + 1), st));
    TGT_HIP_CHECK(dev_alloc((void**)&side.split_grp, sizeof(int32_t) * (size_t)(sc.cap_long + 1), st));
    TGT_HIP_CHECK(dev_alloc((void**)&side.part2split, sizeof(int32_t) * (size_t)(sc.cap_block + 1), st));
    TGT_HIP_CHECK(sc.long_rows.alloc(sizeof(int32_t) * 3 * (size_t)sc.cap_long, st));
    TGT_HIP_CHECK(sc.row_item_off.alloc(sizeof(int32_t) * (size_t)(sc.cap_long + 1), st));
    TGT_HIP_CHECK(sc.row_split_idx.alloc(sizeof(int32_t) * (size_t)sc.cap_long, st));
    TGT_HIP_CHECK(sc.row_part_off.alloc(sizeof(int32_t) * (size_t)sc.cap_long, st));
    TGT_HIP_CHECK(sc.meta.alloc(sizeof(BlockMeta) * (size_t)sc.cap_block, st));
    hipLaunchKernelGGL(k_sched_count, dim3(sc.nwin), dim3(sc.W), 0, st, side.rowptr, N, sc.wave_row_max, skip_empty, counts);
    hipLaunchKernelGGL(k_sched_scan, dim3(1), dim3(1024), 0, st, counts, sc.nwin, offs, hdr);
    hipLaunchKernelGGL(k_sched_fill, dim3(sc.nwin), dim3(sc.W), 0, st, side.rowptr, N, sc.wave_row_max, skip_empty, offs, side.items,
                       sc.long_rows.as<int32_t>(), sc.cap_long);
    hipLaunchKernelGGL(k_cut_rows, dim3(1), dim3(1024), 0, st, sc.long_rows.as<int32_t>(), hdr, sc.cp,
                       sc.row_item_off.as<int32_t>(), sc.row_split_idx.as<int32_t>(), sc.row_part_off.as<int32_t>(),
                       side.split_row, side.split_off, side.split_grp);
    hipLaunchKernelGGL(k_emit_items, dim3((unsigned)((sc.cap_block + 255) / 256)), dim3(256), 0, st, sc.long_rows.as<int32_t>(),
                       hdr, sc.cp, sc.row_item_off.as<int32_t>(), sc.row_split_idx.as<int32_t>(), sc.row_part_off.as<int32_t>(),
                       side.col, side.block_items, sc.meta.as<BlockMeta>(), side.part2split);
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;
}

// The counts are on the host: sizes of the view's schedule and the per-window tables the placement reads.
static void schedule_counts(Side& side, const SideScratch& sc, const int32_t* report, int side_idx) {
    const SchedHeader& h = reinterpret_cast<const SchedHeader*>(report)[side_idx];
    const size_t ncnt = (size_t)kSchedCats * sc.nwin;
    const uint32_t* counts = reinterpret_cast<const uint32_t*>(report) + kReportHead + (size_t)side_idx * 2 * ncnt;
    side.win_class_cnt.assign(counts, counts + ncnt);
    side.win_class_off.assign(counts + ncnt, counts + 2 * ncnt);
    side.n_block_items = h.n_block;
    side.n_items = h.n_block + h.n_wave;
    side.n_split = h.n_split;
    side.n_parts = h.n_parts;
    side.n_groups = h.n_groups;
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
// One XCD's list as runs of waves.
struct XcdList {
    std::vector<Run> runs;
    int32_t waves = 0, xcd = 0;
    void add(uint32_t code, int32_t first, int32_t n, int32_t waves_of_run) {
        if (waves_of_run <= 0) return;
        runs.push_back(Run{waves, waves_of_run, first, n, code, xcd, {0, 0}});
        waves += waves_of_run;
    }
    void pad4() { if (waves % 4) add(kDescNone, 0, 0, 4 - waves % 4); }
};

// Workgroup items homed at window w_items and the waves of window w of one view (either may be -1: none), appended
// to the list.  part 0: the heavy share (segments of ordinary long rows and the rows of the longest class, which
// run for many steps and whose edges have no tie to the window), part 1: the rest (segments of a row that
// spans the graph, which gather exactly the window's rows, and the short rows).
void append_side(XcdList& xl, const Side& s, int w, int w_items, int lpe, bool src_side, int part) {
    if (w_items >= 0) {
        for (int32_t q = s.homed_off[w_items]; q < s.homed_off[w_items + 1]; ++q) {
            const int32_t it = s.homed_idx[q];
            if ((s.block_spread[it] != 0) != (part == 1)) continue;
            xl.pad4();      // close a partly filled workgroup first: a workgroup item takes all four waves
            xl.add(desc_code(kDescBlock, src_side, 0), it, 1, 4);
        }
    }
    if (w < 0) return;
    for (int c = (part == 0 ? 0 : 1); c < (part == 0 ? 1 : kNumClass); ++c) {
        const uint32_t n = s.win_class_cnt[(size_t)w * (kNumClass + 1) + c];
        const int ipw = rows_per_wave(lpe, c);
        xl.add(desc_code((uint32_t)c, src_side, 0), (int32_t)s.win_class_off[(size_t)w * (kNumClass + 1) + c], (int32_t)n,
               (int32_t)((n + ipw - 1) / ipw));
    }
}

// runs of all windows -> block order.  XCD x gets a contiguous range of windows; it first walks the
// heavy share of all its windows (long work first keeps the end of the launch short), then window by window.
// The host vectors and device buffers handed back feed an asynchronous copy and the kernel behind it: the caller
// keeps them until the stream has been synchronised.
int place(const std::vector<const Side*>& sides, int lpe, void** d_out, int32_t* n_blocks, hipStream_t st,
          std::vector<Run>& all_runs, DevBuf& runs_d) {
    const int nwin = sides[0]->n_windows;
    const bool heavy_first = env_int("TGT_HEAVY_FIRST", 1) == 1;
    // 8 contiguous window ranges with about equal numbers of edges and rows
    int bound[9];
    bound[0] = 0;
    {
        std::vector<double> cost(nwin + 1, 0.0);
        for (int w = 0; w < nwin; ++w) {
            double c = 0.0;
            for (size_t k = 0; k < sides.size(); ++k) {
                const Side* sd = sides[k];
                for (int32_t q = sd->homed_off[w]; q < sd->homed_off[w + 1]; ++q) c += 1.0 + sd->block_len[sd->homed_idx[q]] / 128.0;
                for (int kk = 0; kk < kNumClass; ++kk)
                    c += (kk == 0 ? 0.75 : 0.25) * ((sd->win_class_cnt[(size_t)w * (kNumClass + 1) + kk] + rows_per_wave(lpe, kk) - 1) /
                                                    rows_per_wave(lpe, kk));
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
    const int lead = env_int("TGT_SEGMENT_LEAD", 3);
    XcdList xl[8];
    for (int x = 0; x < 8; ++x) {
        XcdList& wv = xl[x];
        wv.xcd = x;
        wv.runs.reserve((size_t)(bound[x + 1] - bound[x] + 8) * 8 * sides.size());
        const int w0 = bound[x], w1 = bound[x + 1];
        if (heavy_first) {
            // one view after the other: the long rows of the destination view gather k and v rows, those of the source
            // view q, dout and the per-node scalars; side by side the two sets compete for the L2 (870 K nodes with
            // 50 edges per row: 3 % faster one after the other; no difference where long rows are few)
            for (size_t k = 0; k < sides.size(); ++k)
                for (int w = w0; w < w1; ++w) append_side(wv, *sides[k], w, w, lpe, k == 1, 0);
            wv.pad4();
        }
        // the segments of the last half of the range go first: when the launch ends no split row is still
        // being added up (those windows give up meeting their segment in the L2)
        const int w_early = w1 - (w1 - w0) / env_int("TGT_EARLY_SHARE", 2);
        for (int w = w_early; w < w1; ++w)
            for (size_t k = 0; k < sides.size(); ++k) append_side(wv, *sides[k], -1, w, lpe, k == 1, 1);
        for (int w = w0 - lead; w < w1; ++w) {
            const int wi = w + lead < w_early ? w + lead : -1;        // segments of the window `lead` ahead
            for (size_t k = 0; k < sides.size(); ++k) {
                if (!heavy_first) append_side(wv, *sides[k], w >= w0 ? w : -1, w >= w0 ? w : -1, lpe, k == 1, 0);
                append_side(wv, *sides[k], w >= w0 ? w : -1, wi >= w0 ? wi : -1, lpe, k == 1, 1);
            }
            wv.pad4();
        }
    }
    int32_t per = 0;
    for (int x = 0; x < 8; ++x) per = std::max(per, (xl[x].waves + 3) / 4);
    const size_t nb = (size_t)per * 8;
    const WaveRecLayout L(lpe);
    const size_t n_rec = nb * 4;
    *n_blocks = (int32_t)nb;
    if (n_rec == 0) return TGT_OK;
    all_runs.clear();
    for (int x = 0; x < 8; ++x) {
        xl[x].add(kDescNone, 0, 0, per * 4 - xl[x].waves);       // behind the end of the list: records that say "nothing"
        all_runs.insert(all_runs.end(), xl[x].runs.begin(), xl[x].runs.end());
    }
    TGT_HIP_CHECK(runs_d.alloc(sizeof(Run) * all_runs.size(), st));
    TGT_HIP_CHECK(hipMemcpyAsync(runs_d.p, all_runs.data(), sizeof(Run) * all_runs.size(), hipMemcpyHostToDevice, st));
    const size_t bytes = n_rec * (size_t)L.stride * sizeof(int32_t);
    TGT_HIP_CHECK(dev_alloc(d_out, bytes, st));
    const Side* sd = sides[0];
    const Side* ss = sides.size() > 1 ? sides[1] : sides[0];
    hipLaunchKernelGGL(k_build_records, dim3((unsigned)all_runs.size()), dim3(256), 0, st, runs_d.as<Run>(), sd->items, ss->items,
                       sd->block_items, ss->block_items, sd->col, sd->eid, ss->col, ss->eid, L, lpe, static_cast<int32_t*>(*d_out));
    TGT_HIP_CHECK(hipGetLastError());
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
    // the descriptors of a shape are made once, whichever thread or stream asks first
    std::lock_guard<std::mutex> lock(plan->sched_mutex);
    if (sc.ready) return &sc;
    std::vector<Run> runs_f, runs_b;
    DevBuf rf, rb;
    int rc = place({&plan->dst}, lpe, &sc.fwd, &sc.fwd_blocks, st, runs_f, rf);
    if (rc == TGT_OK) rc = place({&plan->dst, &plan->src}, lpe, &sc.bwd, &sc.bwd_blocks, st, runs_b, rb);
    // the host vectors feed asynchronous copies: they may go once the stream is idle
    if (hipStreamSynchronize(st) != hipSuccess && rc == TGT_OK) { set_error("hipStreamSynchronize failed"); rc = TGT_ERR_HIP; }
    if (rc != TGT_OK) {
        dev_free(sc.fwd); dev_free(sc.bwd);
        sc = Schedule();
        return nullptr;
    }
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
    dev_free(s.rowptr); dev_free(s.col); dev_free(s.eid); dev_free(s.pos);
    dev_free(s.items); dev_free(s.block_items);
    dev_free(s.split_row); dev_free(s.split_off); dev_free(s.part2split); dev_free(s.split_grp);
    s = Side();
}

static void free_schedules(tgt_plan* plan) {
    for (Schedule& sc : plan->sched) {
        dev_free(sc.fwd); dev_free(sc.bwd);
        sc = Schedule();
    }
}

static int create_impl(const int64_t* d_src, const int64_t* d_dst, int64_t E, int64_t N, hipStream_t st,
                       tgt_plan* plan) {
    plan->N = N;
    plan->E = E;
    TGT_HIP_CHECK(hipGetDevice(&plan->device));
    for (Side* s : {&plan->dst, &plan->src}) {
        TGT_HIP_CHECK(dev_alloc((void**)&s->rowptr, sizeof(int32_t) * (N + 1), st));
        TGT_HIP_CHECK(dev_alloc((void**)&s->col, sizeof(int32_t) * (E ? E : 1), st));
        TGT_HIP_CHECK(dev_alloc((void**)&s->eid, sizeof(int32_t) * (E ? E : 1), st));
    }
    DevBuf s32, d32, report_d;
    RadixSorter sorter;
    const size_t eb = sizeof(uint32_t) * (size_t)(E ? E : 1);
    TGT_HIP_CHECK(s32.alloc(eb, st));
    TGT_HIP_CHECK(d32.alloc(eb, st));
    {
        int rc0 = sorter.init(E, st);
        if (rc0) return rc0;
    }
    // what comes back to the host, in one copy: the two schedule headers, the range-check flag, and per view the
    // per-window row counts and their offsets
    const int W = window_rows();
    const int nwin = (int)((N + W - 1) / W);
    const size_t report_ints = kReportHead + 4 * (size_t)kSchedCats * nwin;
    TGT_HIP_CHECK(report_d.alloc(sizeof(int32_t) * report_ints, st));
    TGT_HIP_CHECK(hipMemsetAsync(report_d.p, 0, sizeof(int32_t) * kReportHead, st));
    int32_t* report = report_d.as<int32_t>();
    if (E > 0) {
        const int T = 256;
        hipLaunchKernelGGL(k_convert_validate, dim3((unsigned)((E + T - 1) / T)), dim3(T), 0, st, d_src,
                           d_dst, E, N, s32.as<uint32_t>(), d32.as<uint32_t>(), report + kReportFlag);
        TGT_HIP_CHECK(hipGetLastError());
    }
    // out-of-range endpoints were replaced by node 0 (and flagged): everything below runs on valid ids
    int rc = build_side(d32.as<uint32_t>(), s32.as<uint32_t>(), E, N, sorter, plan->dst, st);
    if (rc) return rc;
    rc = build_side(s32.as<uint32_t>(), d32.as<uint32_t>(), E, N, sorter, plan->src, st);
    if (rc) return rc;
    SideScratch scr_d, scr_s;
    rc = schedule_device(N, E, plan->dst, scr_d, report, 0, plan->rows_with_edges_only, st);
    if (rc) return rc;
    rc = schedule_device(N, E, plan->src, scr_s, report, 1, plan->rows_with_edges_only, st);
    if (rc) return rc;
    std::vector<int32_t> h_report(report_ints);
    TGT_HIP_CHECK(hipMemcpyAsync(h_report.data(), report, sizeof(int32_t) * report_ints, hipMemcpyDeviceToHost, st));
    TGT_HIP_CHECK(hipStreamSynchronize(st));
    if (h_report[kReportFlag]) {
        set_error("edge_index holds a node id outside [0, %lld)", (long long)N);
        return TGT_ERR_INDEX_RANGE;
    }
    schedule_counts(plan->dst, scr_d, h_report.data(), 0);
    schedule_counts(plan->src, scr_s, h_report.data(), 1);
    // graphs with rows longer than a wave row: where their workgroup items go (second and last read-back)
    std::vector<BlockMeta> meta_d(plan->dst.n_block_items), meta_s(plan->src.n_block_items);
    if (!meta_d.empty())
        TGT_HIP_CHECK(hipMemcpyAsync(meta_d.data(), scr_d.meta.p, sizeof(BlockMeta) * meta_d.size(), hipMemcpyDeviceToHost, st));
    if (!meta_s.empty())
        TGT_HIP_CHECK(hipMemcpyAsync(meta_s.data(), scr_s.meta.p, sizeof(BlockMeta) * meta_s.size(), hipMemcpyDeviceToHost, st));
    if (!meta_d.empty() || !meta_s.empty()) TGT_HIP_CHECK(hipStreamSynchronize(st));
    for (auto sm : {std::make_pair(&plan->dst, &meta_d), std::make_pair(&plan->src, &meta_s)}) {
        Side& sd = *sm.first;
        const std::vector<BlockMeta>& m = *sm.second;
        sd.block_home.resize(m.size()); sd.block_len.resize(m.size()); sd.block_spread.resize(m.size());
        for (size_t i = 0; i < m.size(); ++i) {
            sd.block_home[i] = m[i].home; sd.block_len[i] = m[i].len; sd.block_spread[i] = (uint8_t)m[i].spread;
        }
        // workgroup items by the window they are scheduled with (counting sort: item order is kept inside a window)
        const int nw = sd.n_windows > 0 ? sd.n_windows : 1;
        sd.homed_off.assign((size_t)nw + 1, 0);
        for (int32_t& h : sd.block_home) { h = h < 0 ? 0 : (h >= nw ? nw - 1 : h); sd.homed_off[(size_t)h + 1]++; }
        for (int w = 0; w < nw; ++w) sd.homed_off[(size_t)w + 1] += sd.homed_off[w];
        sd.homed_idx.resize(m.size());
        std::vector<int32_t> at(sd.homed_off.begin(), sd.homed_off.end() - 1);
        for (size_t i = 0; i < m.size(); ++i) sd.homed_idx[at[sd.block_home[i]]++] = (int32_t)i;
    }
    // the shape of the reference's node-level models (hidden 64: 8 heads of 8, or 4 of 16); other shapes on first use
    return plan_schedule(plan, 8, st) ? TGT_OK : TGT_ERR_HIP;
}

// ---------------------------------------------------------------------------
// content key of an edge list
// ---------------------------------------------------------------------------
__device__ __forceinline__ uint64_t mix64(uint64_t x) {
    x ^= x >> 33; x *= 0xff51afd7ed558ccdull;
    x ^= x >> 33; x *= 0xc4ceb9fe1a85ec53ull;
    x ^= x >> 33;
    return x;
}
constexpr int kHashBlocks = 1024;
// Two 64-bit sums over all 2E endpoints of mixed (value, position) pairs: a sum does not depend on the order
// of the additions, so the key is the same whatever the grid does, and a value that moves or changes moves it.
__global__ __launch_bounds__(256) void k_hash_partial(const int64_t* __restrict__ src, const int64_t* __restrict__ dst,
                                                      int64_t E, uint64_t* __restrict__ partial) {
    __shared__ uint64_t sh[2][4];
    uint64_t a = 0, b = 0;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < 2 * E; i += (int64_t)gridDim.x * blockDim.x) {
        const uint64_t v = (uint64_t)(i < E ? src[i] : dst[i - E]);
        a += mix64(v * 0x9e3779b97f4a7c15ull + (uint64_t)i * 0xd6e8feb86659fd93ull + 0x2545f4914f6cdd1dull);
        b += mix64((v + (uint64_t)i * 0xa0761d6478bd642full) ^ 0xe7037ed1a0b428dbull);
    }
    for (int off = 32; off > 0; off >>= 1) { a += __shfl_xor(a, off); b += __shfl_xor(b, off); }
    if ((threadIdx.x & 63) == 0) { sh[0][threadIdx.x >> 6] = a; sh[1][threadIdx.x >> 6] = b; }
    __syncthreads();
    if (threadIdx.x == 0) {
        partial[2 * blockIdx.x] = sh[0][0] + sh[0][1] + sh[0][2] + sh[0][3];
        partial[2 * blockIdx.x + 1] = sh[1][0] + sh[1][1] + sh[1][2] + sh[1][3];
    }
}
__global__ __launch_bounds__(64) void k_hash_final(const uint64_t* __restrict__ partial, int n, int64_t E,
                                                   uint64_t* __restrict__ out) {
    uint64_t a = 0, b = 0;
    for (int i = threadIdx.x; i < n; i += 64) { a += partial[2 * i]; b += partial[2 * i + 1]; }
    for (int off = 32; off > 0; off >>= 1) { a += __shfl_xor(a, off); b += __shfl_xor(b, off); }
    if (threadIdx.x == 0) { out[0] = mix64(a ^ (uint64_t)E); out[1] = mix64(b + (uint64_t)E); }
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
    TGT_HIP_CHECK(tgt::dev_alloc((void**)&plan->src.pos, sizeof(int32_t) * (size_t)(E ? E : 1), st));
    if (E == 0) return TGT_OK;
    tgt::DevBuf inv;
    TGT_HIP_CHECK(inv.alloc(sizeof(int32_t) * (size_t)E, st));
    const unsigned grid = (unsigned)((E + 255) / 256);
    hipLaunchKernelGGL(tgt::k_invert_perm, dim3(grid), dim3(256), 0, st, plan->dst.eid, E, inv.as<int32_t>());
    hipLaunchKernelGGL(tgt::k_compose_perm, dim3(grid), dim3(256), 0, st, plan->src.eid, inv.as<int32_t>(), E,
                       plan->src.pos);
    TGT_HIP_CHECK(hipGetLastError());
    return TGT_OK;      // the scratch buffer goes back to its allocator behind the kernels that read it
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

int tgt_edge_index_hash(const int64_t* d_src, const int64_t* d_dst, int64_t E, void* stream, uint64_t h_key[2]) {
    if (!h_key || E < 0 || (E > 0 && (!d_src || !d_dst))) {
        tgt::set_error("tgt_edge_index_hash: null pointer or E < 0");
        return TGT_ERR_INVALID_ARG;
    }
    hipStream_t st = (hipStream_t)stream;
    const int nb = (int)std::min<int64_t>(tgt::kHashBlocks, std::max<int64_t>(1, (2 * E + 1023) / 1024));
    tgt::DevBuf buf;
    TGT_HIP_CHECK(buf.alloc(sizeof(uint64_t) * (2 * (size_t)nb + 2), st));
    uint64_t* partial = buf.as<uint64_t>();
    hipLaunchKernelGGL(tgt::k_hash_partial, dim3(nb), dim3(256), 0, st, d_src, d_dst, E, partial);
    hipLaunchKernelGGL(tgt::k_hash_final, dim3(1), dim3(64), 0, st, partial, nb, E, partial + 2 * nb);
    TGT_HIP_CHECK(hipGetLastError());
    TGT_HIP_CHECK(hipMemcpyAsync(h_key, partial + 2 * nb, 2 * sizeof(uint64_t), hipMemcpyDeviceToHost, st));
    TGT_HIP_CHECK(hipStreamSynchronize(st));
    return TGT_OK;
}

static int plan_create_checked(const int64_t* d_src, const int64_t* d_dst, int64_t E, int64_t N, void* stream,
                               bool rows_with_edges_only, tgt_plan_t** out_plan) {
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
    plan->rows_with_edges_only = rows_with_edges_only;
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

int tgt_plan_create(const int64_t* d_src, const int64_t* d_dst, int64_t E, int64_t N, void* stream,
                    tgt_plan_t** out_plan) {
    return plan_create_checked(d_src, d_dst, E, N, stream, false, out_plan);
}

int tgt_plan_create_remaining(const int64_t* d_src, const int64_t* d_dst, int64_t E, int64_t N, void* stream,
                              tgt_plan_t** out_plan) {
    return plan_create_checked(d_src, d_dst, E, N, stream, true, out_plan);
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
    if (n == 0) return TGT_OK;
    if (which == TGT_PLAN_ITEMS_DST || which == TGT_PLAN_ITEMS_SRC) {   // workgroup items, then wave items
        const tgt::Side& s = which == TGT_PLAN_ITEMS_DST ? plan->dst : plan->src;
        const int64_t nb = 4 * (int64_t)s.n_block_items;
        if (nb > 0) TGT_HIP_CHECK(hipMemcpy(h_out, s.block_items, sizeof(int32_t) * nb, hipMemcpyDeviceToHost));
        if (n > nb) TGT_HIP_CHECK(hipMemcpy(h_out + nb, s.items, sizeof(int32_t) * (n - nb), hipMemcpyDeviceToHost));
        return TGT_OK;
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
    }
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
