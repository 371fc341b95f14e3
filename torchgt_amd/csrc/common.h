// Shared host-side declarations of the gfx950 sparse-attention library.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include <mutex>
#include <vector>
#include "../../include/torchgt_hip.h"

namespace tgt {

constexpr int kWave = 64;            // CDNA wavefront width
constexpr int kBlock = 256;          // threads per workgroup of the attention kernels (4 waves)
constexpr int kWaveRowMax = 256;     // a row of up to this many edges is walked by (part of) one wave
constexpr int kBlockSeg = 1024;      // longer rows are walked by whole workgroups, in segments of at most this many edges
constexpr int kSpreadSegs = 8;       // rows with more segments than this get shorter segments:
constexpr int kSpreadSeg = 256;      // their length (more workgroups, each next to the rows of its sources; 128 and 512 measured slower)
constexpr int kWindowRows = 128;     // rows of one schedule window (consecutive node ids walked together on one XCD)
constexpr int kCombineFan = 32;      // partial slots one combine step adds (= lane groups of a workgroup at 8 lanes per edge)
constexpr int kNumClass = 5;         // wave item length classes: >32, <=32, <=16, <=8, <=4

void set_error(const char* fmt, ...);
// reduce.hip: up to eight fixed-order sums of workgroup partials in one launch
int reduce_partials(const tgt_reduce_desc* descs, int count, int dtype, hipStream_t st);

#define TGT_HIP_CHECK(expr)                                                        \
    do {                                                                           \
        hipError_t _e = (expr);                                                    \
        if (_e != hipSuccess) {                                                    \
            tgt::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e),  \
                           __FILE__, __LINE__);                                    \
            return TGT_ERR_HIP;                                                    \
        }                                                                          \
    } while (0)

// One schedule entry: `len` consecutive edges starting at sorted position
// `start`, all belonging to node `row`.  part < 0: the item covers the whole row
// and its result is final; part >= 0: the row is split over several workgroups
// and this item's partial sums go to slot `part` of the workspace.
struct Item { int32_t row, start, len, part; };

// Code of a wave record: bits 0-2 kind, bit 3 the view in the backward launch (0 by destination, 1 by source),
// bits 8.. number of rows.
//   kind 0..4: wave items of that length class (count <= rows per wave of the shape)
//   kind 5:    a workgroup item (all four records of the workgroup are equal)
//   kind 7:    nothing
constexpr uint32_t kDescBlock = 5, kDescNone = 7, kDescSrcSide = 8;
__host__ __device__ constexpr uint32_t desc_code(uint32_t kind, uint32_t src_side, uint32_t count) {
    return kind | (src_side ? kDescSrcSide : 0u) | (count << 8);
}

// Edge slots of a lane group: natural slot count of the length classes (>32, <=32, <=16, <=8, <=4),
// capped by the wave (lpe = lanes that cover one edge).
__host__ __device__ constexpr int slots_for_class(int lpe, int cls) {
    const int nat = cls == 0 ? 16 : (cls == 1 ? 8 : (cls == 2 ? 4 : (cls == 3 ? 2 : 1)));
    const int cap = kWave / lpe;
    return nat < cap ? nat : cap;
}
__host__ __device__ constexpr int rows_per_wave(int lpe, int cls) { return kWave / (lpe * slots_for_class(lpe, cls)); }
// Whether the rows of a class fit one step of their slots (four edges per slot), so that a wave's record can
// carry their edges: every class but the longest, unless the wave is too narrow for the class's slots.
__host__ __device__ constexpr bool class_inline(int lpe, int cls) {
    return cls >= 1 && slots_for_class(lpe, cls) * 4 >= (cls == 1 ? 32 : (cls == 2 ? 16 : (cls == 3 ? 8 : 4)));
}

// What one wave of an attention workgroup reads first: its share of the launch, complete.  Workgroup b
// owns records 4b .. 4b+3.  `code` is a descriptor code (kind, view, number of rows).
//   kind 5: `item` is the workgroup item (all four records of the workgroup carry it);
//   kind 0: lane group g = (row i of the wave, slot s), g = i * S + s, S = slots_for_class, works on row row[g]
//   with edges [start[g], start[g] + len[g]) of the view's sorted arrays (the S groups of a row hold the same
//   three numbers; zeros behind the wave's last row);
//   kind 1..4: the same, and the edges inline: col / eid hold for lane group g the four edges s, s + S, s + 2S,
//   s + 3S of its row at [4g, 4g + 4) (an edge past the end of the row repeats the row's last edge; 0 for an
//   empty row).
// No address in a record depends on the kind: a lane asks for code, row, start, len and its four edges at once,
// and one memory round trip gives a wave everything it needs to issue its gathers.  (Kinds without inline edges
// leave col / eid unwritten; what a lane reads there is never used.)
template <int LPE>
struct alignas(128) WaveRec {
    static constexpr int kRows = kWave / LPE;          // most rows a wave can hold (shortest class)
    static constexpr int kEdges = 4 * kWave / LPE;     // four edges per lane group
    uint32_t code;
    int32_t pad[3];
    Item item;
    int32_t row[kRows], start[kRows], len[kRows];
    int32_t col[kEdges], eid[kEdges];
};
// the same layout for code that takes the shape at run time (the builder): offsets in int32 units
struct WaveRecLayout {
    int rows, edges, off_row, off_start, off_len, off_col, off_eid, stride;
    explicit WaveRecLayout(int lpe) {
        rows = kWave / lpe; edges = 4 * kWave / lpe;
        off_row = 8; off_start = off_row + rows; off_len = off_start + rows; off_col = off_len + rows;
        off_eid = off_col + edges;
        stride = (off_eid + edges + 31) / 32 * 32;
    }
};

// One sorted view of the edge list plus its row schedule.
struct Side {
    int32_t* rowptr = nullptr;   // [N+1]
    int32_t* col = nullptr;      // [E] other endpoint
    int32_t* eid = nullptr;      // [E] caller's edge id
    int32_t* pos = nullptr;      // [E] source side only, built on request: position of the edge in the destination-sorted order
    Item* items = nullptr;       // wave items (rows one wave walks) by (window, length class, row); room for N
    Item* block_items = nullptr; // [n_block_items] workgroup items: segments of the rows longer than a wave row
    int32_t* split_row = nullptr;   // [n_split] rows that were split
    int32_t* split_off = nullptr;   // [n_split+1] first partial slot of each split row
    int32_t* part2split = nullptr;  // [n_parts] index into split_row of the row a partial slot belongs to
    int32_t* split_grp = nullptr;   // [n_split+1] first combine group of each split row (a row with more than kCombineFan segments has ceil(segments / kCombineFan) groups)
    int32_t n_items = 0, n_split = 0, n_parts = 0, n_groups = 0;
    int32_t n_block_items = 0;      // workgroup items (n_items counts both kinds)
    // host copies the launch descriptors are made from
    int32_t n_windows = 0;
    std::vector<uint32_t> win_class_off;   // [n_windows * (kNumClass + 1)] wave items of (window, class) start here
    std::vector<uint32_t> win_class_cnt;   // same shape: how many
    std::vector<int32_t> block_home;       // [n_block_items] window the workgroup item is scheduled with
    std::vector<int32_t> block_len;        // [n_block_items] its edges
    std::vector<uint8_t> block_spread;     // [n_block_items] 1: segment of a row with more than kSpreadSegs segments
    std::vector<int32_t> homed_off, homed_idx;   // workgroup items by home window: items homed_idx[homed_off[w] .. homed_off[w+1])
};

// Wave records of one kernel shape (lanes per edge): forward (destination view) and backward
// (both views, window by window).
struct Schedule {
    void* fwd = nullptr;    // WaveRec<lpe> [4 * fwd_blocks]
    void* bwd = nullptr;
    int32_t fwd_blocks = 0, bwd_blocks = 0;
    bool ready = false;
};
constexpr int kNumLpe = 5;   // lanes per edge 1, 2, 4, 8, 16

// Device memory of the library's own (plans, tile sets, scratch of the edge preparation): from the
// allocator set with tgt_set_allocator, hipMalloc / hipFree without one.  `st` is the stream the memory
// is first used on (a caching allocator hands back memory that is safe to reuse on that stream).
hipError_t dev_alloc(void** p, size_t bytes, hipStream_t st);
void dev_free(void* p);

// Device buffer that frees itself.  Freed memory may still be read by kernels already launched on the
// stream it was allocated for: a stream-ordered allocator reuses it behind them, hipFree waits for them.
struct DevBuf {
    void* p = nullptr;
    DevBuf() = default;
    DevBuf(const DevBuf&) = delete;
    DevBuf& operator=(const DevBuf&) = delete;
    ~DevBuf();
    hipError_t alloc(size_t bytes, hipStream_t st = nullptr);
    template <typename T> T* as() const { return (T*)p; }
};

int bits_for(int64_t n);   // bits needed to hold values in [0, n)

// Stable LSD radix sort of (uint32 key, uint32 value) pairs (radix_sort.hip).
class RadixSorter {
public:
    int init(int64_t capacity, hipStream_t st = nullptr);
    // Sorts by the low `bits` bits of the keys.  vals_in == nullptr means values 0..n-1.
    // The results live in the sorter's buffers until the next sort() call; copy a
    // result before passing it as input of another sort().
    int sort(const uint32_t* keys_in, const uint32_t* vals_in, int64_t n, int bits, hipStream_t st,
             const uint32_t** keys_out, const uint32_t** vals_out);
private:
    DevBuf keysA_, keysB_, valsA_, valsB_, hist_, totals_;
    int64_t cap_ = 0;
    int nblocks_ = 0;
};

// nn.GELU() (exact erf form) and F.relu on one value, and dh * d act / du.  One definition for the elementwise kernels
// and for the epilogues of the projections that apply the activation themselves: both give the same bits.
//   GELU: h = 0.5 u (1 + erf(u / sqrt 2));  dh/du = 0.5 (1 + erf(u / sqrt 2)) + u exp(-u^2 / 2) / sqrt(2 pi)
//   RELU: h = max(u, 0);  dh/du = 1 where u > 0
template <bool RELU>
__device__ __forceinline__ float act_value(float u) {
    if (RELU) return u > 0.f ? u : 0.f;
    const float cdf = 0.5f * (1.f + erff(u * 0.70710678118654752f));
    return u * cdf;
}
template <bool RELU>
__device__ __forceinline__ float act_grad(float u, float dh) {
    if (RELU) return u > 0.f ? dh : 0.f;
    const float cdf = 0.5f * (1.f + erff(u * 0.70710678118654752f));
    return dh * (cdf + u * __expf(-0.5f * u * u) * 0.39894228040143268f);
}

// Kernel names of the optional per-kernel timing (timing.hip).
enum KernelSlot { KS_FWD = 0, KS_NODE_SIDE, KS_BWD, KS_DENSE_FWD, KS_DENSE_BWD, KS_TILE_FWD, KS_TILE_BWD, KS_LINEAR_FWD,
                  KS_LINEAR_DX, KS_LINEAR_DW, KS_LAYER_NORM_FWD, KS_LAYER_NORM_BWD, KS_GELU, KS_GRAPH_BIAS_FWD,
                  KS_GRAPH_BIAS_BWD, KS_LOSS, KS_COUNT };

// Scope guard: records a hipEvent on `st` before and after the launches made in
// its scope when timing is enabled; does nothing otherwise.
class KernelTimer {
public:
    // `on` false: times nothing (a caller that must not create events, which taking one from an empty pool does)
    KernelTimer(int slot, hipStream_t st, bool on = true);
    ~KernelTimer();
    KernelTimer(const KernelTimer&) = delete;
    KernelTimer& operator=(const KernelTimer&) = delete;
private:
    int slot_;
    hipStream_t st_;
    hipEvent_t start_;
};

// Sums of the dense tiles of the block path, added by the sparse kernels when they write a row.
struct TileInit {
    const float* acc;          // [N, H, d] sum w v
    const float* Z;            // [N, H]
    const float* dq;           // [N, H, d]
    const float* dk;           // [N, H, d]
    const float* dv;           // [N, H, d]
    const uint8_t* cover_dst;  // [N] 1 where the node is a destination of some tile
    const uint8_t* cover_src;  // [N] 1 where the node is a source of some tile
};

}  // namespace tgt

struct tgt_plan;
namespace tgt {
int sparse_attn_fwd_impl(const tgt_plan* plan, const void* d_q, const void* d_k, const void* d_v, const void* d_bias,
                         int bias_mode, int H, int d, int dtype, void* d_out, float* d_Z, void* d_workspace,
                         int64_t workspace_bytes, void* stream, const TileInit* init);
int sparse_attn_bwd_impl(const tgt_plan* plan, const void* d_q, const void* d_k, const void* d_v, const void* d_bias,
                         int bias_mode, int H, int d, int dtype, const void* d_out, const float* d_Z,
                         const void* d_dout, void* d_dq, void* d_dk, void* d_dv, void* d_dbias, void* d_workspace,
                         int64_t workspace_bytes, void* stream, const TileInit* init, bool skip_node_side);
// nd[i,h] = (1/(Z+eps), dout.out) into the head of the workspace (what the backward walks read)
int sparse_attn_node_side(const tgt_plan* plan, int H, int d, int dtype, const void* d_out, const float* d_Z,
                          const void* d_dout, void* d_workspace, void* stream);
const float2* sparse_attn_nd_ptr(void* d_workspace);
}  // namespace tgt

struct tgt_plan {
    int64_t N = 0, E = 0;
    int device = 0;
    // a plan of the edges that remain beside a tile set: rows without edges have no place in its schedules
    // (the tile kernels write them), so the sparse entry points on their own must refuse it
    bool rows_with_edges_only = false;
    tgt::Side dst;   // edges grouped by destination (query) node
    tgt::Side src;   // edges grouped by source (key/value) node
    tgt::Schedule sched[tgt::kNumLpe];   // by log2(lanes per edge); made on first use of a shape
    std::mutex sched_mutex;              // guards that first use
};
namespace tgt {
// Descriptors for kernels with `lpe` lanes per edge; builds them on first use (allocates, copies and
// synchronises `st` once per plan and shape).  nullptr on error.
const Schedule* plan_schedule(const tgt_plan* plan, int lpe, hipStream_t st);
// The same without building anything: nullptr if the shape has not been used or prepared yet.
const Schedule* plan_schedule_if_ready(const tgt_plan* plan, int lpe);
}
