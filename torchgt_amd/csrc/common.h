// Shared host-side declarations of the gfx950 sparse-attention library.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include "../../include/torchgt_hip.h"

namespace tgt {

constexpr int kWave = 64;            // CDNA wavefront width
constexpr int kBlock = 256;          // threads per workgroup of the attention kernels (4 waves)
constexpr int kSegLen = 256;         // a row longer than this is split into segments of this many edges
constexpr int kNumClass = 5;         // item length classes: >32, <=32, <=16, <=8, <=4

void set_error(const char* fmt, ...);

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
// and its result is final; part >= 0: the row is split and this item's partial
// sums go to slot `part` of the workspace.
struct Item { int32_t row, start, len, part; };

// One sorted view of the edge list plus its row schedule.
struct Side {
    int32_t* rowptr = nullptr;   // [N+1]
    int32_t* col = nullptr;      // [E] other endpoint
    int32_t* eid = nullptr;      // [E] caller's edge id
    Item* items = nullptr;       // [n_items], ordered by length class, longest class first
    int32_t* split_row = nullptr;   // [n_split] rows that were split
    int32_t* split_off = nullptr;   // [n_split+1] first partial slot of each split row
    int32_t n_items = 0, n_split = 0, n_parts = 0;
    int32_t class_off[kNumClass + 1] = {0, 0, 0, 0, 0, 0};   // item index where each class begins
};

}  // namespace tgt

struct tgt_plan {
    int64_t N = 0, E = 0;
    int device = 0;
    tgt::Side dst;   // edges grouped by destination (query) node
    tgt::Side src;   // edges grouped by source (key/value) node
};
