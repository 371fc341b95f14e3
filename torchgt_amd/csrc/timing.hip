// Optional per-kernel timing with HIP events on the launch stream.
//
// The reference measures this path with torch.profiler around whole iterations
// (attn_module.py:415-438).  Here every kernel launch of the library can be
// bracketed by a pair of hipEvents recorded on the stream the kernel runs on, so
// a benchmark can report the duration of one named kernel.  Off by default; when
// off, launches are not touched.
#include "common.h"
#include <mutex>
#include <vector>

namespace tgt {

static const char* kSlotNames[KS_COUNT] = {
    "attn_fwd", "bwd_node_side", "attn_bwd", "dense_fwd", "dense_bwd", "tile_fwd", "tile_bwd",
    "linear_fwd", "linear_dx", "linear_dw", "layer_norm_fwd", "layer_norm_bwd", "gelu",
    "graph_bias_fwd", "graph_bias_bwd", "nll_loss",
};

struct Pending { hipEvent_t start, stop; int slot; };

static std::mutex g_mu;
static bool g_enabled = false;
static std::vector<Pending> g_pending;
static std::vector<hipEvent_t> g_free;
static double g_ms[KS_COUNT] = {0};
static int64_t g_count[KS_COUNT] = {0};

static hipEvent_t take_event() {
    if (!g_free.empty()) {
        hipEvent_t e = g_free.back();
        g_free.pop_back();
        return e;
    }
    hipEvent_t e = nullptr;
    (void)hipEventCreate(&e);
    return e;
}

bool timing_enabled() { return g_enabled; }

KernelTimer::KernelTimer(int slot, hipStream_t st, bool on) : slot_(slot), st_(st), start_(nullptr) {
    if (!g_enabled || !on) return;
    std::lock_guard<std::mutex> lk(g_mu);
    start_ = take_event();
    if (start_) (void)hipEventRecord(start_, st_);
}

KernelTimer::~KernelTimer() {
    if (!start_) return;
    std::lock_guard<std::mutex> lk(g_mu);
    hipEvent_t stop = take_event();
    if (stop) (void)hipEventRecord(stop, st_);
    g_pending.push_back(Pending{start_, stop, slot_});
}

// waits for every recorded pair and folds it into the per-slot totals
static void drain() {
    for (const Pending& p : g_pending) {
        if (p.start && p.stop && hipEventSynchronize(p.stop) == hipSuccess) {
            float ms = 0.f;
            if (hipEventElapsedTime(&ms, p.start, p.stop) == hipSuccess) {
                g_ms[p.slot] += ms;
                g_count[p.slot] += 1;
            }
        }
        if (p.start) g_free.push_back(p.start);
        if (p.stop) g_free.push_back(p.stop);
    }
    g_pending.clear();
}

}  // namespace tgt

extern "C" {

int tgt_timing_enable(int on) {
    std::lock_guard<std::mutex> lk(tgt::g_mu);
    tgt::g_enabled = on != 0;
    return TGT_OK;
}

int tgt_timing_reset(void) {
    std::lock_guard<std::mutex> lk(tgt::g_mu);
    tgt::drain();
    for (int i = 0; i < tgt::KS_COUNT; ++i) { tgt::g_ms[i] = 0; tgt::g_count[i] = 0; }
    return TGT_OK;
}

int tgt_timing_slots(void) { return tgt::KS_COUNT; }

int tgt_timing_read(int slot, const char** name, double* total_ms, int64_t* launches) {
    if (slot < 0 || slot >= tgt::KS_COUNT) return TGT_ERR_INVALID_ARG;
    std::lock_guard<std::mutex> lk(tgt::g_mu);
    tgt::drain();
    if (name) *name = tgt::kSlotNames[slot];
    if (total_ms) *total_ms = tgt::g_ms[slot];
    if (launches) *launches = tgt::g_count[slot];
    return TGT_OK;
}

}  // extern "C"
