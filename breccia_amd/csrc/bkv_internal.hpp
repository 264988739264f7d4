// Internal declarations shared by the translation units of libbreccia_kv.so.
#pragma once

#include <hip/hip_ext.h>
#include <hip/hip_runtime.h>

#include <cstdint>
#include <memory>
#include <string>
#include <vector>

#include "../../include/breccia_kv.h"
#include "allocator.hpp"
#include "attn_plan.hpp"
#include "prefix_tree.hpp"

namespace bkv {

// ---- error plumbing ---------------------------------------------------------
void set_error(const std::string& msg);
bkv_status fail(bkv_status st, const std::string& msg);
bkv_status hip_fail(hipError_t e, const char* what);

#define BKV_HIP(call)                                                 \
    do {                                                              \
        hipError_t e__ = (call);                                      \
        if (e__ != hipSuccess) return ::bkv::hip_fail(e__, #call);    \
    } while (0)

// work-groups the split-K partial-result workspace is sized for (x 8 head rows of 256 floats)
constexpr int32_t kMaxWgs = 4096;
// work-groups (x 8 head rows) the static device scratch of bkv_decode_attn_static is sized for
constexpr int32_t kStaticWgs = 1024;

// ---- geometry ----------------------------------------------------------------
struct Geom {
    int32_t n_layers, n_pages, n_kv, hd, page_cells, layout;
    // bytes of one (page, kv head, cell) row and of one whole page, per pool
    uint32_t k_row_bytes, v_row_bytes;
    uint64_t k_page_bytes, v_page_bytes;
    uint64_t k_pool_bytes, v_pool_bytes;  // one layer
};

// Pinned-host + device slot pairs for argument lists too long for kernel
// arguments (page-pair lists, block-table updates).  A slot is reused only after
// the event recorded behind its last consumer has completed.
struct ParamRing {
    static constexpr int kSlots = 32;
    static constexpr size_t kSlotBytes = 64 * 1024;
    uint8_t* host = nullptr;
    uint8_t* dev = nullptr;
    hipEvent_t ev[kSlots] = {};
    bool used[kSlots] = {};
    int next = 0;
};

// Event pairs around individual kernels while timing is enabled.
struct StageTimer {
    struct Pair {
        int stage;
        hipEvent_t start, stop;
    };
    bool on = false;
    std::vector<Pair> open;       // recorded, not yet read
    uint64_t launches[BKV_STAGE_COUNT] = {};
    double total_ms[BKV_STAGE_COUNT] = {};
};

struct SwapStage {
    static constexpr int kHalves = 2;
    uint8_t* dev[kHalves] = {nullptr, nullptr};
    uint64_t bytes = 0;             // per half
    hipEvent_t ev_stream[kHalves] = {};  // last use on a caller stream
    hipEvent_t ev_side[kHalves] = {};    // last use on the side stream
    int next = 0;
};

// Which stream used a pool-owned workspace last, and an event to order the next one behind it.
struct WorkspaceOrder {
    hipStream_t last = nullptr;
    bool used = false;
    hipEvent_t ev = nullptr;
};

// Where the prefix tree's lower tiers keep their pages: a pinned-host arena of slots and a file,
// slot = one page's bytes of every layer ([layer][K page | V page]).
struct TierStore {
    uint8_t* host = nullptr;    // host_slots slots (pinned; null on a host-only pool)
    int32_t host_slots = 0;
    int fd = -1;                // the file of the disk tier
    int32_t disk_slots = 0;
    uint8_t* bounce = nullptr;  // pinned, between the file and the device: two halves of
    int32_t bounce_slots = 0;   // bounce_slots slots each
    hipEvent_t done = nullptr;  // behind the last transfer enqueued on the side stream
    bool pending = false;       // `done` may not have completed yet
};

}  // namespace bkv

struct bkv_pool {
    bkv_pool_desc desc{};
    bkv::Geom g{};
    std::unique_ptr<bkv::PageAllocator> alloc;
    std::unique_ptr<bkv::PrefixTree> prefix;  // declared after alloc: destroyed first
    bool host_only = false;
    int device = 0;
    int n_cu = 0;

    uint8_t* slab = nullptr;  // every layer's K and V pool, one allocation
    std::vector<uint8_t*> k_layer, v_layer;
    int32_t* table_dev = nullptr;  // [max_seqs][max_pages_per_seq]

    // split-K workspace: partial (m, l) and O per work-group
    float* part_o = nullptr;
    float* part_ml = nullptr;
    int32_t max_wgs = 0;
    int32_t live_plans = 0;  // step plans made from this pool and not yet destroyed
    // block selection: f64 indexer scores [entry][block], grown on demand
    double* sel_scores = nullptr;
    uint64_t sel_scores_cap = 0;  // doubles

    // Streams that used the split-K workspace and the score workspace last: a call on another
    // stream is ordered behind them first (the workspaces are one per pool).
    bkv::WorkspaceOrder attn_ws, sel_ws;
    // the stream of the last block-table scatter, and the event behind it
    bkv::WorkspaceOrder table_sync;

    bkv::ParamRing ring;
    bkv::StageTimer timer;
    bkv::SwapStage stage;
    bkv::TierStore tiers;
    hipStream_t side = nullptr;
    hipEvent_t side_done = nullptr;
    bool side_used = false;
};

namespace bkv {

// Push pending block-table changes to the device arena on `stream`.
bkv_status flush_tables(bkv_pool* p, hipStream_t stream);
// Copy `bytes` of host data into a ring slot and enqueue its upload; returns the
// device address the consumer kernel reads.  `done(stream)` must be called after
// the consumer has been enqueued.
bkv_status ring_upload(bkv_pool* p, const void* host_src, size_t bytes, hipStream_t stream,
                       void** dev_out, int* slot_out);
bkv_status ring_done(bkv_pool* p, int slot, hipStream_t stream);

// While the pool's timer is on: an event pair registered for `stage` that the caller attaches to
// one dispatch (hipExtLaunchKernelGGL), which then reports the kernel's own duration, without
// the event records' own time on the queue.  False (and nothing registered) while it is off.
bool timer_dispatch_events(bkv_pool* p, int stage, hipEvent_t* start, hipEvent_t* stop);
bkv_status timer_collect(bkv_pool* p);

// One kernel launch of a timed stage: a plain launch, or, while the pool times its kernels, one
// that carries an event pair on the dispatch.
template <typename K, typename... Args>
inline void launch_staged(bkv_pool* p, int stage, K kernel, dim3 grid, dim3 block, uint32_t lds,
                          hipStream_t stream, Args... args) {
    hipEvent_t start = nullptr, stop = nullptr;
    if (timer_dispatch_events(p, stage, &start, &stop))
        hipExtLaunchKernelGGL(kernel, grid, block, lds, stream, start, stop, 0, args...);
    else
        hipLaunchKernelGGL(kernel, grid, block, lds, stream, args...);
}

// ---- kernel launchers (each validates nothing: callers have checked) ---------
struct AppendBatch {
    int32_t n;
    int32_t row[BKV_MAX_BATCH];      // block-table row of the sequence
    int32_t pos0[BKV_MAX_BATCH];     // first cell
    int32_t n_tok[BKV_MAX_BATCH];    // tokens of this sequence
    int32_t src0[BKV_MAX_BATCH];     // first source row in k/v
};
hipError_t launch_append(bkv_pool* p, int32_t layer, const AppendBatch& b, int32_t max_tok,
                         const void* k, const void* v, bool src_is_f16, hipStream_t stream);

hipError_t launch_append_kprep(bkv_pool* p, int32_t layer, const AppendBatch& b, int32_t max_tok,
                               const float* k, const float* v, const float* gamma, float eps,
                               const float* table, int32_t n_rot, int32_t max_pos,
                               const int32_t* positions, hipStream_t stream);

// Block selection (select.hip): one entry per (token) list.
struct SelectBatch {
    int32_t n;
    int32_t pos[BKV_MAX_BATCH];       // query position
    int32_t n_blocks[BKV_MAX_BATCH];  // pooled / scored blocks of the entry
    const float* pooled[BKV_MAX_BATCH];  // [n_blocks][idx_dim] (score kernel only)
};
hipError_t launch_idx_score(bkv_pool* p, const SelectBatch& b, const float* q, int32_t idx_n_head, int32_t idx_dim,
                            int32_t idx_block, double* scores, int64_t score_stride, int32_t max_blocks,
                            hipStream_t stream);
hipError_t launch_topk_blocks(bkv_pool* p, const SelectBatch& b, const void* scores, bool scores_f64,
                              int64_t score_stride, int32_t topk_blocks, int32_t idx_block, bool dense,
                              uint32_t* ids, int64_t id_stride, uint32_t* counts, int32_t max_ids,
                              hipStream_t stream);
hipError_t launch_idx_pool(bkv_pool* p, const float* raw, float* tail, const float* gamma, const float* table,
                           float* pooled, int32_t pos0, int32_t tokens, int32_t idx_dim, int32_t idx_block,
                           int32_t n_rot, int32_t max_pos, float eps, hipStream_t stream);
int32_t select_max_topk();
int32_t select_max_idx_head();
int32_t select_max_idx_dim();

struct AttnArgs {
    int32_t n_q_head;
    const float* q;
    const float* gate;
    int64_t gate_seq_stride, gate_head_stride;
    float scale;
    float* out;
    // selection lists; ids == nullptr means the dense selection (every cell 0..=pos)
    const uint32_t* ids = nullptr;
    const uint32_t* counts = nullptr;
    int64_t id_stride = 0;
    int32_t max_ids = 0;
    // fused decode step: new rows [n][n_kv][head_dim] f32; nullptr = plain attention
    const float* new_k = nullptr;
    const float* new_v = nullptr;
    // partial-result workspace other than the pool's own (the static device scratch); nullptr = the pool's
    float* ws_o = nullptr;
    float* ws_ml = nullptr;
    bool timed = true;  // kernels carry stage-timer events while the pool's timer is on
    // the batch lives in a device-resident descriptor (a step plan): the kernels read it there and the
    // split-K launch has this fixed grid
    const AttnBatch* desc = nullptr;
    int32_t desc_grid = 0;
};

// Device-resident state of a step plan (bkv_step_plan_*): the batch as the kernels read it, the last
// cell each entry was checked for, and what the advances did.
struct StepDesc {
    AttnBatch b;
    int32_t horizon[kMaxBatch];
    int32_t status;  // 0, or 1 once an advance was refused at the horizon
    uint32_t steps;  // advances done
};
hipError_t launch_step_advance(StepDesc* d, const AttnPlanLimits& lim, int32_t page_cells, hipStream_t stream);
// Fills wg_base/splits/pps from row/pos (attn_plan.hpp); returns the total work-group count, -1
// when the batch cannot be cut into as few work-groups as the workspace holds.  sel_groups > 0:
// every entry is planned for that many groups of four selected blocks instead of its pages.
AttnPlanLimits attn_plan_limits(int32_t n_cu, int32_t max_wgs, int32_t n_kv, int32_t group);
int32_t plan_attn(const bkv_pool* p, int32_t n_q_head, AttnBatch& b, int32_t sel_groups = 0, int32_t max_wgs = 0);
// The static device scratch of bkv_decode_attn_static: looked up once per device (which must be
// the current one) at pool creation; false from the accessor when that has not happened.
hipError_t attn_static_scratch_init(int device);
bool attn_static_scratch(int device, float** o, float** ml);
hipError_t launch_decode_attn(bkv_pool* p, int32_t layer, const AttnBatch& b, const AttnArgs& a,
                              hipStream_t stream);
// Prefill attention (prefill_attn.hip): one entry per sequence chunk.
struct PrefillBatch {
    int32_t n;
    int32_t row[BKV_MAX_BATCH];     // block-table row
    int32_t pos0[BKV_MAX_BATCH];    // position of the chunk's first token
    int32_t n_tok[BKV_MAX_BATCH];   // tokens of the chunk
    int32_t src0[BKV_MAX_BATCH];    // first token row in q / out
    int32_t wg_base[BKV_MAX_BATCH + 1];
};
// query rows one work-group owns, given how many 64-row work-groups the call's chunks would make
int32_t prefill_rows_per_wg(int32_t layout, int64_t wgs_of_64_rows, int32_t n_cu);
hipError_t launch_prefill_attn(bkv_pool* p, int32_t layer, const PrefillBatch& b, const AttnArgs& a,
                               int32_t rows_per_wg, hipStream_t stream);

hipError_t launch_page_copy(bkv_pool* p, const bkv_page_pair* pairs_dev, int32_t n_pairs,
                            hipStream_t stream);
// Gather (to_stage=1) / scatter (to_stage=0) whole pages between the pools and a
// contiguous staging buffer laid out [page][layer][K bytes | V bytes].
hipError_t launch_page_stage(bkv_pool* p, const int32_t* pages_dev, int32_t n_pages,
                             uint8_t* stage, int to_stage, hipStream_t stream);
hipError_t launch_gather(const bkv_pool* p, int32_t layer, int32_t row, int64_t cell0, int64_t n,
                         float* k_out, float* v_out, hipStream_t stream);
hipError_t launch_table_scatter(int32_t* table, const TableUpdate* upd_dev, int32_t n,
                                hipStream_t stream);
// up to kTableUpdatesInArgs updates, given on the host, as arguments of one small launch
constexpr int32_t kTableUpdatesInArgs = 32;
hipError_t launch_table_scatter_args(int32_t* table, const TableUpdate* upd_host, int32_t n, hipStream_t stream);
hipError_t launch_fill(void* dst, uint64_t bytes, uint32_t word, hipStream_t stream);

}  // namespace bkv
