// Work planning of the split-K decode attention kernels: how a batch of (sequence, position)
// entries is cut into page ranges, one work-group each.  No HIP types: the same function runs
// on the host (every call), in host-only tests and on the device (a decode step replayed from
// a graph re-plans itself there), and has to give the same cut everywhere -- the order in
// which partial results are summed, and with it the last bits of the output, follows the cut.
#pragma once

#include <cstdint>

#if defined(__HIPCC__)
#define BKV_HD __host__ __device__
#else
#define BKV_HD
#endif

namespace bkv {

constexpr int kMaxBatch = 64;  // BKV_MAX_BATCH

struct AttnBatch {
    int32_t n;
    int32_t row[kMaxBatch];          // block-table row
    int32_t pos[kMaxBatch];          // last visible cell
    int32_t wg_base[kMaxBatch + 1];  // first work-group of the entry; [n] = total
    int32_t splits[kMaxBatch];       // page ranges the entry is cut into
    int32_t pps[kMaxBatch];          // pages per split
};

// What bounds a plan.  `per_page` work-groups serve one page range of one entry (kv heads x
// head chunks); `gran` pages are walked side by side by the waves of a work-group, so ranges
// are whole multiples of it; `target` is the number of work-groups that are resident at once
// (one generation: left-over work-groups would run alone after the rest); `max_wgs` is what
// the partial-result workspace holds.
struct AttnPlanLimits {
    int32_t per_page;
    int32_t gran;
    int32_t target;
    int32_t max_wgs;
};

// Fills wg_base / splits / pps of b from pos (sel_groups > 0: every entry is planned for that
// many groups of four selected blocks instead of its pages).  Returns the total work-group
// count, or -1 when even one range per entry exceeds max_wgs (the caller reports it; nothing
// may be launched).  A batch whose smallest cut exceeds `target` is planned with one range per
// entry and runs in more than one generation.  Terminates for every input: the range length
// grows until every entry is a single range, and that cut is accepted.
BKV_HD inline int32_t plan_attn_ranges(const AttnPlanLimits& lim, int32_t page_cells, int32_t sel_groups,
                                       AttnBatch& b) {
    const int64_t per_page = lim.per_page;
    const int64_t gran = lim.gran;
    const int64_t min_total = (int64_t)b.n * per_page;
    if (min_total > lim.max_wgs) return -1;
    int64_t target = lim.target < lim.max_wgs ? lim.target : lim.max_wgs;
    if (target < min_total) target = min_total;
    int64_t total_pages = 0, max_pages = 0;
    for (int i = 0; i < b.n; ++i) {
        const int64_t it = sel_groups > 0 ? sel_groups : b.pos[i] / page_cells + 1;
        total_pages += it;
        if (it > max_pages) max_pages = it;
    }
    int64_t pps = (total_pages * per_page + target - 1) / target;
    pps = (pps + gran - 1) / gran * gran;
    if (pps < gran) pps = gran;
    for (;;) {
        int64_t total = 0;
        for (int i = 0; i < b.n; ++i) {
            const int64_t pages = sel_groups > 0 ? sel_groups : b.pos[i] / page_cells + 1;
            const int64_t splits = (pages + pps - 1) / pps;
            // even the ranges out inside the entry, keeping whole groups of `gran` pages
            int64_t each = (pages + splits - 1) / splits;
            each = (each + gran - 1) / gran * gran;
            b.splits[i] = (int32_t)((pages + each - 1) / each);
            b.pps[i] = (int32_t)each;
            b.wg_base[i] = (int32_t)total;
            total += (int64_t)b.splits[i] * per_page;
        }
        b.wg_base[b.n] = (int32_t)total;
        // pps >= max_pages: one range per entry, total == min_total <= target
        if (total <= target || pps >= max_pages) return (int32_t)total;
        pps += gran;
    }
}

}  // namespace bkv
