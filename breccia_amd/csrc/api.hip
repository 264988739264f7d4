// C ABI of libbreccia_kv.so: argument checking, the pool object, block-table
// mirroring, and the launches.  Every range violation is reported here, on the host,
// before anything reaches the GPU (the reference's contract, crates/breccia-kernels/
// src/qsa/mod.rs:1108-1116).
#include <algorithm>
#include <atomic>
#include <chrono>
#include <cstdio>
#include <cstring>
#include <new>
#include <thread>
#include <unordered_map>

#include <cerrno>
#include <cmath>

#include <fcntl.h>
#include <sys/uio.h>
#include <unistd.h>

#include "bkv_internal.hpp"

namespace bkv {

static thread_local std::string g_last_error;

void set_error(const std::string& msg) { g_last_error = msg; }

bkv_status fail(bkv_status st, const std::string& msg) {
    g_last_error = msg;
    return st;
}

bkv_status hip_fail(hipError_t e, const char* what) {
    g_last_error = std::string(what) + " failed: " + hipGetErrorString(e);
    (void)hipGetLastError();
    return BKV_ERR_HIP;
}

static std::string sfmt(const char* f, long long a = 0, long long b = 0, long long c = 0,
                        long long d = 0) {
    char buf[320];
    std::snprintf(buf, sizeof buf, f, a, b, c, d);
    return buf;
}

static bkv_status from_alloc(AllocErr e, const std::string& msg) {
    switch (e) {
        case AllocErr::Ok: return BKV_OK;
        case AllocErr::Invalid: return fail(BKV_ERR_INVALID, msg);
        case AllocErr::Range: return fail(BKV_ERR_RANGE, msg);
        case AllocErr::NoPages: return fail(BKV_ERR_NO_PAGES, msg);
        default: return fail(BKV_ERR_STATE, msg);
    }
}

static inline hipStream_t S(void* s) { return reinterpret_cast<hipStream_t>(s); }

// ---- bounded host waits ---------------------------------------------------------------
// The reference never waits on its device without a deadline (crates/breccia-vk/src/ctx.rs:
// 1545-1553: WAIT_TIMEOUT_NS = 10 s, then a diagnostic instead of a hang).  Every host-side wait
// of this library -- for a stream, for an event -- polls the HIP query call up to a deadline and
// returns BKV_ERR_TIMEOUT with what it was waiting for; nothing is aborted, the work stays
// enqueued and a later wait can succeed.  The first `poll_us` microseconds of a wait spin on the
// query (a thread that sleeps in hipStreamSynchronize is woken some tens of microseconds after the
// stream has drained, which a decode loop that waits per token would pay every time); after that
// the thread naps 50 us between queries.  Process-wide settings (bkv_wait_options).
static std::atomic<int64_t> g_wait_timeout_ms{10000};
static std::atomic<int64_t> g_wait_poll_us{4000};

template <typename Query>
static bkv_status bounded_wait(Query query, int64_t timeout_ms, const char* call, const std::string& what) {
    const auto t0 = std::chrono::steady_clock::now();
    const auto spin = std::chrono::microseconds(g_wait_poll_us.load(std::memory_order_relaxed));
    for (;;) {
        const hipError_t e = query();
        if (e == hipSuccess) return BKV_OK;
        if (e != hipErrorNotReady) return hip_fail(e, call);
        (void)hipGetLastError();
        const auto waited = std::chrono::steady_clock::now() - t0;
        if (timeout_ms >= 0 && waited >= std::chrono::milliseconds(timeout_ms))
            return fail(BKV_ERR_TIMEOUT, sfmt("timed out after %lld ms waiting for ", timeout_ms) + what +
                                             ": the work is still enqueued, nothing was cancelled");
        if (waited < spin)
            __builtin_ia32_pause();
        else
            std::this_thread::sleep_for(std::chrono::microseconds(50));
    }
}
static bkv_status wait_stream(hipStream_t stream, int64_t timeout_ms, const std::string& what) {
    return bounded_wait([&] { return hipStreamQuery(stream); }, timeout_ms, "hipStreamQuery", what);
}
static bkv_status wait_event(hipEvent_t ev, const std::string& what) {
    return bounded_wait([&] { return hipEventQuery(ev); }, g_wait_timeout_ms.load(std::memory_order_relaxed),
                        "hipEventQuery", what);
}
static int64_t default_timeout_ms() { return g_wait_timeout_ms.load(std::memory_order_relaxed); }

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---- parameter ring ---------------------------------------------------------------
bkv_status ring_upload(bkv_pool* p, const void* host_src, size_t bytes, hipStream_t stream,
                       void** dev_out, int* slot_out) {
    ParamRing& r = p->ring;
    if (bytes > ParamRing::kSlotBytes)
        return fail(BKV_ERR_INVALID, "internal: parameter list larger than a ring slot");
    const int slot = r.next;
    r.next = (r.next + 1) % ParamRing::kSlots;
    if (r.used[slot]) {
        const bkv_status ws = wait_event(r.ev[slot], "the last reader of an argument-ring slot");
        if (ws != BKV_OK) return ws;
    }
    uint8_t* h = r.host + (size_t)slot * ParamRing::kSlotBytes;
    uint8_t* d = r.dev + (size_t)slot * ParamRing::kSlotBytes;
    std::memcpy(h, host_src, bytes);
    BKV_HIP(hipMemcpyAsync(d, h, bytes, hipMemcpyHostToDevice, stream));
    *dev_out = d;
    *slot_out = slot;
    return BKV_OK;
}

bkv_status ring_done(bkv_pool* p, int slot, hipStream_t stream) {
    BKV_HIP(hipEventRecord(p->ring.ev[slot], stream));
    p->ring.used[slot] = true;
    return BKV_OK;
}

// Pages on their way between the prefix tree's tiers: work enqueued on `stream` from here on may
// touch the device pages they leave or land on, so it waits for the transfers (until they are
// known to be over).
static bkv_status wait_for_tier_moves(bkv_pool* p, hipStream_t stream) {
    if (!p->tiers.pending) return BKV_OK;
    if (hipEventQuery(p->tiers.done) == hipSuccess)
        p->tiers.pending = false;
    else
        BKV_HIP(hipStreamWaitEvent(stream, p->tiers.done, 0));
    return BKV_OK;
}

// A pool has one split-K workspace and one score workspace.  Calls on one stream use them in turn
// by themselves; a call that arrives on another stream than the last one is ordered behind it
// with an event recorded there now (behind everything that stream has been given).
static bkv_status order_workspace(WorkspaceOrder& w, hipStream_t stream) {
    if (w.used && w.last != stream) {
        if (!w.ev) BKV_HIP(hipEventCreateWithFlags(&w.ev, hipEventDisableTiming));
        if (hipEventRecord(w.ev, w.last) == hipSuccess) {
            BKV_HIP(hipStreamWaitEvent(stream, w.ev, 0));
        } else {
            // the stream is gone: whatever it was given is ordered by a full synchronisation
            (void)hipGetLastError();
            BKV_HIP(hipDeviceSynchronize());
        }
    }
    w.last = stream;
    w.used = true;
    return BKV_OK;
}

// Block-table updates are scattered on whichever stream brings the next call.  A call on another
// stream reads the same table: it waits for the last scatter (until that is known to be over).
// `may_query` false: only the wait is enqueued, no host-side look at the event (for streams that
// may be under capture).
static bkv_status wait_for_table_scatter(bkv_pool* p, hipStream_t stream, bool may_query) {
    if (!p->table_sync.used || p->table_sync.last == stream) return BKV_OK;
    if (may_query && hipEventQuery(p->table_sync.ev) == hipSuccess) {
        p->table_sync.used = false;
        return BKV_OK;
    }
    (void)hipGetLastError();
    BKV_HIP(hipStreamWaitEvent(stream, p->table_sync.ev, 0));
    return BKV_OK;
}

bkv_status flush_tables(bkv_pool* p, hipStream_t stream) {
    bkv_status tier_st = wait_for_tier_moves(p, stream);
    if (tier_st != BKV_OK) return tier_st;
    const bkv_status ts = wait_for_table_scatter(p, stream, true);
    if (ts != BKV_OK) return ts;
    std::vector<TableUpdate>& pend = p->alloc->pending();
    if (pend.empty()) return BKV_OK;
    if (p->host_only) {
        pend.clear();
        return BKV_OK;
    }
    // Keep the last value per offset: one launch applies updates in no fixed order.
    std::unordered_map<int32_t, int32_t> last;
    last.reserve(pend.size() * 2);
    for (const TableUpdate& u : pend) last[u.offset] = u.value;
    std::vector<TableUpdate> flat;
    flat.reserve(last.size());
    for (const auto& kv : last) flat.push_back(TableUpdate{kv.first, kv.second});
    const size_t per_slot = ParamRing::kSlotBytes / sizeof(TableUpdate);
    if (flat.size() <= (size_t)kTableUpdatesInArgs) {
        // the usual case of a decode loop (a sequence or two opened a page): the updates ride in the
        // arguments of the scatter launch, no upload
        BKV_HIP(launch_table_scatter_args(p->table_dev, flat.data(), (int32_t)flat.size(), stream));
        flat.clear();
    }
    for (size_t at = 0; at < flat.size(); at += per_slot) {
        const size_t n = std::min(per_slot, flat.size() - at);
        void* dev;
        int slot;
        bkv_status st = ring_upload(p, flat.data() + at, n * sizeof(TableUpdate), stream, &dev, &slot);
        if (st != BKV_OK) return st;
        BKV_HIP(launch_table_scatter(p->table_dev, static_cast<const TableUpdate*>(dev), (int32_t)n,
                                     stream));
        st = ring_done(p, slot, stream);
        if (st != BKV_OK) return st;
    }
    pend.clear();
    if (!p->table_sync.ev) BKV_HIP(hipEventCreateWithFlags(&p->table_sync.ev, hipEventDisableTiming));
    BKV_HIP(hipEventRecord(p->table_sync.ev, stream));
    p->table_sync.last = stream;
    p->table_sync.used = true;
    return BKV_OK;
}

static hipEvent_t timer_take_event() {
    hipEvent_t e = nullptr;
    if (hipEventCreate(&e) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    return e;
}

bool timer_dispatch_events(bkv_pool* p, int stage, hipEvent_t* start, hipEvent_t* stop) {
    StageTimer& t = p->timer;
    if (!t.on) return false;
    *start = timer_take_event();
    *stop = timer_take_event();
    if (!*start || !*stop) {
        if (*start) (void)hipEventDestroy(*start);
        if (*stop) (void)hipEventDestroy(*stop);
        return false;
    }
    // every timed launch comes through here: a caller that never reads the timer (bkv_timing_read)
    // must not grow the list of open event pairs without bound
    if (t.open.size() >= 8192) (void)timer_collect(p);
    t.open.push_back(StageTimer::Pair{stage, *start, *stop});
    return true;
}

bkv_status timer_collect(bkv_pool* p) {
    StageTimer& t = p->timer;
    hipError_t err = hipSuccess;
    bool timed_out = false;  // the event pairs are dropped either way; the error text is wait_event's
    for (const StageTimer::Pair& pr : t.open) {
        float ms = 0.0f;
        if (err == hipSuccess && !timed_out) timed_out = wait_event(pr.stop, "a timed kernel") != BKV_OK;
        if (err == hipSuccess && !timed_out) err = hipEventElapsedTime(&ms, pr.start, pr.stop);
        if (err == hipSuccess && !timed_out) {
            t.launches[pr.stage] += 1;
            t.total_ms[pr.stage] += (double)ms;
        }
        // Events are not kept for reuse.  A recorded event holds on to its dispatch, and with it, as
        // measured, to the buffers the dispatch was given: with a pool of idle events, buffers that the
        // caller had freed since were only unmapped when those events were recorded again, and the
        // kernels running at that moment (a 1 GiB page copy) took 20 % longer.
        (void)hipEventDestroy(pr.start);
        (void)hipEventDestroy(pr.stop);
    }
    t.open.clear();
    if (timed_out) return BKV_ERR_TIMEOUT;
    BKV_HIP(err);
    return BKV_OK;
}

static bkv_status need_device(const bkv_pool* p) {
    if (!p) return fail(BKV_ERR_INVALID, "pool is NULL");
    if (p->host_only)
        return fail(BKV_ERR_NO_DEVICE, "this pool was created host-only: it has no device memory");
    return BKV_OK;
}

static void destroy_device_side(bkv_pool* p) {
    if (p->tiers.fd >= 0) (void)::close(p->tiers.fd);
    p->tiers.fd = -1;
    if (p->host_only) return;
    (void)hipDeviceSynchronize();
    if (p->tiers.host) (void)hipHostFree(p->tiers.host);
    if (p->tiers.bounce) (void)hipHostFree(p->tiers.bounce);
    if (p->tiers.done) (void)hipEventDestroy(p->tiers.done);
    if (p->attn_ws.ev) (void)hipEventDestroy(p->attn_ws.ev);
    if (p->sel_ws.ev) (void)hipEventDestroy(p->sel_ws.ev);
    if (p->table_sync.ev) (void)hipEventDestroy(p->table_sync.ev);
    if (p->slab) (void)hipFree(p->slab);
    if (p->table_dev) (void)hipFree(p->table_dev);
    if (p->part_o) (void)hipFree(p->part_o);
    if (p->part_ml) (void)hipFree(p->part_ml);
    if (p->sel_scores) (void)hipFree(p->sel_scores);
    if (p->ring.host) (void)hipHostFree(p->ring.host);
    if (p->ring.dev) (void)hipFree(p->ring.dev);
    for (int i = 0; i < ParamRing::kSlots; ++i)
        if (p->ring.ev[i]) (void)hipEventDestroy(p->ring.ev[i]);
    for (int i = 0; i < SwapStage::kHalves; ++i) {
        if (p->stage.dev[i]) (void)hipFree(p->stage.dev[i]);
        if (p->stage.ev_stream[i]) (void)hipEventDestroy(p->stage.ev_stream[i]);
        if (p->stage.ev_side[i]) (void)hipEventDestroy(p->stage.ev_side[i]);
    }
    if (p->side_done) (void)hipEventDestroy(p->side_done);
    if (p->side) (void)hipStreamDestroy(p->side);
    for (const StageTimer::Pair& pr : p->timer.open) {
        (void)hipEventDestroy(pr.start);
        (void)hipEventDestroy(pr.stop);
    }
}

}  // namespace bkv

using namespace bkv;

extern "C" {

const char* bkv_last_error(void) { return g_last_error.c_str(); }
const char* bkv_version(void) { return "breccia-kv 0.1 (gfx950)"; }

bkv_status bkv_pool_create(const bkv_pool_desc* d, bkv_pool** out) {
    if (!d || !out) return fail(BKV_ERR_INVALID, "pool_create: NULL argument");
    *out = nullptr;
    if (d->n_layers <= 0 || d->n_pages <= 0 || d->n_kv_head <= 0 || d->max_seqs <= 0 ||
        d->max_pages_per_seq <= 0)
        return fail(BKV_ERR_INVALID,
                    "pool_create: n_layers, n_pages, n_kv_head, max_seqs and max_pages_per_seq "
                    "must all be > 0 (a cache needs capacity > 0)");
    if (d->n_kv_head > BKV_MAX_KV_HEAD)
        return fail(BKV_ERR_INVALID, sfmt("pool_create: %lld kv heads; the kernels are built and tested for "
                                          "at most %lld", d->n_kv_head, BKV_MAX_KV_HEAD));
    if (d->head_dim <= 0 || d->head_dim % 32 != 0 || d->head_dim > 256)
        return fail(BKV_ERR_INVALID, sfmt("pool_create: head_dim %lld must be a multiple of 32 "
                                          "(the q8 block) and at most 256", d->head_dim));
    if (d->page_cells != 16)
        return fail(BKV_ERR_INVALID, sfmt("pool_create: page_cells %lld; pages are 16 cells",
                                          d->page_cells));
    if (d->layout < BKV_LAYOUT_F16 || d->layout > BKV_LAYOUT_I8H)
        return fail(BKV_ERR_INVALID, sfmt("pool_create: unknown layout %lld", d->layout));
    if (d->layout == BKV_LAYOUT_I8H && d->head_dim != 256)
        return fail(BKV_ERR_INVALID, "pool_create: the int8 + f16-scale layout is built for "
                                     "head_dim 256 (272-byte rows keep 16-byte alignment)");
    if ((int64_t)d->n_pages * d->page_cells >= (int64_t)1 << 31)
        return fail(BKV_ERR_INVALID, "pool_create: n_pages * page_cells must stay below 2^31");

    bkv_pool* p = new (std::nothrow) bkv_pool();
    if (!p) return fail(BKV_ERR_NOMEM, "pool_create: out of host memory");
    p->desc = *d;
    p->host_only = (d->flags & BKV_POOL_HOST_ONLY) != 0;
    p->max_wgs = kMaxWgs;
    Geom& g = p->g;
    g.n_layers = d->n_layers, g.n_pages = d->n_pages, g.n_kv = d->n_kv_head, g.hd = d->head_dim;
    g.page_cells = d->page_cells, g.layout = d->layout;
    const uint32_t f16_row = (uint32_t)d->head_dim * 2u;
    const uint32_t q8v_row = (uint32_t)(d->head_dim / 32) * 36u;
    const uint32_t i8h_row = (uint32_t)d->head_dim + (uint32_t)(d->head_dim / 32) * 2u;
    g.k_row_bytes = d->layout == BKV_LAYOUT_I8H ? i8h_row : f16_row;
    g.v_row_bytes = d->layout == BKV_LAYOUT_F16 ? f16_row
                    : d->layout == BKV_LAYOUT_Q8V ? q8v_row : i8h_row;
    const uint64_t rows_per_page = (uint64_t)d->n_kv_head * (uint64_t)d->page_cells;
    g.k_page_bytes = rows_per_page * g.k_row_bytes;
    g.v_page_bytes = rows_per_page * g.v_row_bytes;
    g.k_pool_bytes = g.k_page_bytes * (uint64_t)d->n_pages;
    g.v_pool_bytes = g.v_page_bytes * (uint64_t)d->n_pages;
    try {
        p->alloc.reset(new PageAllocator(d->n_pages, d->page_cells, d->max_seqs,
                                         d->max_pages_per_seq));
        p->prefix.reset(new PrefixTree(p->alloc.get(), d->page_cells));
    } catch (const std::bad_alloc&) {
        delete p;
        return fail(BKV_ERR_NOMEM, "pool_create: out of host memory for the block tables");
    }
    if (p->host_only) {
        *out = p;
        return BKV_OK;
    }

    auto bail = [&](bkv_status st) {
        const std::string keep = g_last_error;
        destroy_device_side(p);
        delete p;
        g_last_error = keep;
        return st;
    };
#define BKV_TRY(call)                                                        \
    do {                                                                     \
        hipError_t e__ = (call);                                             \
        if (e__ != hipSuccess) return bail(hip_fail(e__, #call));            \
    } while (0)

    int n_dev = 0;
    if (hipGetDeviceCount(&n_dev) != hipSuccess || n_dev <= 0) {
        (void)hipGetLastError();
        p->host_only = true;  // nothing device-side to tear down
        delete p;
        return fail(BKV_ERR_NO_DEVICE, "pool_create: no HIP device is visible");
    }
    BKV_TRY(hipGetDevice(&p->device));
    hipDeviceProp_t prop;
    BKV_TRY(hipGetDeviceProperties(&prop, p->device));
    p->n_cu = prop.multiProcessorCount;

    const uint64_t layer_bytes = g.k_pool_bytes + g.v_pool_bytes;
    BKV_TRY(hipMalloc(reinterpret_cast<void**>(&p->slab), layer_bytes * (uint64_t)d->n_layers));
    for (int l = 0; l < d->n_layers; ++l) {
        p->k_layer.push_back(p->slab + (uint64_t)l * layer_bytes);
        p->v_layer.push_back(p->slab + (uint64_t)l * layer_bytes + g.k_pool_bytes);
    }
    BKV_TRY(launch_fill(p->slab, layer_bytes * (uint64_t)d->n_layers, 0u, nullptr));
    const uint64_t table_bytes = (uint64_t)d->max_seqs * (uint64_t)d->max_pages_per_seq * 4u;
    BKV_TRY(hipMalloc(reinterpret_cast<void**>(&p->table_dev), (table_bytes + 15u) & ~15ull));
    BKV_TRY(launch_fill(p->table_dev, (table_bytes + 15u) & ~15ull, 0xffffffffu, nullptr));

    BKV_TRY(hipMalloc(reinterpret_cast<void**>(&p->part_o), (uint64_t)p->max_wgs * 8u * 256u * 4u));
    BKV_TRY(hipMalloc(reinterpret_cast<void**>(&p->part_ml), (uint64_t)p->max_wgs * 8u * 2u * 4u));

    BKV_TRY(hipHostMalloc(reinterpret_cast<void**>(&p->ring.host),
                          ParamRing::kSlots * ParamRing::kSlotBytes, hipHostMallocDefault));
    BKV_TRY(hipMalloc(reinterpret_cast<void**>(&p->ring.dev),
                      ParamRing::kSlots * ParamRing::kSlotBytes));
    for (int i = 0; i < ParamRing::kSlots; ++i)
        BKV_TRY(hipEventCreateWithFlags(&p->ring.ev[i], hipEventDisableTiming));

    const uint64_t swap_page = (g.k_page_bytes + g.v_page_bytes) * (uint64_t)d->n_layers;
    p->stage.bytes = std::max<uint64_t>(32ull << 20, 4 * swap_page);
    for (int i = 0; i < SwapStage::kHalves; ++i) {
        BKV_TRY(hipMalloc(reinterpret_cast<void**>(&p->stage.dev[i]), p->stage.bytes));
        BKV_TRY(hipEventCreateWithFlags(&p->stage.ev_stream[i], hipEventDisableTiming));
        BKV_TRY(hipEventCreateWithFlags(&p->stage.ev_side[i], hipEventDisableTiming));
    }
    BKV_TRY(hipStreamCreateWithFlags(&p->side, hipStreamNonBlocking));
    BKV_TRY(hipEventCreateWithFlags(&p->side_done, hipEventDisableTiming));
    // created here rather than on first use: the calls that order work with them create nothing
    BKV_TRY(hipEventCreateWithFlags(&p->attn_ws.ev, hipEventDisableTiming));
    BKV_TRY(hipEventCreateWithFlags(&p->sel_ws.ev, hipEventDisableTiming));
    BKV_TRY(hipEventCreateWithFlags(&p->table_sync.ev, hipEventDisableTiming));
    // this device's copy of the static scratch of bkv_decode_attn_static
    BKV_TRY(attn_static_scratch_init(p->device));
    BKV_TRY(hipDeviceSynchronize());
#undef BKV_TRY
    *out = p;
    return BKV_OK;
}

bkv_status bkv_pool_destroy(bkv_pool* p) {
    if (!p) return fail(BKV_ERR_INVALID, "pool_destroy: NULL pool");
    if (p->live_plans > 0)
        return fail(BKV_ERR_STATE, sfmt("pool_destroy: %lld step plans of this pool are still alive; destroy them "
                                        "first (they point into the pool)", p->live_plans));
    destroy_device_side(p);
    delete p;
    return BKV_OK;
}

bkv_status bkv_pool_reset(bkv_pool* p, void* stream) {
    if (!p) return fail(BKV_ERR_INVALID, "pool_reset: NULL pool");
    p->prefix->clear();
    p->alloc->reset();
    if (p->host_only) {
        p->alloc->pending().clear();
        return BKV_OK;
    }
    const uint64_t layer_bytes = p->g.k_pool_bytes + p->g.v_pool_bytes;
    bkv_status st = wait_for_tier_moves(p, S(stream));
    if (st != BKV_OK) return st;
    BKV_HIP(launch_fill(p->slab, layer_bytes * (uint64_t)p->g.n_layers, 0u, S(stream)));
    return flush_tables(p, S(stream));
}

bkv_status bkv_pool_get_desc(const bkv_pool* p, bkv_pool_desc* out) {
    if (!p || !out) return fail(BKV_ERR_INVALID, "pool_get_desc: NULL argument");
    *out = p->desc;
    return BKV_OK;
}

uint64_t bkv_pool_bytes(const bkv_pool* p) {
    if (!p) return 0;
    return (p->g.k_pool_bytes + p->g.v_pool_bytes) * (uint64_t)p->g.n_layers +
           (uint64_t)p->desc.max_seqs * (uint64_t)p->desc.max_pages_per_seq * 4u;
}

uint64_t bkv_page_bytes(const bkv_pool* p, int which) {
    if (!p) return 0;
    return which ? p->g.v_page_bytes : p->g.k_page_bytes;
}

bkv_status bkv_pool_fill(bkv_pool* p, int byte, void* stream) {
    bkv_status st = need_device(p);
    if (st != BKV_OK) return st;
    const uint32_t b = (uint32_t)(byte & 0xff);
    const uint32_t word = b | (b << 8) | (b << 16) | (b << 24);
    const uint64_t layer_bytes = p->g.k_pool_bytes + p->g.v_pool_bytes;
    st = wait_for_tier_moves(p, S(stream));
    if (st != BKV_OK) return st;
    BKV_HIP(launch_fill(p->slab, layer_bytes * (uint64_t)p->g.n_layers, word, S(stream)));
    return BKV_OK;
}

bkv_status bkv_pool_layer_ptr(const bkv_pool* p, int32_t layer, int which, void** dev_ptr,
                              uint64_t* bytes) {
    bkv_status st = need_device(p);
    if (st != BKV_OK) return st;
    if (layer < 0 || layer >= p->g.n_layers)
        return fail(BKV_ERR_RANGE, sfmt("layer %lld is outside 0..%lld", layer, p->g.n_layers));
    if (dev_ptr) *dev_ptr = which ? p->v_layer[(size_t)layer] : p->k_layer[(size_t)layer];
    if (bytes) *bytes = which ? p->g.v_pool_bytes : p->g.k_pool_bytes;
    return BKV_OK;
}

// ---- allocator ----------------------------------------------------------------------
bkv_status bkv_seq_create(bkv_pool* p, int32_t* seq_out) {
    if (!p || !seq_out) return fail(BKV_ERR_INVALID, "seq_create: NULL argument");
    std::string err;
    return from_alloc(p->alloc->seq_create(seq_out, err), err);
}

bkv_status bkv_seq_create_identity(bkv_pool* p, int32_t n_pages, int32_t* seq_out) {
    if (!p || !seq_out) return fail(BKV_ERR_INVALID, "seq_create_identity: NULL argument");
    std::string err;
    return from_alloc(p->alloc->seq_create_identity(n_pages, seq_out, err), err);
}

bkv_status bkv_seq_fork(bkv_pool* p, int32_t parent, int64_t n_tokens, int32_t* child_out) {
    if (!p || !child_out) return fail(BKV_ERR_INVALID, "seq_fork: NULL argument");
    std::string err;
    return from_alloc(p->alloc->seq_fork(parent, n_tokens, child_out, err), err);
}

bkv_status bkv_seq_free(bkv_pool* p, int32_t seq) {
    if (!p) return fail(BKV_ERR_INVALID, "seq_free: NULL pool");
    std::string err;
    return from_alloc(p->alloc->seq_free(seq, err), err);
}

// Moves the bytes behind the prefix tree's tier bookkeeping (defined with the swap path below).
static bkv_status run_tier_moves(bkv_pool* p, const std::vector<TierMove>& moves);

// Make `want` device pages free by evicting cached prefixes: demoted to the lower tiers when the
// pool has them, dropped otherwise.
static bkv_status prefix_make_room(bkv_pool* p, int32_t want, int32_t* freed) {
    std::vector<TierMove> moves;
    const int32_t n = p->prefix->evict(want, p->prefix->tiered() ? &moves : nullptr);
    if (freed) *freed = n;
    return run_tier_moves(p, moves);
}

bkv_status bkv_seq_reserve(bkv_pool* p, int32_t seq, int64_t new_len, bkv_page_pair* cow,
                           int32_t cow_cap, int32_t* n_cow) {
    if (!p) return fail(BKV_ERR_INVALID, "seq_reserve: NULL pool");
    std::string err;
    static_assert(sizeof(PagePair) == sizeof(bkv_page_pair), "pair layouts must agree");
    AllocErr e = p->alloc->seq_reserve(seq, new_len, reinterpret_cast<PagePair*>(cow), cow_cap, n_cow, err);
    if (e == AllocErr::NoPages && p->prefix->nodes() > 0) {
        // Out of free pages: cached prefixes that nobody uses are the first thing to go
        // (least recently used first), then the request is tried once more.
        const int64_t grow = (new_len - p->alloc->seq_len(seq) + p->g.page_cells - 1) / p->g.page_cells + 1;
        const int64_t missing = grow - p->alloc->free_pages();
        if (missing > 0) {
            int32_t freed = 0;
            const bkv_status st = prefix_make_room(p, (int32_t)missing, &freed);
            if (st != BKV_OK) return st;
            if (freed > 0) {
                err.clear();
                e = p->alloc->seq_reserve(seq, new_len, reinterpret_cast<PagePair*>(cow), cow_cap, n_cow, err);
            }
        }
    }
    return from_alloc(e, err);
}

// ---- prefix tree ----------------------------------------------------------------------------
static bkv_status prefix_args(const bkv_pool* p, const char* what, const int32_t* tokens, int64_t n) {
    if (!p) return fail(BKV_ERR_INVALID, std::string(what) + ": NULL pool");
    if (n < 0 || (n > 0 && !tokens))
        return fail(BKV_ERR_INVALID, std::string(what) + sfmt(": %lld tokens and a NULL pointer", n));
    return BKV_OK;
}

bkv_status bkv_prefix_match(bkv_pool* p, const int32_t* tokens, int64_t n_tokens,
                            int64_t* matched_tokens) {
    bkv_status st = prefix_args(p, "prefix_match", tokens, n_tokens);
    if (st != BKV_OK) return st;
    std::vector<PrefixTree::Node*> chain;
    p->prefix->match_nodes(tokens, n_tokens, false, chain);
    if (matched_tokens) *matched_tokens = (int64_t)chain.size() * p->g.page_cells;
    return BKV_OK;
}

// The chain of listed pages that matches tokens[0..n), with its lower part brought back to fresh
// device pages as far as pages can be had (other cached prefixes make room if they must; the
// chain itself is held meanwhile).  The transfers are enqueued, not awaited.
static bkv_status promote_matched_chain(bkv_pool* p, const int32_t* tokens, int64_t n_tokens,
                                        std::vector<PrefixTree::Node*>& chain) {
    p->prefix->match_nodes(tokens, n_tokens, true, chain);
    if ((int64_t)chain.size() > p->alloc->max_pages_per_seq()) chain.resize((size_t)p->alloc->max_pages_per_seq());
    int32_t lower = 0;
    for (const PrefixTree::Node* x : chain) lower += PrefixTree::tier_of(x) != Tier::Device;
    if (lower == 0) return BKV_OK;
    std::vector<TierMove> moves;
    p->prefix->pin_nodes(chain, +1);
    const int32_t missing = lower - p->alloc->free_pages();
    if (missing > 0) p->prefix->evict(missing, &moves);
    p->prefix->promote(chain, lower, moves);
    p->prefix->pin_nodes(chain, -1);
    return run_tier_moves(p, moves);
}

bkv_status bkv_prefix_prefetch(bkv_pool* p, const int32_t* tokens, int64_t n_tokens, int64_t* device_tokens) {
    bkv_status st = prefix_args(p, "prefix_prefetch", tokens, n_tokens);
    if (st != BKV_OK) return st;
    std::vector<PrefixTree::Node*> chain;
    st = promote_matched_chain(p, tokens, n_tokens, chain);
    if (st != BKV_OK) return st;
    int64_t on_device = 0;
    for (const PrefixTree::Node* x : chain) {
        if (PrefixTree::tier_of(x) != Tier::Device) break;
        ++on_device;
    }
    if (device_tokens) *device_tokens = on_device * p->g.page_cells;
    return BKV_OK;
}

bkv_status bkv_seq_create_from_prefix(bkv_pool* p, const int32_t* tokens, int64_t n_tokens,
                                      int32_t* seq_out, int64_t* matched_tokens) {
    bkv_status st = prefix_args(p, "seq_create_from_prefix", tokens, n_tokens);
    if (st != BKV_OK) return st;
    if (!seq_out) return fail(BKV_ERR_INVALID, "seq_create_from_prefix: NULL output");
    std::vector<PrefixTree::Node*> chain;
    st = promote_matched_chain(p, tokens, n_tokens, chain);
    if (st != BKV_OK) return st;
    std::vector<int32_t> pages;
    for (const PrefixTree::Node* x : chain) {
        if (PrefixTree::tier_of(x) != Tier::Device) break;
        pages.push_back(PrefixTree::page_of(x));
    }
    std::string err;
    st = from_alloc(p->alloc->seq_create_shared(pages.data(), (int32_t)pages.size(), seq_out, err), err);
    if (st != BKV_OK) return st;
    if (matched_tokens) *matched_tokens = (int64_t)pages.size() * p->g.page_cells;
    return BKV_OK;
}

bkv_status bkv_prefix_insert(bkv_pool* p, int32_t seq, const int32_t* tokens, int64_t n_tokens,
                             int32_t* new_pages) {
    bkv_status st = prefix_args(p, "prefix_insert", tokens, n_tokens);
    if (st != BKV_OK) return st;
    if (!p->alloc->seq_valid(seq))
        return fail(BKV_ERR_RANGE, sfmt("prefix_insert: sequence %lld is not live", seq));
    if (n_tokens > p->alloc->seq_len(seq))
        return fail(BKV_ERR_RANGE, sfmt("prefix_insert: %lld tokens listed but sequence %lld holds %lld",
                                        n_tokens, seq, p->alloc->seq_len(seq)));
    std::string err;
    const int32_t added = p->prefix->insert(tokens, n_tokens, p->alloc->seq_table(seq),
                                            p->alloc->seq_n_pages(seq), err);
    if (added < 0) return fail(BKV_ERR_STATE, err);
    if (new_pages) *new_pages = added;
    return BKV_OK;
}

bkv_status bkv_prefix_evict(bkv_pool* p, int32_t want_pages, int32_t* freed) {
    if (!p) return fail(BKV_ERR_INVALID, "prefix_evict: NULL pool");
    if (want_pages < 0) return fail(BKV_ERR_INVALID, sfmt("prefix_evict: %lld pages wanted", want_pages));
    return prefix_make_room(p, want_pages, freed);
}

bkv_status bkv_prefix_pin(bkv_pool* p, const int32_t* tokens, int64_t n_tokens, int32_t pin,
                          int64_t* affected_tokens) {
    bkv_status st = prefix_args(p, "prefix_pin", tokens, n_tokens);
    if (st != BKV_OK) return st;
    const int32_t n = p->prefix->pin(tokens, n_tokens, pin ? +1 : -1);
    if (affected_tokens) *affected_tokens = (int64_t)n * p->g.page_cells;
    return BKV_OK;
}

bkv_status bkv_prefix_stats(const bkv_pool* p, int32_t* nodes, int32_t* evictable_pages,
                            int32_t* pinned_nodes) {
    if (!p) return fail(BKV_ERR_INVALID, "prefix_stats: NULL pool");
    if (nodes) *nodes = p->prefix->nodes();
    if (evictable_pages) *evictable_pages = p->prefix->evictable_pages();
    if (pinned_nodes) *pinned_nodes = p->prefix->pinned_nodes();
    return BKV_OK;
}

bkv_status bkv_prefix_clear(bkv_pool* p) {
    if (!p) return fail(BKV_ERR_INVALID, "prefix_clear: NULL pool");
    p->prefix->clear();
    return BKV_OK;
}

bkv_status bkv_seq_truncate(bkv_pool* p, int32_t seq, int64_t new_len) {
    if (!p) return fail(BKV_ERR_INVALID, "seq_truncate: NULL pool");
    std::string err;
    return from_alloc(p->alloc->seq_truncate(seq, new_len, err), err);
}

int64_t bkv_seq_len(const bkv_pool* p, int32_t seq) {
    if (!p || !p->alloc->seq_valid(seq)) return -1;
    return p->alloc->seq_len(seq);
}
int64_t bkv_seq_capacity(const bkv_pool* p, int32_t seq) {
    if (!p || !p->alloc->seq_valid(seq)) return -1;
    return p->alloc->seq_capacity(seq);
}
int32_t bkv_seq_n_pages(const bkv_pool* p, int32_t seq) {
    if (!p || !p->alloc->seq_valid(seq)) return -1;
    return p->alloc->seq_n_pages(seq);
}
const int32_t* bkv_seq_block_table(const bkv_pool* p, int32_t seq) {
    if (!p || !p->alloc->seq_valid(seq)) return nullptr;
    return p->alloc->seq_table(seq);
}
int32_t bkv_page_refcount(const bkv_pool* p, int32_t page) {
    if (!p || page < 0 || page >= p->g.n_pages) return -1;
    return p->alloc->refcount(page);
}
int32_t bkv_pool_free_pages(const bkv_pool* p) { return p ? p->alloc->free_pages() : -1; }

bkv_status bkv_pool_set_free_order(bkv_pool* p, const int32_t* order, int32_t n) {
    if (!p || (n > 0 && !order)) return fail(BKV_ERR_INVALID, "pool_set_free_order: NULL argument");
    std::string err;
    return from_alloc(p->alloc->set_free_order(order, n, err), err);
}

bkv_status bkv_pool_check(const bkv_pool* p) {
    if (!p) return fail(BKV_ERR_INVALID, "pool_check: NULL pool");
    std::string err;
    if (!p->alloc->check(err)) return fail(BKV_ERR_STATE, "allocator invariant broken: " + err);
    if (!p->prefix->check(err)) return fail(BKV_ERR_STATE, err);
    return BKV_OK;
}

// ---- append ------------------------------------------------------------------------
// Cells [c0, c1) of a live sequence may be written only when they have been reserved
// (bkv_seq_reserve moved the sequence's length past them) and every page they lie on is on the
// device and held by this sequence alone: a page that a fork, a cached prefix or another
// sequence still shares would change under its other holders.  bkv_seq_reserve is what replaces
// such a page (and reports the copy to make); writing without it is a state error here, before
// anything is launched.
static bkv_status check_writable(const bkv_pool* p, const char* what, int32_t seq, int64_t c0, int64_t c1) {
    const int64_t len = p->alloc->seq_len(seq);
    if (c1 > len)
        return fail(BKV_ERR_RANGE, std::string(what) + sfmt(" would write cells %lld..%lld of sequence %lld but "
                                                            "only %lld are reserved (bkv_seq_reserve first)",
                                                            c0, c1, seq, len));
    const int32_t* row = p->alloc->seq_table(seq);
    for (int64_t c = c0 / p->g.page_cells; c <= (c1 - 1) / p->g.page_cells; ++c) {
        if (row[c] < 0)
            return fail(BKV_ERR_STATE, std::string(what) + sfmt(": logical page %lld of sequence %lld is "
                                                                "swapped out", c, seq));
        if (p->alloc->refcount(row[c]) != 1)
            return fail(BKV_ERR_STATE, std::string(what) + sfmt(": logical page %lld of sequence %lld (page %lld) "
                                                                "has %lld holders; bkv_seq_reserve replaces a "
                                                                "shared page before it is written",
                                                                c, seq, row[c], p->alloc->refcount(row[c])));
    }
    return BKV_OK;
}

// Range checks shared by the append entry points (qsa/mod.rs:1108-1116: a write past the
// cache is an error before anything is launched) and the per-sequence launch arguments.
static bkv_status build_append_batch(bkv_pool* p, int32_t layer, int32_t n_seqs, const int32_t* seqs,
                                     const int64_t* pos0, const int32_t* n_tokens, AppendBatch& b,
                                     int64_t& total, int32_t& max_tok) {
    if (!p) return fail(BKV_ERR_INVALID, "append: NULL pool");
    if (layer < 0 || layer >= p->g.n_layers)
        return fail(BKV_ERR_RANGE, sfmt("append: layer %lld is outside 0..%lld", layer,
                                        p->g.n_layers));
    if (n_seqs < 0 || n_seqs > BKV_MAX_BATCH)
        return fail(BKV_ERR_INVALID, sfmt("append: %lld sequences in one call; the limit is %lld",
                                          n_seqs, BKV_MAX_BATCH));
    if (n_seqs > 0 && (!seqs || !pos0 || !n_tokens))
        return fail(BKV_ERR_INVALID, "append: NULL sequence / position / token-count array");
    b = AppendBatch{};
    total = 0;
    max_tok = 0;
    for (int i = 0; i < n_seqs; ++i) {
        if (!p->alloc->seq_valid(seqs[i]))
            return fail(BKV_ERR_RANGE, sfmt("append: sequence %lld is not live", seqs[i]));
        if (n_tokens[i] < 0 || pos0[i] < 0)
            return fail(BKV_ERR_RANGE, sfmt("append: entry %lld has pos0 %lld, n_tokens %lld", i,
                                            pos0[i], n_tokens[i]));
        const int64_t end = pos0[i] + n_tokens[i];
        const int64_t cap = p->alloc->seq_capacity(seqs[i]);
        if (end > cap)
            return fail(BKV_ERR_RANGE,
                        sfmt("append would write cells %lld..%lld of sequence %lld but it holds "
                             "%lld (a write past the block table would land on an unmapped page)",
                             pos0[i], end, seqs[i], cap));
        if (n_tokens[i] > 0) {
            bkv_status wst = check_writable(p, "append", seqs[i], pos0[i], end);
            if (wst != BKV_OK) return wst;
        }
        b.row[i] = seqs[i];
        b.pos0[i] = (int32_t)pos0[i];
        b.n_tok[i] = n_tokens[i];
        b.src0[i] = (int32_t)total;
        total += n_tokens[i];
        max_tok = std::max(max_tok, n_tokens[i]);
    }
    b.n = n_seqs;
    if (total > ((int64_t)1 << 30))
        return fail(BKV_ERR_INVALID, "append: more than 2^30 tokens in one call");
    return need_device(p);
}

static bkv_status append_rows(bkv_pool* p, int32_t layer, int32_t n_seqs, const int32_t* seqs,
                              const int64_t* pos0, const int32_t* n_tokens, const void* k_dev,
                              const void* v_dev, bool src_is_f16, void* stream) {
    AppendBatch b;
    int64_t total;
    int32_t max_tok;
    bkv_status st = build_append_batch(p, layer, n_seqs, seqs, pos0, n_tokens, b, total, max_tok);
    if (st != BKV_OK) return st;
    if (total == 0) return flush_tables(p, S(stream));
    if (!k_dev || !v_dev || !aligned16(k_dev) || !aligned16(v_dev))
        return fail(BKV_ERR_INVALID, "append: k/v device pointers must be non-NULL and 16-byte "
                                     "aligned");
    st = flush_tables(p, S(stream));
    if (st != BKV_OK) return st;
    BKV_HIP(launch_append(p, layer, b, max_tok, k_dev, v_dev, src_is_f16, S(stream)));
    return BKV_OK;
}

bkv_status bkv_append(bkv_pool* p, int32_t layer, int32_t n_seqs, const int32_t* seqs,
                      const int64_t* pos0, const int32_t* n_tokens, const float* k_dev,
                      const float* v_dev, void* stream) {
    return append_rows(p, layer, n_seqs, seqs, pos0, n_tokens, k_dev, v_dev, false, stream);
}

bkv_status bkv_append_f16(bkv_pool* p, int32_t layer, int32_t n_seqs, const int32_t* seqs,
                          const int64_t* pos0, const int32_t* n_tokens, const uint16_t* k_dev,
                          const uint16_t* v_dev, void* stream) {
    return append_rows(p, layer, n_seqs, seqs, pos0, n_tokens, k_dev, v_dev, true, stream);
}

bkv_status bkv_append_kprep(bkv_pool* p, int32_t layer, int32_t n_seqs, const int32_t* seqs,
                            const int64_t* pos0, const int32_t* n_tokens, const float* k_dev,
                            const float* v_dev, const float* k_gamma_dev, float eps,
                            const float* rope_table_dev, int32_t n_rot, int32_t max_pos,
                            const int32_t* positions_dev, void* stream) {
    AppendBatch b;
    int64_t total;
    int32_t max_tok;
    bkv_status st = build_append_batch(p, layer, n_seqs, seqs, pos0, n_tokens, b, total, max_tok);
    if (st != BKV_OK) return st;
    if (n_rot <= 0 || n_rot % 2 != 0 || n_rot > p->g.hd)
        return fail(BKV_ERR_INVALID, sfmt("append_kprep: n_rot %lld must be even and within 2..%lld",
                                          n_rot, p->g.hd));
    if (max_pos <= 0)
        return fail(BKV_ERR_INVALID, sfmt("append_kprep: a rotary table of %lld positions", max_pos));
    if (!(eps >= 0.0f)) return fail(BKV_ERR_INVALID, "append_kprep: eps must be >= 0");
    if (total == 0) return flush_tables(p, S(stream));
    if (!k_dev || !v_dev || !aligned16(k_dev) || !aligned16(v_dev))
        return fail(BKV_ERR_INVALID, "append_kprep: k/v device pointers must be non-NULL and "
                                     "16-byte aligned");
    if (!k_gamma_dev || !rope_table_dev || ((uintptr_t)rope_table_dev & 7u))
        return fail(BKV_ERR_INVALID, "append_kprep: gamma and the rotary table must be non-NULL "
                                     "device pointers (table 8-byte aligned)");
    st = flush_tables(p, S(stream));
    if (st != BKV_OK) return st;
    BKV_HIP(launch_append_kprep(p, layer, b, max_tok, k_dev, v_dev, k_gamma_dev, eps,
                                rope_table_dev, n_rot, max_pos, positions_dev, S(stream)));
    return BKV_OK;
}

bkv_status bkv_rope_table(double freq_base, int32_t n_rot, int32_t max_pos, float* host_out) {
    if (n_rot <= 0 || n_rot % 2 != 0)
        return fail(BKV_ERR_INVALID, sfmt("rope_table: n_rot %lld must be even and positive", n_rot));
    if (max_pos <= 0) return fail(BKV_ERR_INVALID, "rope_table: an empty table");
    if (!host_out) return fail(BKV_ERR_INVALID, "rope_table: NULL output");
    const int half = n_rot / 2;
    for (int64_t pos = 0; pos < max_pos; ++pos)
        for (int i = 0; i < half; ++i) {
            const double inv = std::pow(freq_base, -2.0 * (double)i / (double)n_rot);
            const double ang = (double)pos * inv;
            host_out[(pos * half + i) * 2] = (float)std::cos(ang);
            host_out[(pos * half + i) * 2 + 1] = (float)std::sin(ang);
        }
    return BKV_OK;
}

// ---- decode attention ----------------------------------------------------------------
// Shared by the dense and the selection-list entry points.
static bkv_status decode_attn_common(bkv_pool* p, int32_t layer, int32_t n, const int32_t* seqs,
                                     const int64_t* pos, int32_t n_q_head, const float* q_dev,
                                     const float* gate_dev, int64_t gate_seq_stride,
                                     int64_t gate_head_stride, float scale, const uint32_t* ids_dev,
                                     int64_t id_stride, const uint32_t* counts_dev, int32_t max_ids,
                                     bool select, float* out_dev, void* stream,
                                     const float* new_k_dev = nullptr, const float* new_v_dev = nullptr,
                                     bool step = false, bool static_ws = false) {
    if (!p) return fail(BKV_ERR_INVALID, "decode_attn: NULL pool");
    if (layer < 0 || layer >= p->g.n_layers)
        return fail(BKV_ERR_RANGE, sfmt("decode_attn: layer %lld is outside 0..%lld", layer,
                                        p->g.n_layers));
    if (n < 0 || n > BKV_MAX_BATCH)
        return fail(BKV_ERR_INVALID, sfmt("decode_attn: %lld entries in one call; the limit is "
                                          "%lld", n, BKV_MAX_BATCH));
    if (n_q_head <= 0 || n_q_head % p->g.n_kv != 0 || n_q_head / p->g.n_kv > BKV_MAX_HEAD_GROUP)
        return fail(BKV_ERR_INVALID,
                    sfmt("decode_attn: %lld q heads over %lld kv heads (need a whole group of at "
                         "most %lld)", n_q_head, p->g.n_kv, BKV_MAX_HEAD_GROUP));
    if (p->g.hd != 256)
        return fail(BKV_ERR_INVALID, sfmt("decode_attn is built for head_dim 256, pool has %lld",
                                          p->g.hd));
    if (select) {
        if (p->g.page_cells % 4 != 0)
            return fail(BKV_ERR_INVALID, "decode_attn_select: 4-cell blocks need a page size that "
                                         "is a multiple of 4");
        if (max_ids <= 0 || max_ids > (1 << 24))
            return fail(BKV_ERR_INVALID, sfmt("decode_attn_select: max_ids %lld is outside "
                                              "1..2^24", max_ids));
        if (id_stride < max_ids)
            return fail(BKV_ERR_INVALID, sfmt("decode_attn_select: id_stride %lld is smaller than "
                                              "max_ids %lld", id_stride, max_ids));
    }
    if (n > 0 && (!seqs || !pos)) return fail(BKV_ERR_INVALID, "decode_attn: NULL seqs / pos");
    AttnBatch b{};
    for (int i = 0; i < n; ++i) {
        if (!p->alloc->seq_valid(seqs[i]))
            return fail(BKV_ERR_RANGE, sfmt("decode_attn: sequence %lld is not live", seqs[i]));
        const int64_t cap = p->alloc->seq_capacity(seqs[i]);
        if (pos[i] < 0 || pos[i] >= cap)
            return fail(BKV_ERR_RANGE, sfmt("decode_attn: position %lld of sequence %lld is "
                                            "outside its %lld addressable cells", pos[i], seqs[i],
                                            cap));
        if (!p->alloc->seq_resident(seqs[i], pos[i] + 1))
            return fail(BKV_ERR_STATE, sfmt("decode_attn: sequence %lld has swapped-out pages "
                                            "below position %lld", seqs[i], pos[i]));
        if (step) {
            const bkv_status wst = check_writable(p, "decode_step", seqs[i], pos[i], pos[i] + 1);
            if (wst != BKV_OK) return wst;
        }
        if (step)
            for (int j = 0; j < i; ++j)
                if (seqs[j] == seqs[i])
                    return fail(BKV_ERR_INVALID, sfmt("decode_step: sequence %lld appears twice; one "
                                                      "new token per sequence and call", seqs[i]));
        b.row[i] = seqs[i];
        b.pos[i] = (int32_t)pos[i];
    }
    b.n = n;
    bkv_status st = need_device(p);
    if (st != BKV_OK) return st;
    if (n == 0) return BKV_OK;
    if (!q_dev || !out_dev || !aligned16(q_dev) || !aligned16(out_dev))
        return fail(BKV_ERR_INVALID, "decode_attn: q/out device pointers must be non-NULL and "
                                     "16-byte aligned");
    if (step && (!new_k_dev || !new_v_dev || !aligned16(new_k_dev) || !aligned16(new_v_dev)))
        return fail(BKV_ERR_INVALID, "decode_step: k/v device pointers must be non-NULL and 16-byte "
                                     "aligned");
    if (select && (!ids_dev || !counts_dev || ((uintptr_t)ids_dev & 3u) || ((uintptr_t)counts_dev & 3u)))
        return fail(BKV_ERR_INVALID, "decode_attn_select: ids/counts device pointers must be "
                                     "non-NULL and 4-byte aligned");
    // the cut into work-groups comes before anything is enqueued: a batch it cannot serve is an
    // error like any other size violation
    const int32_t ws_wgs = static_ws ? kStaticWgs : p->max_wgs;
    if (plan_attn(p, n_q_head, b, select ? (max_ids + 3) / 4 : 0, ws_wgs) < 0)
        return fail(BKV_ERR_INVALID,
                    sfmt(static_ws ? "decode_attn_static: %lld entries x %lld kv heads need more work-groups than "
                                     "the static scratch holds (%lld); use smaller batches or bkv_decode_attn"
                                   : "decode_attn: %lld entries x %lld kv heads need more work-groups than the "
                                     "partial-result workspace holds (%lld); use smaller batches",
                         n, p->g.n_kv,
                         attn_plan_limits(p->n_cu, ws_wgs, p->g.n_kv, n_q_head / p->g.n_kv).max_wgs));
    AttnArgs a;
    if (static_ws) {
        if (!attn_static_scratch(p->device, &a.ws_o, &a.ws_ml))
            return fail(BKV_ERR_STATE, "decode_attn_static: the static scratch of this device was not set up");
        a.timed = false;
        // A stream under capture cannot record the usual way block-table changes travel (it may wait on
        // the host for a free ring slot): as for step plans, they are made before the capture.
        if (!p->alloc->pending().empty() || p->tiers.pending) {
            hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
            if (stream && hipStreamIsCapturing(S(stream), &cs) == hipSuccess && cs != hipStreamCaptureStatusNone)
                return fail(BKV_ERR_STATE, "decode_attn_static: block-table changes are pending while the stream is "
                                           "being captured; make allocator calls, then any eager call, before the "
                                           "capture");
            (void)hipGetLastError();
        }
    }
    st = flush_tables(p, S(stream));
    if (st != BKV_OK) return st;
    a.n_q_head = n_q_head;
    a.q = q_dev;
    a.gate = gate_dev;
    a.gate_seq_stride = gate_seq_stride;
    a.gate_head_stride = gate_head_stride;
    a.scale = scale;
    a.out = out_dev;
    if (select) {
        a.ids = ids_dev;
        a.counts = counts_dev;
        a.id_stride = id_stride;
        a.max_ids = max_ids;
    }
    if (step) {
        a.new_k = new_k_dev;
        a.new_v = new_v_dev;
    }
    // the pool's own workspace is ordered across streams; the static scratch is the device's, shared by
    // every pool, and overlapping calls on it are the caller's to avoid
    if (!static_ws) {
        st = order_workspace(p->attn_ws, S(stream));
        if (st != BKV_OK) return st;
    }
    BKV_HIP(launch_decode_attn(p, layer, b, a, S(stream)));
    return BKV_OK;
}

bkv_status bkv_attn_plan(int32_t n_cu, int32_t n_kv_head, int32_t n_q_head, int32_t n, const int64_t* pos,
                         int32_t sel_groups, int32_t* splits_out, int32_t* pps_out, int32_t* total_out) {
    if (n_cu <= 0 || n_kv_head <= 0 || n_kv_head > BKV_MAX_KV_HEAD)
        return fail(BKV_ERR_INVALID, sfmt("attn_plan: %lld compute units, %lld kv heads", n_cu, n_kv_head));
    if (n_q_head <= 0 || n_q_head % n_kv_head != 0 || n_q_head / n_kv_head > BKV_MAX_HEAD_GROUP)
        return fail(BKV_ERR_INVALID, sfmt("attn_plan: %lld q heads over %lld kv heads (need a whole group of "
                                          "at most %lld)", n_q_head, n_kv_head, BKV_MAX_HEAD_GROUP));
    if (n < 0 || n > BKV_MAX_BATCH || (n > 0 && !pos) || sel_groups < 0)
        return fail(BKV_ERR_INVALID, sfmt("attn_plan: %lld entries (limit %lld), sel_groups %lld", n,
                                          BKV_MAX_BATCH, sel_groups));
    AttnBatch b{};
    b.n = n;
    for (int i = 0; i < n; ++i) {
        if (pos[i] < 0 || pos[i] > 0x7ffffff0)
            return fail(BKV_ERR_RANGE, sfmt("attn_plan: position %lld of entry %lld", pos[i], i));
        b.pos[i] = (int32_t)pos[i];
    }
    const AttnPlanLimits lim = attn_plan_limits(n_cu, kMaxWgs, n_kv_head, n_q_head / n_kv_head);
    const int32_t total = plan_attn_ranges(lim, 16, sel_groups, b);
    if (total < 0)
        return fail(BKV_ERR_INVALID, sfmt("attn_plan: %lld entries x %lld kv heads need more work-groups than "
                                          "the partial-result workspace holds (%lld)", n, n_kv_head, lim.max_wgs));
    for (int i = 0; i < n; ++i) {
        if (splits_out) splits_out[i] = b.splits[i];
        if (pps_out) pps_out[i] = b.pps[i];
    }
    if (total_out) *total_out = total;
    return BKV_OK;
}

bkv_status bkv_decode_attn(bkv_pool* p, int32_t layer, int32_t n, const int32_t* seqs,
                           const int64_t* pos, int32_t n_q_head, const float* q_dev,
                           const float* gate_dev, int64_t gate_seq_stride,
                           int64_t gate_head_stride, float scale, float* out_dev, void* stream) {
    return decode_attn_common(p, layer, n, seqs, pos, n_q_head, q_dev, gate_dev, gate_seq_stride,
                              gate_head_stride, scale, nullptr, 0, nullptr, 0, false, out_dev, stream);
}

bkv_status bkv_decode_attn_static(bkv_pool* p, int32_t layer, int32_t n, const int32_t* seqs,
                                  const int64_t* pos, int32_t n_q_head, const float* q_dev,
                                  const float* gate_dev, int64_t gate_seq_stride,
                                  int64_t gate_head_stride, float scale, float* out_dev, void* stream) {
    return decode_attn_common(p, layer, n, seqs, pos, n_q_head, q_dev, gate_dev, gate_seq_stride,
                              gate_head_stride, scale, nullptr, 0, nullptr, 0, false, out_dev, stream,
                              nullptr, nullptr, false, true);
}

bkv_status bkv_decode_step(bkv_pool* p, int32_t layer, int32_t n, const int32_t* seqs, const int64_t* pos,
                           const float* k_new_dev, const float* v_new_dev, int32_t n_q_head,
                           const float* q_dev, const float* gate_dev, int64_t gate_seq_stride,
                           int64_t gate_head_stride, float scale, float* out_dev, void* stream) {
    return decode_attn_common(p, layer, n, seqs, pos, n_q_head, q_dev, gate_dev, gate_seq_stride,
                              gate_head_stride, scale, nullptr, 0, nullptr, 0, false, out_dev, stream,
                              k_new_dev, v_new_dev, true);
}

// ---- step plans: a decode step whose batch lives on the device -------------------------------
struct bkv_step_plan {
    bkv_pool* pool = nullptr;
    StepDesc* dev = nullptr;
    float* part_o = nullptr;  // the plan's own split-K workspace: no sharing, nothing to order
    float* part_ml = nullptr;
    int32_t n = 0, n_q_head = 0, grid = 0;
    AttnPlanLimits lim{};
    // The descriptor is uploaded on the stream of bkv_step_plan_create, rewritten by every advance
    // and read by every decode: a call that arrives on another stream than the plan's last one is
    // ordered behind it with an event recorded there at that moment.
    WorkspaceOrder order;
    // what the plan was checked for: cells first[i]..last[i] of sequence seq[i]
    int32_t seq[kMaxBatch] = {};
    int64_t first[kMaxBatch] = {}, last[kMaxBatch] = {};
};

// The cells a plan was created for must still be what they were then (reserved, on the device, held
// by the sequence alone): a host call that enqueues the plan's kernels looks again, so that a
// sequence freed, forked, truncated or evicted in between is an error here and not a write into
// somebody else's page.  (A replayed graph makes no host call; there the rule is the caller's.)
static bkv_status plan_cells_unchanged(const bkv_step_plan* pl, const char* what) {
    const bkv_pool* p = pl->pool;
    for (int i = 0; i < pl->n; ++i) {
        if (!p->alloc->seq_valid(pl->seq[i]))
            return fail(BKV_ERR_STATE, std::string(what) + sfmt(": sequence %lld of the plan is no longer live",
                                                                pl->seq[i]));
        if (pl->last[i] >= p->alloc->seq_capacity(pl->seq[i]) || !p->alloc->seq_resident(pl->seq[i], pl->last[i] + 1))
            return fail(BKV_ERR_STATE, std::string(what) + sfmt(": sequence %lld of the plan lost pages below cell "
                                                                "%lld since the plan was made", pl->seq[i],
                                                                pl->last[i]));
        const bkv_status wst = check_writable(p, what, pl->seq[i], pl->first[i], pl->last[i] + 1);
        if (wst != BKV_OK) return wst == BKV_ERR_RANGE ? fail(BKV_ERR_STATE, g_last_error) : wst;
    }
    return BKV_OK;
}

bkv_status bkv_step_plan_create(bkv_pool* p, int32_t n, const int32_t* seqs, const int64_t* pos,
                                int32_t horizon, int32_t n_q_head, void* stream, bkv_step_plan** out) {
    if (!p || !out) return fail(BKV_ERR_INVALID, "step_plan_create: NULL argument");
    *out = nullptr;
    if (n <= 0 || n > BKV_MAX_BATCH || !seqs || !pos)
        return fail(BKV_ERR_INVALID, sfmt("step_plan_create: %lld entries (1..%lld) or NULL seqs / pos", n,
                                          BKV_MAX_BATCH));
    if (horizon <= 0) return fail(BKV_ERR_INVALID, sfmt("step_plan_create: a horizon of %lld tokens", horizon));
    if (n_q_head <= 0 || n_q_head % p->g.n_kv != 0 || n_q_head / p->g.n_kv > BKV_MAX_HEAD_GROUP)
        return fail(BKV_ERR_INVALID, sfmt("step_plan_create: %lld q heads over %lld kv heads (need a whole group "
                                          "of at most %lld)", n_q_head, p->g.n_kv, BKV_MAX_HEAD_GROUP));
    if (p->g.hd != 256)
        return fail(BKV_ERR_INVALID, sfmt("step_plan_create: built for head_dim 256, pool has %lld", p->g.hd));
    StepDesc host{};
    for (int i = 0; i < n; ++i) {
        if (!p->alloc->seq_valid(seqs[i]))
            return fail(BKV_ERR_RANGE, sfmt("step_plan_create: sequence %lld is not live", seqs[i]));
        for (int j = 0; j < i; ++j)
            if (seqs[j] == seqs[i])
                return fail(BKV_ERR_INVALID, sfmt("step_plan_create: sequence %lld appears twice; one new token "
                                                  "per sequence and step", seqs[i]));
        const int64_t last = pos[i] + horizon - 1;  // the last cell a step of this plan may write and attend
        if (pos[i] < 0 || last >= p->alloc->seq_capacity(seqs[i]))
            return fail(BKV_ERR_RANGE, sfmt("step_plan_create: cells %lld..%lld of sequence %lld are outside its "
                                            "addressable cells", pos[i], last, seqs[i]));
        if (!p->alloc->seq_resident(seqs[i], last + 1))
            return fail(BKV_ERR_STATE, sfmt("step_plan_create: sequence %lld has swapped-out pages below position "
                                            "%lld", seqs[i], last));
        const bkv_status wst = check_writable(p, "step_plan_create", seqs[i], pos[i], last + 1);
        if (wst != BKV_OK) return wst;
        host.b.row[i] = seqs[i];
        host.b.pos[i] = (int32_t)pos[i];
        host.horizon[i] = (int32_t)last;
    }
    host.b.n = n;
    bkv_status st = need_device(p);
    if (st != BKV_OK) return st;
    const int32_t group = n_q_head / p->g.n_kv;
    const AttnPlanLimits lim = attn_plan_limits(p->n_cu, p->max_wgs, p->g.n_kv, group);
    if (plan_attn_ranges(lim, p->g.page_cells, 0, host.b) < 0)
        return fail(BKV_ERR_INVALID, sfmt("step_plan_create: %lld entries x %lld kv heads need more work-groups "
                                          "than the partial-result workspace holds (%lld)", n, p->g.n_kv,
                                          lim.max_wgs));
    bkv_step_plan* pl = new (std::nothrow) bkv_step_plan();
    if (!pl) return fail(BKV_ERR_NOMEM, "step_plan_create: out of host memory");
    pl->pool = p;
    ++p->live_plans;
    pl->n = n;
    pl->n_q_head = n_q_head;
    pl->lim = lim;
    for (int i = 0; i < n; ++i) {
        pl->seq[i] = seqs[i];
        pl->first[i] = pos[i];
        pl->last[i] = host.horizon[i];
    }
    // no cut of this batch, at any position, has more work-groups than this
    pl->grid = std::max<int32_t>(std::min(lim.target, lim.max_wgs), n * lim.per_page);
    auto bail = [&](bkv_status err) {
        const std::string keep = g_last_error;
        (void)bkv_step_plan_destroy(pl);
        g_last_error = keep;
        return err;
    };
    hipError_t e = hipMalloc(reinterpret_cast<void**>(&pl->dev), sizeof(StepDesc));
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void**>(&pl->part_o), (size_t)pl->grid * group * 256 * 4);
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void**>(&pl->part_ml), (size_t)pl->grid * group * 2 * 4);
    if (e != hipSuccess) return bail(hip_fail(e, "hipMalloc (step plan)"));
    st = flush_tables(p, S(stream));
    if (st != BKV_OK) return bail(st);
    void* staged;
    int slot;
    st = ring_upload(p, &host, sizeof(host), S(stream), &staged, &slot);
    if (st != BKV_OK) return bail(st);
    e = hipMemcpyAsync(pl->dev, staged, sizeof(host), hipMemcpyDeviceToDevice, S(stream));
    if (e != hipSuccess) return bail(hip_fail(e, "hipMemcpyAsync (step plan)"));
    st = ring_done(p, slot, S(stream));
    if (st != BKV_OK) return bail(st);
    pl->order.last = S(stream);
    pl->order.used = true;
    *out = pl;
    return BKV_OK;
}

bkv_status bkv_step_plan_destroy(bkv_step_plan* pl) {
    if (!pl) return fail(BKV_ERR_INVALID, "step_plan_destroy: NULL plan");
    (void)hipDeviceSynchronize();
    if (pl->order.ev) (void)hipEventDestroy(pl->order.ev);
    if (pl->dev) (void)hipFree(pl->dev);
    if (pl->part_o) (void)hipFree(pl->part_o);
    if (pl->part_ml) (void)hipFree(pl->part_ml);
    if (pl->pool) --pl->pool->live_plans;
    delete pl;
    return BKV_OK;
}

bkv_status bkv_step_plan_decode(bkv_step_plan* pl, int32_t layer, const float* k_new_dev, const float* v_new_dev,
                                const float* q_dev, const float* gate_dev, int64_t gate_seq_stride,
                                int64_t gate_head_stride, float scale, float* out_dev, void* stream) {
    if (!pl) return fail(BKV_ERR_INVALID, "step_plan_decode: NULL plan");
    bkv_pool* p = pl->pool;
    if (layer < 0 || layer >= p->g.n_layers)
        return fail(BKV_ERR_RANGE, sfmt("step_plan_decode: layer %lld is outside 0..%lld", layer, p->g.n_layers));
    if (!q_dev || !out_dev || !k_new_dev || !v_new_dev || !aligned16(q_dev) || !aligned16(out_dev) ||
        !aligned16(k_new_dev) || !aligned16(v_new_dev))
        return fail(BKV_ERR_INVALID, "step_plan_decode: q / out / k / v device pointers must be non-NULL and "
                                     "16-byte aligned");
    const bkv_status still = plan_cells_unchanged(pl, "step_plan_decode");
    if (still != BKV_OK) return still;
    // Block-table changes made since the last call still travel the usual way, which a stream under
    // capture cannot record (it waits on the host for a free ring slot): make them before capturing.
    if (!p->alloc->pending().empty() || p->tiers.pending) {
        hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
        if (stream && hipStreamIsCapturing(S(stream), &cs) == hipSuccess && cs != hipStreamCaptureStatusNone)
            return fail(BKV_ERR_STATE, "step_plan_decode: block-table changes are pending while the stream is being "
                                       "captured; make allocator calls, then any eager call, before the capture");
        (void)hipGetLastError();
        const bkv_status st = flush_tables(p, S(stream));
        if (st != BKV_OK) return st;
    }
    // Nothing pending does not mean nothing in flight: the last scatter may still run on another
    // stream (the wait is a stream operation a capture can record), and so may the plan's own last
    // upload or advance.
    bkv_status ord = wait_for_table_scatter(p, S(stream), false);
    if (ord == BKV_OK) ord = order_workspace(pl->order, S(stream));
    if (ord != BKV_OK) return ord;
    AttnBatch b{};
    b.n = pl->n;
    AttnArgs a;
    a.n_q_head = pl->n_q_head;
    a.q = q_dev;
    a.gate = gate_dev;
    a.gate_seq_stride = gate_seq_stride;
    a.gate_head_stride = gate_head_stride;
    a.scale = scale;
    a.out = out_dev;
    a.new_k = k_new_dev;
    a.new_v = v_new_dev;
    a.ws_o = pl->part_o;
    a.ws_ml = pl->part_ml;
    a.timed = false;
    a.desc = &pl->dev->b;
    a.desc_grid = pl->grid;
    BKV_HIP(launch_decode_attn(p, layer, b, a, S(stream)));
    return BKV_OK;
}

bkv_status bkv_step_plan_advance(bkv_step_plan* pl, void* stream) {
    if (!pl) return fail(BKV_ERR_INVALID, "step_plan_advance: NULL plan");
    const bkv_status ord = order_workspace(pl->order, S(stream));
    if (ord != BKV_OK) return ord;
    BKV_HIP(launch_step_advance(pl->dev, pl->lim, pl->pool->g.page_cells, S(stream)));
    return BKV_OK;
}

bkv_status bkv_step_plan_state(bkv_step_plan* pl, void* stream, int64_t* pos_out, uint32_t* steps_out,
                               int32_t* status_out) {
    if (!pl) return fail(BKV_ERR_INVALID, "step_plan_state: NULL plan");
    StepDesc host;
    const bkv_status ord = order_workspace(pl->order, S(stream));
    if (ord != BKV_OK) return ord;
    const bkv_status ws = wait_stream(S(stream), default_timeout_ms(), "the stream of a step plan");
    if (ws != BKV_OK) return ws;
    BKV_HIP(hipMemcpy(&host, pl->dev, sizeof(host), hipMemcpyDeviceToHost));
    if (pos_out)
        for (int i = 0; i < pl->n; ++i) pos_out[i] = host.b.pos[i];
    if (steps_out) *steps_out = host.steps;
    if (status_out) *status_out = host.status;
    return BKV_OK;
}

bkv_status bkv_decode_attn_select(bkv_pool* p, int32_t layer, int32_t n, const int32_t* seqs,
                                  const int64_t* pos, int32_t n_q_head, const float* q_dev,
                                  const float* gate_dev, int64_t gate_seq_stride,
                                  int64_t gate_head_stride, float scale, const uint32_t* ids_dev,
                                  int64_t id_stride, const uint32_t* counts_dev, int32_t max_ids,
                                  float* out_dev, void* stream) {
    return decode_attn_common(p, layer, n, seqs, pos, n_q_head, q_dev, gate_dev, gate_seq_stride,
                              gate_head_stride, scale, ids_dev, id_stride, counts_dev, max_ids, true,
                              out_dev, stream);
}

// ---- prefill attention ---------------------------------------------------------------------
bkv_status bkv_prefill_attn(bkv_pool* p, int32_t layer, int32_t n_seqs, const int32_t* seqs,
                            const int64_t* pos0, const int32_t* n_tokens, int32_t n_q_head,
                            const float* q_dev, const float* gate_dev, int64_t gate_tok_stride,
                            int64_t gate_head_stride, float scale, float* out_dev, void* stream) {
    if (!p) return fail(BKV_ERR_INVALID, "prefill_attn: NULL pool");
    if (layer < 0 || layer >= p->g.n_layers)
        return fail(BKV_ERR_RANGE, sfmt("prefill_attn: layer %lld is outside 0..%lld", layer, p->g.n_layers));
    if (n_seqs < 0 || n_seqs > BKV_MAX_BATCH)
        return fail(BKV_ERR_INVALID, sfmt("prefill_attn: %lld chunks in one call; the limit is %lld", n_seqs,
                                          BKV_MAX_BATCH));
    if (n_q_head <= 0 || n_q_head % p->g.n_kv != 0)
        return fail(BKV_ERR_INVALID, sfmt("prefill_attn: %lld q heads over %lld kv heads (need a whole "
                                          "group)", n_q_head, p->g.n_kv));
    if (p->g.hd != 256 || p->g.page_cells != 16)
        return fail(BKV_ERR_INVALID, "prefill_attn is built for head_dim 256 and 16-cell pages");
    if (n_seqs > 0 && (!seqs || !pos0 || !n_tokens))
        return fail(BKV_ERR_INVALID, "prefill_attn: NULL sequence / position / token-count array");
    PrefillBatch b{};
    const int64_t group = n_q_head / p->g.n_kv;
    int64_t total = 0, wgs = 0;
    for (int i = 0; i < n_seqs; ++i) {
        if (!p->alloc->seq_valid(seqs[i]))
            return fail(BKV_ERR_RANGE, sfmt("prefill_attn: sequence %lld is not live", seqs[i]));
        if (n_tokens[i] < 0 || pos0[i] < 0)
            return fail(BKV_ERR_RANGE, sfmt("prefill_attn: chunk %lld has pos0 %lld, n_tokens %lld", i, pos0[i],
                                            n_tokens[i]));
        const int64_t end = pos0[i] + n_tokens[i];
        if (end > p->alloc->seq_capacity(seqs[i]))
            return fail(BKV_ERR_RANGE, sfmt("prefill_attn: positions up to %lld of sequence %lld are outside "
                                            "its %lld addressable cells", end - 1, seqs[i],
                                            p->alloc->seq_capacity(seqs[i])));
        if (n_tokens[i] > 0 && !p->alloc->seq_resident(seqs[i], end))
            return fail(BKV_ERR_STATE, sfmt("prefill_attn: sequence %lld has swapped-out pages below "
                                            "position %lld", seqs[i], end - 1));
        b.row[i] = seqs[i];
        b.pos0[i] = (int32_t)pos0[i];
        b.n_tok[i] = n_tokens[i];
        b.src0[i] = (int32_t)total;
        total += n_tokens[i];
        wgs += ((int64_t)n_tokens[i] * group + 63) / 64 * p->g.n_kv;  // as 64-row work-groups
        if (total > ((int64_t)1 << 24) || wgs > ((int64_t)1 << 30))
            return fail(BKV_ERR_INVALID, "prefill_attn: more than 2^24 tokens in one call");
    }
    b.n = n_seqs;
    const int64_t rows_per_wg = prefill_rows_per_wg(p->g.layout, wgs, p->n_cu);
    wgs = 0;
    for (int i = 0; i < n_seqs; ++i) {
        b.wg_base[i] = (int32_t)wgs;
        wgs += ((int64_t)n_tokens[i] * group + rows_per_wg - 1) / rows_per_wg * p->g.n_kv;
    }
    b.wg_base[n_seqs] = (int32_t)wgs;
    bkv_status st = need_device(p);
    if (st != BKV_OK) return st;
    if (total == 0) return BKV_OK;
    if (!q_dev || !out_dev || !aligned16(q_dev) || !aligned16(out_dev))
        return fail(BKV_ERR_INVALID, "prefill_attn: q/out device pointers must be non-NULL and 16-byte "
                                     "aligned");
    st = flush_tables(p, S(stream));
    if (st != BKV_OK) return st;
    AttnArgs a;
    a.n_q_head = n_q_head;
    a.q = q_dev;
    a.gate = gate_dev;
    a.gate_seq_stride = gate_tok_stride;
    a.gate_head_stride = gate_head_stride;
    a.scale = scale;
    a.out = out_dev;
    BKV_HIP(launch_prefill_attn(p, layer, b, a, (int32_t)rows_per_wg, S(stream)));
    return BKV_OK;
}

// ---- block selection ---------------------------------------------------------------------
static bkv_status select_common_checks(bkv_pool* p, const char* what, int32_t n, const int64_t* pos,
                                       int32_t topk_blocks, const uint32_t* ids_dev, int64_t id_stride,
                                       const uint32_t* counts_dev, int32_t max_ids) {
    if (!p) return fail(BKV_ERR_INVALID, std::string(what) + ": NULL pool");
    if (n < 0 || n > BKV_MAX_BATCH)
        return fail(BKV_ERR_INVALID, std::string(what) + sfmt(": %lld lists in one call; the limit is "
                                                              "%lld", n, BKV_MAX_BATCH));
    if (n > 0 && !pos) return fail(BKV_ERR_INVALID, std::string(what) + ": NULL pos");
    if (topk_blocks <= 0 || topk_blocks > select_max_topk())
        return fail(BKV_ERR_INVALID, std::string(what) + sfmt(": topk_blocks %lld is outside 1..%lld",
                                                              topk_blocks, select_max_topk()));
    if (max_ids <= 0 || id_stride < max_ids)
        return fail(BKV_ERR_INVALID, std::string(what) + sfmt(": max_ids %lld / id_stride %lld (need "
                                                              "0 < max_ids <= id_stride)", max_ids,
                                                              id_stride));
    for (int i = 0; i < n; ++i)
        if (pos[i] < 0 || pos[i] > 0x7fffffff)
            return fail(BKV_ERR_RANGE, std::string(what) + sfmt(": position %lld of list %lld", pos[i], i));
    bkv_status st = need_device(p);
    if (st != BKV_OK) return st;
    if (n > 0 && (!ids_dev || !counts_dev || ((uintptr_t)ids_dev & 3u) || ((uintptr_t)counts_dev & 3u)))
        return fail(BKV_ERR_INVALID, std::string(what) + ": ids/counts device pointers must be "
                                                         "non-NULL and 4-byte aligned");
    return BKV_OK;
}

bkv_status bkv_idx_pool(bkv_pool* p, float* pooled_dev, int32_t max_blocks, float* tail_dev,
                        const float* idx_k_dev, int64_t pos0, int32_t tokens, const float* gamma_dev,
                        float eps, const float* rope_table_dev, int32_t n_rot, int32_t max_pos,
                        int32_t idx_dim, void* stream) {
    if (!p) return fail(BKV_ERR_INVALID, "idx_pool: NULL pool");
    if (idx_dim <= 0 || idx_dim > select_max_idx_dim() || idx_dim % 2 != 0)
        return fail(BKV_ERR_INVALID, sfmt("idx_pool: idx_dim %lld is outside 2..%lld", idx_dim,
                                          select_max_idx_dim()));
    if (n_rot <= 0 || n_rot % 2 != 0 || n_rot > idx_dim)
        return fail(BKV_ERR_INVALID, sfmt("idx_pool: n_rot %lld must be even and within 2..%lld", n_rot,
                                          idx_dim));
    if (max_pos <= 0) return fail(BKV_ERR_INVALID, "idx_pool: an empty rotary table");
    if (tokens < 0 || pos0 < 0 || pos0 + tokens > 0x7fffffff)
        return fail(BKV_ERR_RANGE, sfmt("idx_pool: %lld tokens at position %lld", tokens, pos0));
    if (!(eps >= 0.0f)) return fail(BKV_ERR_INVALID, "idx_pool: eps must be >= 0");
    const int64_t blocks_after = (pos0 + tokens) / 4;
    if (blocks_after > max_blocks)
        return fail(BKV_ERR_RANGE, sfmt("idx_pool would write pooled rows up to %lld but the buffer "
                                        "holds %lld", blocks_after, max_blocks));
    bkv_status st = need_device(p);
    if (st != BKV_OK) return st;
    if (tokens == 0) return BKV_OK;
    if (!pooled_dev || !tail_dev || !idx_k_dev || !gamma_dev || !rope_table_dev)
        return fail(BKV_ERR_INVALID, "idx_pool: NULL device pointer");
    BKV_HIP(launch_idx_pool(p, idx_k_dev, tail_dev, gamma_dev, rope_table_dev, pooled_dev, (int32_t)pos0, tokens,
                            idx_dim, 4, n_rot, max_pos, eps, S(stream)));
    return BKV_OK;
}

bkv_status bkv_topk_blocks(bkv_pool* p, int32_t n, const int64_t* pos, const float* scores_dev,
                           int32_t n_blocks, int32_t topk_blocks, int32_t dense, uint32_t* ids_dev,
                           int64_t id_stride, uint32_t* counts_dev, int32_t max_ids, void* stream) {
    bkv_status st = select_common_checks(p, "topk_blocks", n, pos, topk_blocks, ids_dev, id_stride,
                                         counts_dev, max_ids);
    if (st != BKV_OK) return st;
    if (n_blocks < 0) return fail(BKV_ERR_INVALID, sfmt("topk_blocks: n_blocks %lld", n_blocks));
    if (n == 0) return BKV_OK;
    if (!dense && n_blocks > 0 && (!scores_dev || ((uintptr_t)scores_dev & 3u)))
        return fail(BKV_ERR_INVALID, "topk_blocks: scores device pointer must be non-NULL and "
                                     "4-byte aligned");
    SelectBatch b{};
    b.n = n;
    for (int i = 0; i < n; ++i) {
        b.pos[i] = (int32_t)pos[i];
        b.n_blocks[i] = n_blocks;
    }
    BKV_HIP(launch_topk_blocks(p, b, scores_dev, false, n_blocks, topk_blocks, 4, dense != 0, ids_dev,
                               id_stride, counts_dev, max_ids, S(stream)));
    return BKV_OK;
}

bkv_status bkv_select_blocks(bkv_pool* p, int32_t n, const int64_t* pos, const float* idx_q_dev,
                             const float* const* pooled_dev, const int32_t* n_blocks,
                             int32_t idx_n_head, int32_t idx_dim, int32_t topk_blocks,
                             uint32_t* ids_dev, int64_t id_stride, uint32_t* counts_dev,
                             int32_t max_ids, void* stream) {
    bkv_status st = select_common_checks(p, "select_blocks", n, pos, topk_blocks, ids_dev, id_stride,
                                         counts_dev, max_ids);
    if (st != BKV_OK) return st;
    if (idx_n_head <= 0 || idx_n_head > select_max_idx_head() || idx_dim <= 0 ||
        idx_dim > select_max_idx_dim())
        return fail(BKV_ERR_INVALID, sfmt("select_blocks: %lld indexer heads of %lld values (limits "
                                          "%lld, %lld)", idx_n_head, idx_dim, select_max_idx_head(),
                                          select_max_idx_dim()));
    if (n == 0) return BKV_OK;
    if (!n_blocks || !pooled_dev || !idx_q_dev || ((uintptr_t)idx_q_dev & 3u))
        return fail(BKV_ERR_INVALID, "select_blocks: NULL n_blocks / pooled / idx_q");
    SelectBatch b{};
    b.n = n;
    int32_t max_blocks = 0;
    for (int i = 0; i < n; ++i) {
        if (n_blocks[i] < 0 || (n_blocks[i] > 0 && (!pooled_dev[i] || ((uintptr_t)pooled_dev[i] & 3u))))
            return fail(BKV_ERR_INVALID, sfmt("select_blocks: list %lld has %lld blocks and a NULL or "
                                              "misaligned pooled pointer", i, n_blocks[i]));
        b.pos[i] = (int32_t)pos[i];
        b.n_blocks[i] = n_blocks[i];
        b.pooled[i] = pooled_dev[i];
        max_blocks = std::max(max_blocks, n_blocks[i]);
    }
    const uint64_t stride = ((uint64_t)std::max(max_blocks, 1) + 63u) & ~(uint64_t)63u;
    const uint64_t need = stride * (uint64_t)n;
    if (need > p->sel_scores_cap) {
        // grow the score workspace; earlier launches may still read the old one
        BKV_HIP(hipDeviceSynchronize());
        if (p->sel_scores) BKV_HIP(hipFree(p->sel_scores));
        p->sel_scores = nullptr;
        p->sel_scores_cap = 0;
        const uint64_t cap = std::max<uint64_t>(need, (uint64_t)BKV_MAX_BATCH * 8192u);
        BKV_HIP(hipMalloc(reinterpret_cast<void**>(&p->sel_scores), cap * sizeof(double)));
        p->sel_scores_cap = cap;
    }
    const bkv_status ws = order_workspace(p->sel_ws, S(stream));
    if (ws != BKV_OK) return ws;
    if (max_blocks > 0)
        BKV_HIP(launch_idx_score(p, b, idx_q_dev, idx_n_head, idx_dim, 4, p->sel_scores, (int64_t)stride,
                                 max_blocks, S(stream)));
    BKV_HIP(launch_topk_blocks(p, b, p->sel_scores, true, (int64_t)stride, topk_blocks, 4, false, ids_dev,
                               id_stride, counts_dev, max_ids, S(stream)));
    return BKV_OK;
}

// ---- page copy -------------------------------------------------------------------------
bkv_status bkv_page_copy(bkv_pool* p, const bkv_page_pair* pairs, int32_t n_pairs, void* stream) {
    if (!p) return fail(BKV_ERR_INVALID, "page_copy: NULL pool");
    if (n_pairs < 0 || (n_pairs > 0 && !pairs))
        return fail(BKV_ERR_INVALID, "page_copy: bad pair list");
    std::vector<int32_t> dsts;
    dsts.reserve((size_t)n_pairs);
    for (int i = 0; i < n_pairs; ++i) {
        if (pairs[i].src < 0 || pairs[i].src >= p->g.n_pages || pairs[i].dst < 0 ||
            pairs[i].dst >= p->g.n_pages)
            return fail(BKV_ERR_RANGE, sfmt("page_copy: pair %lld (%lld -> %lld) is outside the "
                                            "%lld-page pool", i, pairs[i].src, pairs[i].dst,
                                            p->g.n_pages));
        dsts.push_back(pairs[i].dst);
    }
    std::sort(dsts.begin(), dsts.end());
    if (std::adjacent_find(dsts.begin(), dsts.end()) != dsts.end())
        return fail(BKV_ERR_INVALID, "page_copy: a destination page appears twice");
    bkv_status st = need_device(p);
    if (st != BKV_OK) return st;
    st = wait_for_tier_moves(p, S(stream));
    if (st != BKV_OK) return st;
    const int32_t per_launch = (int32_t)(ParamRing::kSlotBytes / sizeof(bkv_page_pair));
    for (int32_t at = 0; at < n_pairs; at += per_launch) {
        const int32_t n = std::min(per_launch, n_pairs - at);
        void* dev;
        int slot;
        st = ring_upload(p, pairs + at, (size_t)n * sizeof(bkv_page_pair), S(stream), &dev, &slot);
        if (st != BKV_OK) return st;
        BKV_HIP(launch_page_copy(p, static_cast<const bkv_page_pair*>(dev), n, S(stream)));
        st = ring_done(p, slot, S(stream));
        if (st != BKV_OK) return st;
    }
    return BKV_OK;
}

// ---- swap --------------------------------------------------------------------------------
uint64_t bkv_swap_page_bytes(const bkv_pool* p) {
    if (!p) return 0;
    return (p->g.k_page_bytes + p->g.v_page_bytes) * (uint64_t)p->g.n_layers;
}

bkv_status bkv_host_alloc(bkv_pool* p, uint64_t bytes, void** host_out) {
    bkv_status st = need_device(p);
    if (st != BKV_OK) return st;
    if (!host_out || bytes == 0) return fail(BKV_ERR_INVALID, "host_alloc: bad argument");
    void* h = nullptr;
    const hipError_t e = hipHostMalloc(&h, bytes, hipHostMallocDefault);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return fail(BKV_ERR_NOMEM, sfmt("host_alloc: hipHostMalloc of %lld bytes of pinned host "
                                        "memory failed: ", (long long)bytes) +
                                       hipGetErrorString(e));
    }
    *host_out = h;
    return BKV_OK;
}

bkv_status bkv_host_free(bkv_pool* p, void* host) {
    bkv_status st = need_device(p);
    if (st != BKV_OK) return st;
    if (!host) return BKV_OK;
    BKV_HIP(hipHostFree(host));
    return BKV_OK;
}

static bkv_status swap_move(bkv_pool* p, const int32_t* pages, int32_t n, uint8_t* host, bool out,
                            hipStream_t stream) {
    const uint64_t slab = bkv_swap_page_bytes(p);
    const int32_t per_chunk = (int32_t)std::min<uint64_t>(
        std::min<uint64_t>(p->stage.bytes / slab, ParamRing::kSlotBytes / 4),
        (uint64_t)(65535 / (p->g.n_layers * 2)));
    if (per_chunk <= 0) return fail(BKV_ERR_INVALID, "swap: a page slab exceeds the staging buffer");
    for (int32_t at = 0; at < n; at += per_chunk) {
        const int32_t m = std::min(per_chunk, n - at);
        SwapStage& sg = p->stage;
        const int h = sg.next;
        sg.next = (sg.next + 1) % SwapStage::kHalves;
        uint8_t* hostp = host + (uint64_t)at * slab;
        void* pages_dev;
        int slot;
        if (out) {
            // the half is free once its last transfer (side stream) and its last unpack kernel (a
            // swap-in, possibly on another caller stream) are over
            BKV_HIP(hipStreamWaitEvent(stream, sg.ev_side[h], 0));
            BKV_HIP(hipStreamWaitEvent(stream, sg.ev_stream[h], 0));
            bkv_status st = ring_upload(p, pages + at, (size_t)m * 4, stream, &pages_dev, &slot);
            if (st != BKV_OK) return st;
            BKV_HIP(launch_page_stage(p, static_cast<const int32_t*>(pages_dev), m, sg.dev[h], 1,
                                      stream));
            st = ring_done(p, slot, stream);
            if (st != BKV_OK) return st;
            BKV_HIP(hipEventRecord(sg.ev_stream[h], stream));
            BKV_HIP(hipStreamWaitEvent(p->side, sg.ev_stream[h], 0));
            BKV_HIP(hipMemcpyAsync(hostp, sg.dev[h], (uint64_t)m * slab, hipMemcpyDeviceToHost,
                                   p->side));
            BKV_HIP(hipEventRecord(sg.ev_side[h], p->side));
        } else {
            BKV_HIP(hipStreamWaitEvent(p->side, sg.ev_stream[h], 0));
            BKV_HIP(hipMemcpyAsync(sg.dev[h], hostp, (uint64_t)m * slab, hipMemcpyHostToDevice,
                                   p->side));
            BKV_HIP(hipEventRecord(sg.ev_side[h], p->side));
            BKV_HIP(hipStreamWaitEvent(stream, sg.ev_side[h], 0));
            bkv_status st = ring_upload(p, pages + at, (size_t)m * 4, stream, &pages_dev, &slot);
            if (st != BKV_OK) return st;
            BKV_HIP(launch_page_stage(p, static_cast<const int32_t*>(pages_dev), m, sg.dev[h], 0,
                                      stream));
            st = ring_done(p, slot, stream);
            if (st != BKV_OK) return st;
            BKV_HIP(hipEventRecord(sg.ev_stream[h], stream));
        }
    }
    BKV_HIP(hipEventRecord(p->side_done, p->side));
    p->side_used = true;
    return BKV_OK;
}

static bkv_status check_pages(const bkv_pool* p, const int32_t* pages, int32_t n, const void* host,
                              const char* who) {
    if (n < 0 || (n > 0 && (!pages || !host)))
        return fail(BKV_ERR_INVALID, std::string(who) + ": bad page list or host buffer");
    for (int i = 0; i < n; ++i)
        if (pages[i] < 0 || pages[i] >= p->g.n_pages)
            return fail(BKV_ERR_RANGE, std::string(who) + sfmt(": page %lld (entry %lld) is outside "
                                                               "the %lld-page pool", pages[i], i,
                                                               p->g.n_pages));
    return BKV_OK;
}

bkv_status bkv_swap_out(bkv_pool* p, const int32_t* pages, int32_t n, void* pinned_host,
                        void* stream) {
    if (!p) return fail(BKV_ERR_INVALID, "swap_out: NULL pool");
    bkv_status st = check_pages(p, pages, n, pinned_host, "swap_out");
    if (st != BKV_OK) return st;
    st = need_device(p);
    if (st != BKV_OK) return st;
    if (n == 0) return BKV_OK;
    st = wait_for_tier_moves(p, S(stream));
    if (st != BKV_OK) return st;
    return swap_move(p, pages, n, static_cast<uint8_t*>(pinned_host), true, S(stream));
}

bkv_status bkv_swap_in(bkv_pool* p, const int32_t* pages, int32_t n, const void* pinned_host,
                       void* stream) {
    if (!p) return fail(BKV_ERR_INVALID, "swap_in: NULL pool");
    bkv_status st = check_pages(p, pages, n, pinned_host, "swap_in");
    if (st != BKV_OK) return st;
    std::vector<int32_t> sorted(pages, pages + n);
    std::sort(sorted.begin(), sorted.end());
    if (std::adjacent_find(sorted.begin(), sorted.end()) != sorted.end())
        return fail(BKV_ERR_INVALID, "swap_in: a destination page appears twice");
    st = need_device(p);
    if (st != BKV_OK) return st;
    if (n == 0) return BKV_OK;
    st = wait_for_tier_moves(p, S(stream));
    if (st != BKV_OK) return st;
    return swap_move(p, pages, n, const_cast<uint8_t*>(static_cast<const uint8_t*>(pinned_host)),
                     false, S(stream));
}

static bkv_status wait_side(bkv_pool* p, int64_t timeout_ms) {
    return wait_stream(p->side, timeout_ms, "the pool's side stream (page transfers to or from host memory)");
}

bkv_status bkv_swap_wait_for(bkv_pool* p, int64_t timeout_ms) {
    bkv_status st = need_device(p);
    if (st != BKV_OK) return st;
    return wait_side(p, timeout_ms);
}

bkv_status bkv_swap_wait(bkv_pool* p) { return bkv_swap_wait_for(p, default_timeout_ms()); }

bkv_status bkv_stream_wait(void* stream, int64_t timeout_ms) {
    return wait_stream(S(stream), timeout_ms, "a caller stream");
}

bkv_status bkv_wait_options(int64_t timeout_ms, int64_t poll_us) {
    if (timeout_ms == 0) return fail(BKV_ERR_INVALID, "wait_options: a default timeout of 0 ms would fail every wait; "
                                                      "negative = no deadline");
    if (poll_us < 0) return fail(BKV_ERR_INVALID, "wait_options: the spin window cannot be negative");
    g_wait_timeout_ms.store(timeout_ms, std::memory_order_relaxed);
    g_wait_poll_us.store(poll_us, std::memory_order_relaxed);
    return BKV_OK;
}

bkv_status bkv_wait_options_get(int64_t* timeout_ms, int64_t* poll_us) {
    if (timeout_ms) *timeout_ms = g_wait_timeout_ms.load(std::memory_order_relaxed);
    if (poll_us) *poll_us = g_wait_poll_us.load(std::memory_order_relaxed);
    return BKV_OK;
}

bkv_status bkv_swap_fence(bkv_pool* p, void* stream) {
    bkv_status st = need_device(p);
    if (st != BKV_OK) return st;
    if (p->side_used) BKV_HIP(hipStreamWaitEvent(S(stream), p->side_done, 0));
    return BKV_OK;
}

bkv_status bkv_seq_evict(bkv_pool* p, int32_t seq, int32_t lp0, int32_t n, void* pinned_host,
                         void* stream) {
    if (!p) return fail(BKV_ERR_INVALID, "seq_evict: NULL pool");
    if (n > 0 && !pinned_host) return fail(BKV_ERR_INVALID, "seq_evict: NULL host buffer");
    if (!p->host_only) {
        // The device copy reads the pages through ids taken before they are freed.
        bkv_status st = flush_tables(p, S(stream));
        if (st != BKV_OK) return st;
    }
    std::vector<int32_t> phys;
    std::string err;
    const AllocErr e = p->alloc->seq_detach_pages(seq, lp0, n, phys, err);
    if (e != AllocErr::Ok) return from_alloc(e, err);
    if (p->host_only || n == 0) return BKV_OK;
    return swap_move(p, phys.data(), n, static_cast<uint8_t*>(pinned_host), true, S(stream));
}

bkv_status bkv_seq_restore(bkv_pool* p, int32_t seq, int32_t lp0, int32_t n,
                           const void* pinned_host, void* stream) {
    if (!p) return fail(BKV_ERR_INVALID, "seq_restore: NULL pool");
    if (n > 0 && !pinned_host) return fail(BKV_ERR_INVALID, "seq_restore: NULL host buffer");
    std::vector<int32_t> phys;
    std::string err;
    const AllocErr e = p->alloc->seq_attach_pages(seq, lp0, n, phys, err);
    if (e != AllocErr::Ok) return from_alloc(e, err);
    if (p->host_only || n == 0) return BKV_OK;
    bkv_status st = swap_move(p, phys.data(), n,
                              const_cast<uint8_t*>(static_cast<const uint8_t*>(pinned_host)), false,
                              S(stream));
    if (st != BKV_OK) return st;
    return flush_tables(p, S(stream));
}

// ---- lower tiers of the prefix tree ------------------------------------------------------
// The bytes behind the tree's bookkeeping.  Transfers between the device and the host arena go
// through the swap path on the side stream (runs of consecutive slots as one transfer); the file
// is written from the arena and read into a pinned bounce buffer of two halves.  Work enqueued by
// later calls waits for `tiers.done` (wait_for_tier_moves).  A host-only pool keeps the books only.
static bkv_status tier_io_failed(bkv_pool* p, const char* what) {
    const std::string msg = std::string("prefix tiers: ") + what + " failed: " + std::strerror(errno) +
                            "; the cached prefixes were dropped";
    p->prefix->clear();
    return fail(BKV_ERR_STATE, msg);
}

// Device <-> arena transfers of moves[i..j), all of one kind: independent of each other, so they
// go in slot order, every run of consecutive slots as one transfer.
static bkv_status tier_arena_transfers(bkv_pool* p, std::vector<TierMove> run, bool out) {
    const uint64_t slab = bkv_swap_page_bytes(p);
    // A slot can be filled twice in one list (its first tenant was dropped again to make room):
    // the last move into a slot is the one whose bytes stay.
    std::stable_sort(run.begin(), run.end(),
                     [](const TierMove& a, const TierMove& b) { return a.host_slot < b.host_slot; });
    {
        size_t kept = 0;
        for (size_t i = 0; i < run.size(); ++i)
            if (i + 1 == run.size() || run[i + 1].host_slot != run[i].host_slot) run[kept++] = run[i];
        run.resize(kept);
    }
    std::vector<int32_t> pages;
    for (size_t i = 0; i < run.size();) {
        size_t j = i + 1;
        while (j < run.size() && run[j].host_slot == run[j - 1].host_slot + 1) ++j;
        pages.clear();
        for (size_t k = i; k < j; ++k) pages.push_back(run[k].page);
        const bkv_status st = swap_move(p, pages.data(), (int32_t)pages.size(),
                                        p->tiers.host + (uint64_t)run[i].host_slot * slab, out, p->side);
        if (st != BKV_OK) return st;
        i = j;
    }
    return BKV_OK;
}

static bkv_status run_tier_moves(bkv_pool* p, const std::vector<TierMove>& moves) {
    if (moves.empty() || p->host_only) return BKV_OK;
    TierStore& ts = p->tiers;
    const uint64_t slab = bkv_swap_page_bytes(p);
    // The list is an eviction (arena -> file and device -> arena moves, interleaved victim by
    // victim) followed by a promotion (arena -> device, then file -> device).  The eviction's moves
    // are queued and go out in batches -- first the queued file writes (gathered over consecutive
    // file slots), then the queued copies (merged over consecutive arena slots) -- which keeps the
    // list's order wherever it matters: a slot's write before the copy that refills it.  Only a
    // write that reads a slot a queued copy fills needs the batch out and finished first.
    size_t n_evict = 0;
    while (n_evict < moves.size() && (moves[n_evict].kind == TierMove::DeviceToHost ||
                                      moves[n_evict].kind == TierMove::HostToDisk))
        ++n_evict;
    if (n_evict > 0) {
        // the pages that leave were written on streams this call does not know, and the arena slots
        // that go on to the file may still be on their way in
        BKV_HIP(hipDeviceSynchronize());
        std::vector<TierMove> writes, copies;
        std::unordered_map<int32_t, int> copy_slots;
        const auto flush = [&](bool wait) -> bkv_status {
            for (size_t i = 0; i < writes.size();) {
                size_t j = i + 1;
                while (j < writes.size() && j - i < 512 && writes[j].disk_slot == writes[j - 1].disk_slot + 1) ++j;
                std::vector<iovec> iov(j - i);
                for (size_t k = i; k < j; ++k) {
                    iov[k - i].iov_base = ts.host + (uint64_t)writes[k].host_slot * slab;
                    iov[k - i].iov_len = slab;
                }
                const ssize_t w = ::pwritev(ts.fd, iov.data(), (int)iov.size(),
                                            (off_t)((uint64_t)writes[i].disk_slot * slab));
                if (w < 0) return tier_io_failed(p, "a write to the disk tier");
                // a short write: the slots it did not finish go out one by one
                for (size_t k = i + (size_t)w / slab; k < j; ++k)
                    if (::pwrite(ts.fd, ts.host + (uint64_t)writes[k].host_slot * slab, slab,
                                 (off_t)((uint64_t)writes[k].disk_slot * slab)) != (ssize_t)slab)
                        return tier_io_failed(p, "a write to the disk tier");
                i = j;
            }
            writes.clear();
            if (!copies.empty()) {
                const bkv_status st = tier_arena_transfers(p, copies, true);
                if (st != BKV_OK) return st;
                copies.clear();
                copy_slots.clear();
                if (wait) {
                    const bkv_status ws = wait_side(p, default_timeout_ms());
                    if (ws != BKV_OK) return ws;
                }
            }
            return BKV_OK;
        };
        for (size_t i = 0; i < n_evict; ++i) {
            const TierMove& m = moves[i];
            if (m.kind == TierMove::HostToDisk) {
                if (copy_slots.count(m.host_slot)) {
                    const bkv_status st = flush(true);
                    if (st != BKV_OK) return st;
                }
                writes.push_back(m);
            } else {
                copies.push_back(m);
                copy_slots[m.host_slot] = 1;
            }
        }
        const bkv_status st = flush(false);
        if (st != BKV_OK) return st;
    }
    // ---- promotion ---------------------------------------------------------------------------
    std::vector<TierMove> from_host, from_disk;
    for (size_t i = n_evict; i < moves.size(); ++i)
        (moves[i].kind == TierMove::HostToDevice ? from_host : from_disk).push_back(moves[i]);
    if (!from_host.empty()) {
        const bkv_status st = tier_arena_transfers(p, from_host, false);
        if (st != BKV_OK) return st;
    }
    if (!from_disk.empty()) {
        // file -> one half of the bounce buffer -> device, runs of consecutive file slots as one
        // read; the next read overlaps the previous half's upload
        std::sort(from_disk.begin(), from_disk.end(),
                  [](const TierMove& a, const TierMove& b) { return a.disk_slot < b.disk_slot; });
        // an earlier call's upload may still be reading the bounce buffer
        {
            const bkv_status ws = wait_side(p, default_timeout_ms());
            if (ws != BKV_OK) return ws;
        }
        bool half_in_flight[2] = {false, false};
        int half = 0;
        std::vector<int32_t> pages;
        for (size_t i = 0; i < from_disk.size();) {
            size_t j = i + 1;
            while (j < from_disk.size() && j - i < (size_t)ts.bounce_slots &&
                   from_disk[j].disk_slot == from_disk[j - 1].disk_slot + 1)
                ++j;
            uint8_t* buf = ts.bounce + (uint64_t)half * ts.bounce_slots * slab;
            if (half_in_flight[half]) {
                const bkv_status ws = wait_side(p, default_timeout_ms());
                if (ws != BKV_OK) return ws;
                half_in_flight[0] = half_in_flight[1] = false;
            }
            const uint64_t bytes = (uint64_t)(j - i) * slab;
            if (::pread(ts.fd, buf, bytes, (off_t)((uint64_t)from_disk[i].disk_slot * slab)) != (ssize_t)bytes)
                return tier_io_failed(p, "a read from the disk tier");
            pages.clear();
            for (size_t k = i; k < j; ++k) pages.push_back(from_disk[k].page);
            const bkv_status st = swap_move(p, pages.data(), (int32_t)pages.size(), buf, false, p->side);
            if (st != BKV_OK) return st;
            half_in_flight[half] = true;
            half ^= 1;
            i = j;
        }
    }
    BKV_HIP(hipEventRecord(ts.done, p->side));
    ts.pending = true;
    return BKV_OK;
}

bkv_status bkv_prefix_tiers(bkv_pool* p, uint64_t host_bytes, const char* disk_path, uint64_t disk_bytes) {
    if (!p) return fail(BKV_ERR_INVALID, "prefix_tiers: NULL pool");
    const uint64_t slab = bkv_swap_page_bytes(p);
    const uint64_t cap = (uint64_t)1 << 30;
    const uint64_t host_slots = std::min(host_bytes / slab, cap);
    const uint64_t disk_slots = disk_path ? std::min(disk_bytes / slab, cap) : 0;
    if (disk_slots > 0 && host_slots == 0)
        return fail(BKV_ERR_INVALID, "prefix_tiers: the disk tier is fed from the host tier, which has no room "
                                     "for a single page");
    TierStore& ts = p->tiers;
    // what the lower tiers hold now goes first
    p->prefix->set_tiers(0, 0);
    if (!p->host_only) {
        const bkv_status ws = wait_side(p, default_timeout_ms());
        if (ws != BKV_OK) return ws;
        if (ts.host) BKV_HIP(hipHostFree(ts.host));
        if (ts.bounce) BKV_HIP(hipHostFree(ts.bounce));
    }
    ts.host = ts.bounce = nullptr;
    ts.pending = false;
    if (ts.fd >= 0) (void)::close(ts.fd);
    ts.fd = -1;
    ts.host_slots = ts.disk_slots = 0;
    if (host_slots == 0) return BKV_OK;
    if (!p->host_only) {
        void* mem = nullptr;
        if (hipHostMalloc(&mem, host_slots * slab, hipHostMallocDefault) != hipSuccess) {
            (void)hipGetLastError();
            return fail(BKV_ERR_NOMEM, sfmt("prefix_tiers: cannot pin %lld bytes of host memory",
                                            (long long)(host_slots * slab)));
        }
        ts.host = static_cast<uint8_t*>(mem);
        if (!ts.done) BKV_HIP(hipEventCreateWithFlags(&ts.done, hipEventDisableTiming));
    }
    if (disk_slots > 0) {
        ts.fd = ::open(disk_path, O_RDWR | O_CREAT | O_TRUNC, 0600);
        if (ts.fd < 0)
            return fail(BKV_ERR_INVALID, std::string("prefix_tiers: cannot open ") + disk_path + ": " +
                                             std::strerror(errno));
        if (!p->host_only) {
            void* mem = nullptr;
            // two halves of up to 4 MiB
            ts.bounce_slots = (int32_t)std::max<uint64_t>(1, std::min<uint64_t>(((uint64_t)4 << 20) / slab, disk_slots));
            if (hipHostMalloc(&mem, 2 * (uint64_t)ts.bounce_slots * slab, hipHostMallocDefault) != hipSuccess) {
                (void)hipGetLastError();
                return fail(BKV_ERR_NOMEM, "prefix_tiers: cannot pin the bounce buffer of the disk tier");
            }
            ts.bounce = static_cast<uint8_t*>(mem);
        }
    }
    ts.host_slots = (int32_t)host_slots;
    ts.disk_slots = (int32_t)disk_slots;
    p->prefix->set_tiers(ts.host_slots, ts.disk_slots);
    return BKV_OK;
}

bkv_status bkv_prefix_tier_stats(const bkv_pool* p, int32_t* nodes_by_tier, uint64_t* moved) {
    if (!p) return fail(BKV_ERR_INVALID, "prefix_tier_stats: NULL pool");
    const TierStats& st = p->prefix->stats();
    if (nodes_by_tier)
        for (int t = 0; t < 3; ++t) nodes_by_tier[t] = st.nodes[t];
    if (moved) {
        moved[0] = st.to_host;
        moved[1] = st.to_disk;
        moved[2] = st.promoted;
        moved[3] = st.dropped;
    }
    return BKV_OK;
}

// ---- gather ------------------------------------------------------------------------------
bkv_status bkv_gather(bkv_pool* p, int32_t layer, int32_t seq, int64_t cell0, int64_t n,
                      float* k_out_dev, float* v_out_dev, void* stream) {
    if (!p) return fail(BKV_ERR_INVALID, "gather: NULL pool");
    if (layer < 0 || layer >= p->g.n_layers)
        return fail(BKV_ERR_RANGE, sfmt("gather: layer %lld is outside 0..%lld", layer,
                                        p->g.n_layers));
    if (!p->alloc->seq_valid(seq))
        return fail(BKV_ERR_RANGE, sfmt("gather: sequence %lld is not live", seq));
    if (cell0 < 0 || n < 0 || cell0 + n > p->alloc->seq_capacity(seq))
        return fail(BKV_ERR_RANGE, sfmt("gather: cells %lld..%lld are outside the sequence's %lld",
                                        cell0, cell0 + n, p->alloc->seq_capacity(seq)));
    if (n > 0) {
        const int32_t* row = p->alloc->seq_table(seq);
        for (int64_t c = cell0 / p->g.page_cells; c <= (cell0 + n - 1) / p->g.page_cells; ++c)
            if (row[c] < 0)
                return fail(BKV_ERR_STATE, sfmt("gather: logical page %lld is swapped out", c));
    }
    bkv_status st = need_device(p);
    if (st != BKV_OK) return st;
    if (n == 0) return BKV_OK;
    if (!k_out_dev || !v_out_dev) return fail(BKV_ERR_INVALID, "gather: NULL output");
    st = flush_tables(p, S(stream));
    if (st != BKV_OK) return st;
    BKV_HIP(launch_gather(p, layer, seq, cell0, n, k_out_dev, v_out_dev, S(stream)));
    return BKV_OK;
}

// ---- per-kernel timing ---------------------------------------------------------------
bkv_status bkv_timing_enable(bkv_pool* p, int on) {
    bkv_status st = need_device(p);
    if (st != BKV_OK) return st;
    if (!on && p->timer.on) {
        st = timer_collect(p);
        if (st != BKV_OK) return st;
    }
    p->timer.on = on != 0;
    return BKV_OK;
}

bkv_status bkv_timing_reset(bkv_pool* p) {
    bkv_status st = need_device(p);
    if (st != BKV_OK) return st;
    st = timer_collect(p);
    if (st != BKV_OK) return st;
    for (int i = 0; i < BKV_STAGE_COUNT; ++i) {
        p->timer.launches[i] = 0;
        p->timer.total_ms[i] = 0.0;
    }
    return BKV_OK;
}

bkv_status bkv_timing_read(bkv_pool* p, int stage, uint64_t* launches, double* total_ms) {
    bkv_status st = need_device(p);
    if (st != BKV_OK) return st;
    if (stage < 0 || stage >= BKV_STAGE_COUNT)
        return fail(BKV_ERR_RANGE, sfmt("timing_read: stage %lld is outside 0..%lld", stage,
                                        BKV_STAGE_COUNT));
    st = timer_collect(p);
    if (st != BKV_OK) return st;
    if (launches) *launches = p->timer.launches[stage];
    if (total_ms) *total_ms = p->timer.total_ms[stage];
    return BKV_OK;
}

}  // extern "C"
