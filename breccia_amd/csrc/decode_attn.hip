// Paged decode attention for gfx950: what the split-K kernels of decode_attn_mfma.hip share -- the
// cut of a batch into work-groups, the merge kernel, the launch.  Together they replace the
// reference's four dispatches (scores -> softmax -> split apply -> reduce:
// crates/breccia-kernels/shaders/qsa_attn_scores_small.comp, ops_softmax.comp,
// qsa_attn_apply_split.comp, qsa_attn_apply_reduce.comp) and must agree with its f64 CPU attend
// (crates/breccia-kernels/src/qsa/cpu.rs:197-246).
//
// Shape of the work: for one (sequence, kv head) every K row and V row is read once and used by
// all q heads of the group -- an HBM-bound stream.  A work-group of four waves owns one (entry, kv
// head, page range); a wave owns whole pages (16 cells); the four waves' running (m, l, O) are
// folded in LDS and written as one partial per work-group; the merge kernel combines the page
// ranges of a head and applies sigmoid(gate).
#include <atomic>

#include "decode_attn_common.hpp"

namespace bkv {

namespace {

struct MergeParams {
    AttnBatch b;
    const AttnBatch* bd;  // DESC: the batch is read from this device-resident copy
    const float* part_o;
    const float* part_ml;
    const float* gate;
    float* out;
    int64_t gate_seq_stride, gate_head_stride;
    int32_t n_kv, n_q, group;
    uint32_t inv_group16;  // small_divisor_inverse(group)
};

constexpr int kMergeGroups = 16;   // waves of a work-group; wave g sums splits g, g + 16, ...
constexpr int kMergeInFlight = 8;  // partial rows (16 bytes a lane) a wave requests per round

// One work-group per (entry, q head): 16 waves.  Lane d4 of wave g owns head-dim elements
// 4 d4 .. 4 d4 + 3 of splits g, g + 16, ...; it requests its first 8 partial rows straight away,
// and only then are the per-split (m, l) pairs staged in LDS and the maximum agreed, so the two
// round trips to memory overlap.  One round covers 128 splits.
template <bool DESC>
__global__ __launch_bounds__(64 * kMergeGroups) void decode_attn_merge_kernel(const MergeParams P) {
    constexpr int kMaxStaged = 1024;
    constexpr int kThreads = 64 * kMergeGroups;
    __shared__ float sm[kMaxStaged];
    __shared__ float sl[kMaxStaged];
    __shared__ __attribute__((aligned(16))) float red[kMergeGroups][kHd];
    __shared__ float red_l[kMergeGroups];
    __shared__ float wave_max[kMergeGroups];
    // grid (q heads, entries): no division at the head of a kernel that is all latency
    const int e = blockIdx.y;
    const int h = blockIdx.x;
    const int kvh = small_div(h, P.inv_group16);
    const int hl = h - kvh * P.group;
    int splits, base;
    if constexpr (DESC) {
        const batch_desc_ptr D = (batch_desc_ptr)(uintptr_t)P.bd;
        splits = D->splits[e];
        base = D->wg_base[e];
    } else {
        splits = P.b.splits[e];
        base = P.b.wg_base[e];
    }
    const int wg0 = base + kvh;
    const int d4 = threadIdx.x & 63;
    const int g = threadIdx.x >> 6;
    const size_t ostride = (size_t)P.n_kv * P.group * kHd;  // floats between consecutive splits
    const float* po = P.part_o + ((size_t)wg0 * P.group + hl) * kHd + 4 * d4;
    const float* pml = P.part_ml + ((size_t)wg0 * P.group + hl) * 2;
    const size_t mlstride = (size_t)P.n_kv * P.group * 2;

    f4 v[kMergeInFlight];
#pragma unroll
    for (int u = 0; u < kMergeInFlight; ++u) {
        const int s = g + u * kMergeGroups;
        v[u] = s < splits ? *reinterpret_cast<const f4*>(po + (size_t)s * ostride) : f4{0.0f, 0.0f, 0.0f, 0.0f};
    }
    // the gate of the element this thread writes at the end is requested with the partial rows, not after
    // the sums (a trip to memory at the tail of a kernel that is all latency)
    float gt = 0.0f;
    if (P.gate && threadIdx.x < kHd)
        gt = P.gate[(size_t)e * P.gate_seq_stride + (size_t)h * P.gate_head_stride + threadIdx.x];
    // stage (m, l) and agree on the maximum: per-thread max over its splits, wave reduction,
    // then one LDS slot per wave (a serial scan over the splits would cost a dependent LDS
    // round trip per split)
    float my_m = -INFINITY;
    for (int s = threadIdx.x; s < splits; s += kThreads) {
        const float ms = pml[(size_t)s * mlstride];
        if (s < kMaxStaged) {
            sm[s] = ms;
            sl[s] = pml[(size_t)s * mlstride + 1];
        }
        my_m = fmaxf(my_m, ms);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) my_m = fmaxf(my_m, __shfl_xor(my_m, off, 64));
    if ((threadIdx.x & 63) == 0) wave_max[g] = my_m;
    __syncthreads();
    const auto m_of = [&](int s) { return s < kMaxStaged ? sm[s] : pml[(size_t)s * mlstride]; };
    const auto l_of = [&](int s) { return s < kMaxStaged ? sl[s] : pml[(size_t)s * mlstride + 1]; };
    float mx = wave_max[0];
#pragma unroll
    for (int w = 1; w < kMergeGroups; ++w) mx = fmaxf(mx, wave_max[w]);
    f4 acc = f4{0.0f, 0.0f, 0.0f, 0.0f};
    float lsum = 0.0f;
#pragma unroll
    for (int u = 0; u < kMergeInFlight; ++u) {
        const int s = g + u * kMergeGroups;
        if (s < splits) {
            const float ms = m_of(s);
            const float f = ms == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(ms - mx);
            acc += v[u] * f;
            lsum = fmaf(f, l_of(s), lsum);
        }
    }
    // further rounds for split lists beyond 128
    for (int s0 = g + kMergeInFlight * kMergeGroups; s0 < splits; s0 += kMergeInFlight * kMergeGroups) {
#pragma unroll
        for (int u = 0; u < kMergeInFlight; ++u) {
            const int s = s0 + u * kMergeGroups;
            v[u] = s < splits ? *reinterpret_cast<const f4*>(po + (size_t)s * ostride) : f4{0.0f, 0.0f, 0.0f, 0.0f};
        }
#pragma unroll
        for (int u = 0; u < kMergeInFlight; ++u) {
            const int s = s0 + u * kMergeGroups;
            if (s < splits) {
                const float ms = m_of(s);
                const float f = ms == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(ms - mx);
                acc += v[u] * f;
                lsum = fmaf(f, l_of(s), lsum);
            }
        }
    }
    *reinterpret_cast<f4*>(&red[g][4 * d4]) = acc;
    if (d4 == 0) red_l[g] = lsum;
    __syncthreads();
    // the first four waves fold the 16 rows: thread d sums element d
    if (threadIdx.x >= kHd) return;
    const int d = threadIdx.x;
    float r = 0.0f, lt = 0.0f;
#pragma unroll
    for (int k = 0; k < kMergeGroups; ++k) {
        r += red[k][d];
        lt += red_l[k];
    }
    r = lt > 0.0f ? r / lt : 0.0f;
    if (P.gate) {
        // sigmoid in the overflow-free form of the reference (qsa/cpu.rs:84-91)
        float sg;
        if (gt >= 0.0f) {
            sg = 1.0f / (1.0f + expf(-gt));
        } else {
            const float t = expf(gt);
            sg = t / (1.0f + t);
        }
        r *= sg;
    }
    P.out[((size_t)e * P.n_q + h) * kHd + d] = r;
}

}  // namespace

// The limits a plan of this pool geometry works under.  The partial-result workspace holds
// max_wgs x 8 head rows and a work-group writes `group` of them.
AttnPlanLimits attn_plan_limits(int32_t n_cu, int32_t max_wgs, int32_t n_kv, int32_t group) {
    AttnPlanLimits lim;
    lim.per_page = n_kv;
    lim.gran = kWaves;
    // All work-groups should be resident at once (one generation): a handful of left-over
    // work-groups would run alone after the rest and double the kernel's time.  Two work-groups
    // fit a compute unit (registers and LDS of the kernels).
    lim.target = (n_cu > 0 ? n_cu : 256) * 2;
    lim.max_wgs = group > 8 ? (int32_t)((int64_t)max_wgs * 8 / group) : max_wgs;
    return lim;
}

int32_t plan_attn(const bkv_pool* p, int32_t n_q_head, AttnBatch& b, int32_t sel_groups, int32_t max_wgs) {
    const AttnPlanLimits lim =
        attn_plan_limits(p->n_cu, max_wgs > 0 ? max_wgs : p->max_wgs, p->g.n_kv, n_q_head / p->g.n_kv);
    return plan_attn_ranges(lim, kPage, sel_groups, b);
}

// ---- partial results without an allocation -----------------------------------------------------
// For callers that may not allocate device memory (a stream under capture, a tight serving loop):
// the split-K partials of bkv_decode_attn_static live in this array, one copy per GPU, held from
// the moment the library is loaded until the process ends.  Host code never uses the array's name
// as an address: each device's copy has its own address, looked up once per device below.
struct AttnStaticScratch {
    float o[(size_t)kStaticWgs * 8 * kHd];
    float ml[(size_t)kStaticWgs * 8 * 2];
};
static __device__ __align__(256) unsigned char scratch[sizeof(AttnStaticScratch)];

constexpr int kMaxDevices = 64;
// One address per device, looked up once; pools may be created from several threads at once, so the
// table is atomic (two threads that race on one device store the same address).
static std::atomic<void*> g_scratch_ptr[kMaxDevices];

// Makes `device` current for the lookup (every GPU holds its own copy of the array at its own
// address) and restores the caller's device afterwards.
hipError_t attn_static_scratch_init(int device) {
    if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
    if (g_scratch_ptr[device].load(std::memory_order_acquire)) return hipSuccess;
    int current = -1;
    hipError_t e = hipGetDevice(&current);
    if (e != hipSuccess) return e;
    if (current != device) {
        e = hipSetDevice(device);
        if (e != hipSuccess) return e;
    }
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (current != device) {
        const hipError_t back = hipSetDevice(current);
        if (e == hipSuccess) e = back;
    }
    if (e != hipSuccess) return e;
    g_scratch_ptr[device].store(ptr, std::memory_order_release);
    return hipSuccess;
}

bool attn_static_scratch(int device, float** o, float** ml) {
    if (device < 0 || device >= kMaxDevices) return false;
    void* ptr = g_scratch_ptr[device].load(std::memory_order_acquire);
    if (!ptr) return false;
    AttnStaticScratch* s = static_cast<AttnStaticScratch*>(ptr);
    *o = s->o;
    *ml = s->ml;
    return true;
}

hipError_t launch_decode_attn(bkv_pool* p, int32_t layer, const AttnBatch& b, const AttnArgs& a,
                              hipStream_t stream) {
    const int32_t n_kv = p->g.n_kv;
    const int32_t group = a.n_q_head / n_kv;
    AttnKernelParams kp;
    kp.b = b;
    kp.bd = a.desc;
    kp.kpool = p->k_layer[(size_t)layer];
    kp.vpool = p->v_layer[(size_t)layer];
    kp.tables = p->table_dev;
    kp.q = a.q;
    kp.part_o = a.ws_o ? a.ws_o : p->part_o;
    kp.part_ml = a.ws_ml ? a.ws_ml : p->part_ml;
    kp.max_pages_per_seq = p->desc.max_pages_per_seq;
    kp.n_kv = n_kv;
    kp.n_q = a.n_q_head;
    kp.group = group;
    kp.inv_kv16 = small_divisor_inverse(n_kv);
    kp.scale_log2e = a.scale * kLog2e;
    kp.ids = a.ids;
    kp.counts = a.counts;
    kp.id_stride = a.id_stride;
    kp.max_ids = a.max_ids;
    kp.new_k = a.new_k;
    kp.new_v = a.new_v;
    kp.kpool_w = p->k_layer[(size_t)layer];
    kp.vpool_w = p->v_layer[(size_t)layer];
    const bool sel = a.ids != nullptr;
    const bool step = a.new_k != nullptr;
    const int32_t total = a.desc ? a.desc_grid : b.wg_base[b.n];
    // one work-group per unit, every head of the kv head in it; while the pool times its kernels,
    // the events ride on the dispatch
    hipEvent_t ev_start = nullptr, ev_stop = nullptr;
    if (a.timed) (void)timer_dispatch_events(p, BKV_STAGE_ATTN_SPLIT, &ev_start, &ev_stop);
    hipError_t err = launch_decode_attn_mfma(kp, p->g.layout, step, sel, total, stream, ev_start, ev_stop);
    if (err != hipSuccess) return err;
    MergeParams mp;
    mp.b = b;
    mp.bd = a.desc;
    mp.part_o = kp.part_o;
    mp.part_ml = kp.part_ml;
    mp.gate = a.gate;
    mp.out = a.out;
    mp.gate_seq_stride = a.gate_seq_stride;
    mp.gate_head_stride = a.gate_head_stride;
    mp.n_kv = n_kv;
    mp.n_q = a.n_q_head;
    mp.group = group;
    mp.inv_group16 = small_divisor_inverse(group);
    const dim3 mgrid((unsigned)a.n_q_head, (unsigned)b.n), mblock(64 * kMergeGroups);
    if (a.desc)
        hipLaunchKernelGGL(decode_attn_merge_kernel<true>, mgrid, mblock, 0, stream, mp);
    else if (a.timed)
        launch_staged(p, BKV_STAGE_ATTN_MERGE, decode_attn_merge_kernel<false>, mgrid, mblock, 0, stream, mp);
    else
        hipLaunchKernelGGL(decode_attn_merge_kernel<false>, mgrid, mblock, 0, stream, mp);
    return hipGetLastError();
}

// ---- a decode step that re-plans itself on the device ------------------------------------------
// One wave, lane i = entry i: every entry moves on by one cell and the batch is cut again with the
// arithmetic of plan_attn_ranges (attn_plan.hpp) -- the sums and the running offsets as wave
// reductions -- so that a replayed launch reads what a fresh call would have been given, bit for
// bit.  An entry that would pass the last cell the plan was checked for stops the advance
// (nothing moves, the status word says so).
__device__ __forceinline__ long long wave_sum(long long v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}
__device__ __forceinline__ long long wave_max(long long v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const long long o = __shfl_xor(v, off, 64);
        v = o > v ? o : v;
    }
    return v;
}
__global__ __launch_bounds__(64) void step_advance_kernel(StepDesc* d, AttnPlanLimits lim, int32_t page_cells) {
    static_assert(kMaxBatch <= 64, "one lane per entry");
    const int i = threadIdx.x;
    const int n = d->b.n;
    const bool live = i < n;
    int pos = live ? d->b.pos[i] : 0;
    const bool past = live && pos + 1 > d->horizon[i];
    if (__builtin_amdgcn_ballot_w64(past) != 0) {
        if (i == 0) d->status = 1;
        return;
    }
    pos += 1;
    const long long per_page = lim.per_page, gran = lim.gran;
    const long long min_total = (long long)n * per_page;
    long long target = lim.target < lim.max_wgs ? lim.target : lim.max_wgs;
    if (target < min_total) target = min_total;
    const long long pages = live ? pos / page_cells + 1 : 0;
    const long long total_pages = wave_sum(pages), max_pages = wave_max(pages);
    long long pps = (total_pages * per_page + target - 1) / target;
    pps = (pps + gran - 1) / gran * gran;
    if (pps < gran) pps = gran;
    long long my_splits = 0, each = gran, total = 0;
    for (;;) {
        if (live) {
            const long long splits = (pages + pps - 1) / pps;
            // even the ranges out inside the entry, keeping whole groups of `gran` pages
            each = (pages + splits - 1) / splits;
            each = (each + gran - 1) / gran * gran;
            my_splits = (pages + each - 1) / each;
        }
        total = wave_sum(my_splits * per_page);
        if (total <= target || pps >= max_pages) break;
        pps += gran;
    }
    // first work-group of every entry: the sum over the entries before it
    long long incl = my_splits * per_page;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const long long o = __shfl_up(incl, off, 64);
        if (i >= off) incl += o;
    }
    if (live) {
        d->b.pos[i] = pos;
        d->b.splits[i] = (int32_t)my_splits;
        d->b.pps[i] = (int32_t)each;
        d->b.wg_base[i] = (int32_t)(incl - my_splits * per_page);
    }
    if (i == 0) {
        d->b.wg_base[n] = (int32_t)total;
        d->steps += 1u;
    }
}

hipError_t launch_step_advance(StepDesc* d, const AttnPlanLimits& lim, int32_t page_cells, hipStream_t stream) {
    hipLaunchKernelGGL(step_advance_kernel, dim3(1), dim3(64), 0, stream, d, lim, page_cells);
    return hipGetLastError();
}

}  // namespace bkv
