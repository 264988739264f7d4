// Paged decode attention for gfx950: one split-K online-softmax kernel and one merge
// kernel.  Replaces the reference's four dispatches (scores -> softmax -> split
// apply -> reduce: crates/breccia-kernels/shaders/qsa_attn_scores_small.comp,
// ops_softmax.comp, qsa_attn_apply_split.comp, qsa_attn_apply_reduce.comp) and must
// agree with its f64 CPU attend (crates/breccia-kernels/src/qsa/cpu.rs:197-246).
//
// Shape of the work: for one (sequence, kv head) every 512-byte f16 K row and V row
// is read once and used by all q heads of the group -- a GEMV-shaped, HBM-bound
// stream (about `group` flop per byte), so there is no MFMA here; the design goal
// is to keep the VALU almost purely on FMAs while 16-byte row loads stay in flight.
//
// Work-group = 4 waves, all on one (entry, kv head, head chunk, page range).  A wave
// owns whole pages (16 cells).  Lane l of a wave owns 8 consecutive head-dim elements
// (l % 32) of the rows with parity l / 32, so one 16-byte load per lane covers two
// rows and a page is 8 loads of K and 8 of V.  q (HG heads x 8 elements) and the
// output accumulators (HG x 8) live in registers.
//   scores: per row HG partial dots per lane -> transposed through LDS so that each
//           lane finishes one (row, head) sum (no butterfly of selects)
//   softmax: running max per head in base 2, per-lane partial denominators, the
//           max is agreed across the 8..16 lanes of a head with three or four shuffles
//   P.V   : probabilities go back through LDS (broadcast reads), FMAs straight from
//           the f16 V registers
// Partial (m, l, O) of the four waves are merged in LDS and written per work-group;
// the merge kernel combines the splits and applies sigmoid(gate).
#include "bkv_internal.hpp"
#include "f16_rule.hpp"
#include "lane_groups.hpp"

namespace bkv {

namespace {

constexpr int kHd = 256;      // head_dim the kernel is built for
constexpr int kPage = 16;     // cells per page
constexpr int kWaves = 4;
constexpr int kBlock = 64 * kWaves;
constexpr float kLog2e = 1.4426950408889634f;

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));

struct AttnKernelParams {
    AttnBatch b;
    const uint8_t* kpool;
    const uint8_t* vpool;
    const int32_t* tables;
    const float* q;
    float* part_o;
    float* part_ml;
    int32_t max_pages_per_seq;
    int32_t n_kv, n_q, group, n_hc;
    float scale_log2e;
    // selection lists (decode_attn_kernel<..., true> only): entry e attends the 4-cell blocks
    // ids[e * id_stride + 0 .. min(counts[e], max_ids))
    const uint32_t* ids;
    const uint32_t* counts;
    int64_t id_stride;
    int32_t max_ids;
    // fused decode step (decode_attn_kernel<..., STEP = true> only): the K/V row of cell pos of
    // entry e comes from new_k / new_v [n][n_kv][head_dim] f32 and is stored into the pool on the way
    const float* new_k;
    const float* new_v;
    uint8_t* kpool_w;
    uint8_t* vpool_w;
};

__device__ __forceinline__ void wave_lds_sync() {
    // LDS operations of one wave execute in order; this only stops the compiler from
    // moving a lane's reads above other lanes' writes.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <int CTRL>
__device__ __forceinline__ float dpp(float v) {
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
constexpr int kDppXor1 = 0xB1;  // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;  // quad_perm [2,3,0,1]

constexpr int kDppRor8 = 0x128;  // row_ror:8 == lane ^ 8 inside a row of 16

__device__ __forceinline__ float xor_max(float v, int mask) {
    return fmaxf(v, __shfl_xor(v, mask, 64));
}
__device__ __forceinline__ float xor_sum(float v, int mask) { return v + __shfl_xor(v, mask, 64); }

// Lane exchanges across 16 and 32 lanes with the gfx950 permlane swaps, written as inline
// assembly because this toolchain's builtin returns its first result twice.
//   v_permlane16_swap a, b : a.row1 <-> b.row0 and a.row3 <-> b.row2 (rows of 16 lanes)
//   v_permlane32_swap a, b : a.lanes[32..63] <-> b.lanes[0..31]
// The s_nop covers the wait states a VALU write needs before a permlane reads it.  The asm
// statements are not `volatile`: a volatile asm counts as a possible memory write and would
// turn the uniform block-table loads behind it into vector loads.
__device__ __forceinline__ void permlane16_swap(float& a, float& b) {
    asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ void permlane32_swap(float& a, float& b) {
    asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}
// Swapping a register with a copy of itself puts both partners' values side by side.
__device__ __forceinline__ void both16(float v, float& a, float& b) {
    a = v;
    b = v;
    permlane16_swap(a, b);
}
__device__ __forceinline__ void both32(float v, float& a, float& b) {
    a = v;
    b = v;
    permlane32_swap(a, b);
}
// max / sum over the lanes that differ in bits 3, 4 and 5 (the 8 lanes holding one head)
__device__ __forceinline__ float max_bits345(float v) {
    float a, b;
    v = fmaxf(v, dpp<kDppRor8>(v));
    both16(v, a, b);
    v = fmaxf(a, b);
    both32(v, a, b);
    return fmaxf(a, b);
}
__device__ __forceinline__ float sum_bits345(float v) {
    float a, b;
    v += dpp<kDppRor8>(v);
    both16(v, a, b);
    v = a + b;
    both32(v, a, b);
    return a + b;
}

// f16 -> f32 as a separate conversion.  Folding the conversion into the multiply-add
// (v_fma_mix_f32) would save the convert, but on gfx950 that packed-encoding instruction
// issues from one wave at a time, while plain v_fma_f32 from two waves of a SIMD overlap
// (measured: ~4.8 vs ~2.5 cycles per wave-instruction); with every converted element
// feeding HG multiply-adds the separate convert is the cheaper form.  The empty asm keeps
// the compiler from folding it back.
__device__ __forceinline__ float widen(_Float16 h) {
    float f = (float)h;
    asm("" : "+v"(f));
    return f;
}

// ---- row buffers -------------------------------------------------------------------
// A lane owns 8 consecutive head-dim elements (dl = lane % 32) of the rows with parity
// hw = lane / 32, i.e. rows 2i + hw, i = 0..7, of a 16-cell page.  A RowBuf holds that
// lane's share of the 8 rows in registers for one of the three row encodings:
//   kRowF16   256 f16                          one 16-byte load per row
//   kRowQ8    8 x [f32 scale][32 x i8]         (reference q8_0 V, shaders/qsa_kv_append.comp:
//             38-44; value = i8 * scale, qsa_attn_apply.comp:70-77): 8 code bytes + scale
//   kRowI8H   [256 x i8][8 x f16 scale]        8 code bytes + the block's f16 scale
// K/V rows are read exactly once per kernel: nontemporal loads keep them from displacing
// the block tables, q and the split partials in the caches.
constexpr int kRowF16 = 0, kRowQ8 = 1, kRowI8H = 2;
typedef unsigned v4u __attribute__((ext_vector_type(4)));
typedef unsigned v2u __attribute__((ext_vector_type(2)));

__host__ __device__ constexpr int row_bytes_of(int enc) {
    return enc == kRowF16 ? kHd * 2 : enc == kRowQ8 ? (kHd / 32) * 36 : kHd + (kHd / 32) * 2;
}

template <int ENC>
struct RowBuf;

template <>
struct RowBuf<kRowF16> {
    half8 r[8];
    // base = first byte of a run of rows of one kv head; the lane's row of pair `ia` in that
    // run goes to register group i
    __device__ __forceinline__ void load(const uint8_t* base, int ia, int i, int lane) {
        r[i] = __builtin_bit_cast(
            half8, __builtin_nontemporal_load(reinterpret_cast<const v4u*>(base) + ia * 64 + lane));
    }
    __device__ __forceinline__ float elem(int i, int j) const { return widen(r[i][j]); }
    static constexpr bool kScaled = false;
    __device__ __forceinline__ float scale(int) const { return 1.0f; }
    __device__ __forceinline__ void zero(int i) {
#pragma unroll
        for (int j = 0; j < 8; ++j) r[i][j] = (_Float16)0.0f;
    }
};

__device__ __forceinline__ float code_to_float(v2u w, int j) {
    // sign-extending byte convert (one SDWA instruction per element)
    const int sh = (j & 3) * 8;
    return (float)(int)(int8_t)((j < 4 ? w.x : w.y) >> sh);
}

template <>
struct RowBuf<kRowQ8> {
    v2u code[8];
    float sc[8];
    __device__ __forceinline__ void load(const uint8_t* base, int ia, int i, int lane) {
        const int row = 2 * ia + (lane >> 5), dl = lane & 31;
        const uint8_t* blk = base + row * row_bytes_of(kRowQ8) + (dl >> 2) * 36;
        sc[i] = __builtin_nontemporal_load(reinterpret_cast<const float*>(blk));
        const unsigned* c = reinterpret_cast<const unsigned*>(blk + 4 + (dl & 3) * 8);
        code[i].x = __builtin_nontemporal_load(c);
        code[i].y = __builtin_nontemporal_load(c + 1);
    }
    __device__ __forceinline__ float elem(int i, int j) const { return code_to_float(code[i], j); }
    static constexpr bool kScaled = true;
    __device__ __forceinline__ float scale(int i) const { return sc[i]; }
    __device__ __forceinline__ void zero(int i) {
        code[i].x = code[i].y = 0u;
        sc[i] = 0.0f;
    }
};

template <>
struct RowBuf<kRowI8H> {
    v2u code[8];
    unsigned short sc[8];
    __device__ __forceinline__ void load(const uint8_t* base, int ia, int i, int lane) {
        const int row = 2 * ia + (lane >> 5), dl = lane & 31;
        const uint8_t* rp = base + row * row_bytes_of(kRowI8H);
        code[i] = __builtin_nontemporal_load(reinterpret_cast<const v2u*>(rp + dl * 8));
        sc[i] = __builtin_nontemporal_load(
            reinterpret_cast<const unsigned short*>(rp + kHd + (dl >> 2) * 2));
    }
    __device__ __forceinline__ float elem(int i, int j) const { return code_to_float(code[i], j); }
    static constexpr bool kScaled = true;
    // f16 scale under the cache's load rule (exponent field 0 reads as zero)
    __device__ __forceinline__ float scale(int i) const {
        const unsigned h = sc[i];
        const float f = (float)__builtin_bit_cast(_Float16, sc[i]);
        return (h & 0x7c00u) == 0 ? 0.0f : f;
    }
    __device__ __forceinline__ void zero(int i) {
        code[i].x = code[i].y = 0u;
        sc[i] = 0;
    }
};

// Where the 16 rows of one loop iteration live.  Dense: one page (one run of 16 rows).
// Selection: four selected blocks of four cells (crates/breccia-kernels/src/qsa/cpu.rs:
// 248-257: block b covers cells 4b..4b+3), each a run of 4 rows inside some page; `id` keeps
// the block ids for the causal test, 0xffffffff for a slot past the end of the list.
template <bool SEL>
struct RowRuns {
    const uint8_t* k[SEL ? 4 : 1];
    const uint8_t* v[SEL ? 4 : 1];
    uint32_t id[SEL ? 4 : 1];
};

// cell 4*id + r of a selected block is attended iff it is not past the query's position
// (shaders/qsa_attn_scores_small.comp: `cell > pos` is a dead slot)
__device__ __forceinline__ bool block_cell_live(uint32_t id, int r, int pos) {
    return id < 0x40000000u && id * 4u + (uint32_t)r <= (uint32_t)pos;
}

// HG = q heads carried by one wave (8 or 4); KENC / VENC = row encodings of the K and V pools;
// SEL = attend the cells of a per-entry list of selected blocks instead of every cell 0..=pos.
// STEP = the decode step in one launch: the row of cell pos is taken from the caller's f32 K/V
// (stored under the cache's f16 rule, exactly what the append kernel stores) and written to
// the pool by the wave that owns the last page, so no append launch precedes the attention.
template <int HG, int KENC, int VENC, bool SEL, bool STEP = false>
__global__ __launch_bounds__(kBlock, HG == 8 ? 2 : 3) void decode_attn_kernel(const AttnKernelParams P) {
    constexpr int HQ = HG / 4;           // float4 groups of heads
    constexpr int NB = HG / 4;           // score batches per page (8 float4 slots each)
    constexpr int RP = 8 / NB;           // row pairs per batch
    // xs: per wave 8 slots x 64 lanes of float4 = 8 KiB; reused for the final merge.
    __shared__ f4 xs[kWaves][8 * 64];
    __shared__ __attribute__((aligned(16))) float ps[kWaves][kPage][HG];
    __shared__ __attribute__((aligned(16))) float alphas[kWaves][HG];
    __shared__ float wave_m[kWaves][HG];
    __shared__ float wave_l[kWaves][HG];

    // ---- which (entry, kv head, head chunk, page range) ---------------------------
    // A unit is (entry, page range, kv head); its n_hc head chunks read the same K/V rows.
    // Work-groups go to the 8 XCDs round-robin by index, so the chunks of a unit are placed 8
    // indices apart: same XCD (same L2), dispatched together.  `wg` is the unit's slot in
    // the partial-result workspace, independent of the dispatch order.
    const int n_units = P.b.wg_base[P.b.n] / P.n_hc;
    const int blk = blockIdx.x / (8 * P.n_hc);
    const int rblk = blockIdx.x - blk * (8 * P.n_hc);
    const int hc = rblk >> 3;
    const int unit = blk * 8 + (rblk & 7);
    if (unit >= n_units) return;
    int e = 0;
    while (e + 1 < P.b.n && unit * P.n_hc >= P.b.wg_base[e + 1]) ++e;
    const int splits = P.b.splits[e];
    const int rem = unit - P.b.wg_base[e] / P.n_hc;
    const int split = rem / P.n_kv;
    const int kvh = rem - split * P.n_kv;
    const int wg = P.b.wg_base[e] + hc * splits * P.n_kv + rem;
    const int pos = P.b.pos[e];
    // Block-table row (and selection list) through the constant address space: neither is
    // written while this kernel runs, and constant-space loads at uniform addresses are always
    // scalar loads.
    typedef const __attribute__((address_space(4))) int32_t* table_ptr;
    typedef const __attribute__((address_space(4))) uint32_t* list_ptr;
    const table_ptr bt = (table_ptr)(uintptr_t)(P.tables + (size_t)P.b.row[e] * (size_t)P.max_pages_per_seq);
    uint32_t n_sel = 0;
    list_ptr sel = nullptr;
    if constexpr (SEL) {
        n_sel = min(((list_ptr)(uintptr_t)P.counts)[e], (uint32_t)P.max_ids);
        sel = (list_ptr)(uintptr_t)(P.ids + (size_t)e * (size_t)P.id_stride);
    }
    // loop iterations of this entry: pages, or groups of four selected blocks
    const int n_pages = SEL ? (int)((n_sel + 3u) >> 2) : pos / kPage + 1;
    const int pps = P.b.pps[e];
    const int pg0 = split * pps;
    const int pg1 = min(pg0 + pps, n_pages);

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int hw = lane >> 5;   // row parity this lane loads
    const int dl = lane & 31;   // 8-element slice of the head dim

    constexpr size_t kKHead = (size_t)kPage * row_bytes_of(KENC);  // bytes of one kv head's rows
    constexpr size_t kVHead = (size_t)kPage * row_bytes_of(VENC);
    const size_t k_page = (size_t)P.n_kv * kKHead, v_page = (size_t)P.n_kv * kVHead;
    const size_t k_head_off = (size_t)kvh * kKHead, v_head_off = (size_t)kvh * kVHead;

    // K and V rows of a page sit in registers.  Every register group is refilled with the
    // next page's row right after its last use, so each load has a whole page of work in
    // front of it and 16 row loads per wave stay in flight.
    // Row runs of iteration g.  A selected block id is clamped to the blocks at or below `pos`
    // for addressing (so that no list content can reach outside the sequence's pages); its
    // cells past `pos`, and slots past the end of the list, are masked where they are used.
    const auto locate = [&](int g, RowRuns<SEL>& rr) {
        if constexpr (SEL) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t at = (uint32_t)g * 4u + (uint32_t)j;
                const uint32_t id = sel[min(at, n_sel - 1u)];
                rr.id[j] = at < n_sel ? id : 0xffffffffu;
                const uint32_t idc = min(id, (uint32_t)pos >> 2);
                const int32_t phys = bt[idc >> 2];
                const size_t in_page = (size_t)(idc & 3u) * 4u;
                rr.k[j] = P.kpool + (size_t)phys * k_page + k_head_off + in_page * row_bytes_of(KENC);
                rr.v[j] = P.vpool + (size_t)phys * v_page + v_head_off + in_page * row_bytes_of(VENC);
            }
        } else {
            const int32_t phys = bt[g];
            rr.k[0] = P.kpool + (size_t)phys * k_page + k_head_off;
            rr.v[0] = P.vpool + (size_t)phys * v_page + v_head_off;
            rr.id[0] = 0;
        }
    };
    // row pair i of an iteration: run i/2, pair i%2 of that run (selection), or pair i of the page
    const auto load_k = [&](RowBuf<KENC>& buf, const RowRuns<SEL>& rr, int i) {
        if constexpr (SEL) buf.load(rr.k[i >> 1], i & 1, i, lane); else buf.load(rr.k[0], i, i, lane);
    };
    const auto load_v = [&](RowBuf<VENC>& buf, const RowRuns<SEL>& rr, int i) {
        if constexpr (SEL) buf.load(rr.v[i >> 1], i & 1, i, lane); else buf.load(rr.v[0], i, i, lane);
    };

    int pg = pg0 + wave;
    RowBuf<KENC> kk;
    RowBuf<VENC> vv;
    RowRuns<SEL> cur{};
    if (pg < pg1) {
        locate(pg, cur);
#pragma unroll
        for (int i = 0; i < 8; ++i) load_k(kk, cur, i);
#pragma unroll
        for (int i = 0; i < 8; ++i) load_v(vv, cur, i);
    }

    __builtin_amdgcn_sched_barrier(0);

    // ---- q slice (dead heads of a padded chunk stay zero) ---------------------------
    float q[HG][8];
#pragma unroll
    for (int h = 0; h < HG; ++h) {
        const int hl = hc * HG + h;
        if (hl < P.group) {
            const float* qp =
                P.q + ((size_t)e * P.n_q + (size_t)kvh * P.group + hl) * kHd + dl * 8;
            const float4 a = *reinterpret_cast<const float4*>(qp);
            const float4 c = *reinterpret_cast<const float4*>(qp + 4);
            q[h][0] = a.x, q[h][1] = a.y, q[h][2] = a.z, q[h][3] = a.w;
            q[h][4] = c.x, q[h][5] = c.y, q[h][6] = c.z, q[h][7] = c.w;
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) q[h][j] = 0.0f;
        }
    }

    // The first page's rows (requested above) and q travel together; both must have arrived
    // before the page loop starts: a wait for q placed inside the loop would also drain the
    // row loads that are kept in flight there on every iteration.
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0), other counters untouched
    __builtin_amdgcn_sched_barrier(0);

    float o[HG][8];
#pragma unroll
    for (int h = 0; h < HG; ++h)
#pragma unroll
        for (int j = 0; j < 8; ++j) o[h][j] = 0.0f;

    // ---- this lane's role when it finishes score sums ------------------------------
    // part: which quarter of the 32 slices it adds; slot/rhw: which float4 slot and row
    // parity; after the quad combine it keeps component `part`, i.e. one head.
    const int part = lane & 3;
    const int rslot = ((lane >> 4) << 1) | ((lane >> 2) & 1);
    const int rhw = (lane >> 3) & 1;
    const int my_head = (HG == 8) ? (lane & 7) : (lane & 3);
    const int rbase = rslot * 64 + rhw * 32 + part * 8;
    float m_run = -INFINITY;  // running max of this lane's head (base-2 logits)
    float l_run = 0.0f;       // this lane's share of the denominator

    // Two waves share a SIMD (one from each resident work-group) and the issue arbiter
    // prefers the older one whenever priorities are equal; it then finishes a third earlier
    // and leaves the younger wave alone, with nothing to overlap its latencies, for the rest
    // of the kernel (measured: 47 vs 64 us loop times on every CU).  The younger wave (odd
    // wave slot) therefore raises its priority on two of every three pages; the older one
    // never does.  Measured loop times with this duty cycle: 52.8 vs 51.3 us.
    unsigned slot;
    asm("s_getreg_b32 %0, hwreg(HW_REG_HW_ID, 0, 4)" : "=s"(slot));  // wave slot within the SIMD
    const bool younger = (slot & 1u) != 0;
    unsigned turn = 0;

    while (pg < pg1) {
        if constexpr (STEP) {
            static_assert(!STEP || (KENC == kRowF16 && VENC == kRowF16 && !SEL),
                          "the fused step is built for f16 pools and the dense selection");
            if (pg == n_pages - 1) {
                // This wave holds the page of cell pos.  Its pool row is stale (the token has
                // not been appended): replace the lane's share of it with the new row, and let
                // the lanes of that row's parity store it.
                const int r = pos & (kPage - 1);
                const size_t src = ((size_t)e * P.n_kv + (size_t)kvh) * kHd + (size_t)dl * 8;
                const float4 ka = *reinterpret_cast<const float4*>(P.new_k + src);
                const float4 kb = *reinterpret_cast<const float4*>(P.new_k + src + 4);
                const float4 va = *reinterpret_cast<const float4*>(P.new_v + src);
                const float4 vb = *reinterpret_cast<const float4*>(P.new_v + src + 4);
                v4u kw, vw;
                kw.x = f16_store_pair(ka.x, ka.y), kw.y = f16_store_pair(ka.z, ka.w);
                kw.z = f16_store_pair(kb.x, kb.y), kw.w = f16_store_pair(kb.z, kb.w);
                vw.x = f16_store_pair(va.x, va.y), vw.y = f16_store_pair(va.z, va.w);
                vw.z = f16_store_pair(vb.x, vb.y), vw.w = f16_store_pair(vb.z, vb.w);
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    if (2 * i + hw == r) {
                        kk.r[i] = __builtin_bit_cast(half8, kw);
                        vv.r[i] = __builtin_bit_cast(half8, vw);
                    }
                }
                if (hw == (r & 1) && hc == 0) {
                    const size_t off = (size_t)(cur.k[0] - P.kpool) + (size_t)r * (kHd * 2) + (size_t)dl * 16;
                    *reinterpret_cast<v4u*>(P.kpool_w + off) = kw;
                    const size_t voff = (size_t)(cur.v[0] - P.vpool) + (size_t)r * (kHd * 2) + (size_t)dl * 16;
                    *reinterpret_cast<v4u*>(P.vpool_w + voff) = vw;
                }
            }
        }
        if (younger && turn != 0)
            __builtin_amdgcn_s_setprio(2);
        else
            __builtin_amdgcn_s_setprio(0);
        turn = turn == 2 ? 0 : turn + 1;
        // The next page is fetched unconditionally (the last iteration re-reads its own
        // page): one straight-line load sequence lets the compiler count outstanding loads
        // exactly instead of draining them at a control-flow join.
        const int pg_next = pg + kWaves;
        RowRuns<SEL> nxt;
        locate(min(pg_next, pg1 - 1), nxt);

        // ---- scores: partial dots -> LDS transpose -> one (row, head) per lane ------
        float sval[NB];
#pragma unroll
        for (int bch = 0; bch < NB; ++bch) {
#pragma unroll
            for (int ip = 0; ip < RP; ++ip) {
                const int i = bch * RP + ip;
                // element-major order: HG independent accumulators between dependent FMAs
                float s[HG];
                {
                    const float k0 = kk.elem(i, 0);
#pragma unroll
                    for (int h = 0; h < HG; ++h) s[h] = k0 * q[h][0];
                }
#pragma unroll
                for (int j = 1; j < 8; ++j) {
                    const float kj = kk.elem(i, j);
#pragma unroll
                    for (int h = 0; h < HG; ++h) s[h] = fmaf(kj, q[h][j], s[h]);
                }
                if (RowBuf<KENC>::kScaled) {
                    // the lane's 8 elements lie inside one 32-element block: one scale per row
                    const float ks = kk.scale(i);
#pragma unroll
                    for (int h = 0; h < HG; ++h) s[h] *= ks;
                }
                load_k(kk, nxt, i);
#pragma unroll
                for (int hq = 0; hq < HQ; ++hq) {
                    const int slot = (HG == 8) ? (ip * 2 + hq) : i;
                    f4 w;
                    w.x = s[hq * 4 + 0], w.y = s[hq * 4 + 1], w.z = s[hq * 4 + 2],
                    w.w = s[hq * 4 + 3];
                    xs[wave][slot * 64 + lane] = w;
                }
            }
            wave_lds_sync();
            f4 acc = xs[wave][rbase + (lane & 7)];
#pragma unroll
            for (int k = 1; k < 8; ++k) acc += xs[wave][rbase + ((k + lane) & 7)];
            wave_lds_sync();
            float r0 = acc.x + dpp<kDppXor1>(acc.x);
            float r1 = acc.y + dpp<kDppXor1>(acc.y);
            float r2 = acc.z + dpp<kDppXor1>(acc.z);
            float r3 = acc.w + dpp<kDppXor1>(acc.w);
            r0 += dpp<kDppXor2>(r0);
            r1 += dpp<kDppXor2>(r1);
            r2 += dpp<kDppXor2>(r2);
            r3 += dpp<kDppXor2>(r3);
            sval[bch] = part == 0 ? r0 : part == 1 ? r1 : part == 2 ? r2 : r3;
        }

        // ---- online softmax for this lane's head -------------------------------------
        float sv[NB];
        int rowv[NB];
        float pm = -INFINITY;
#pragma unroll
        for (int bch = 0; bch < NB; ++bch) {
            const int i = (HG == 8) ? (bch * RP + (lane >> 4)) : rslot;
            rowv[bch] = 2 * i + rhw;
            bool live;
            if constexpr (SEL) {
                const int j = rowv[bch] >> 2;
                const uint32_t id = j == 0 ? cur.id[0] : j == 1 ? cur.id[1] : j == 2 ? cur.id[2] : cur.id[3];
                live = block_cell_live(id, rowv[bch] & 3, pos);
            } else {
                live = pg * kPage + rowv[bch] <= pos;
            }
            sv[bch] = live ? sval[bch] * P.scale_log2e : -INFINITY;
            pm = fmaxf(pm, sv[bch]);
        }
        if (HG == 4) pm = xor_max(pm, 4);
        pm = max_bits345(pm);
        const float m_new = fmaxf(m_run, pm);
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        const bool changed = __builtin_amdgcn_ballot_w64(m_new > m_run) != 0;
        float psum = 0.0f;
#pragma unroll
        for (int bch = 0; bch < NB; ++bch) {
            const float pv = __builtin_amdgcn_exp2f(sv[bch] - m_new);
            psum += pv;
            ps[wave][rowv[bch]][my_head] = pv;
        }
        l_run = l_run * alpha + psum;
        m_run = m_new;
        if (changed && (lane >> 3) == 0 && (HG == 8 || (lane & 4) == 0))
            alphas[wave][my_head] = alpha;
        wave_lds_sync();

        // ---- P.V ------------------------------------------------------------------
        if (changed) {
#pragma unroll
            for (int h = 0; h < HG; ++h) {
                const float a = alphas[wave][h];
#pragma unroll
                for (int j = 0; j < 8; ++j) o[h][j] *= a;
            }
        }
        // Rows that are not attended may hold anything (even NaN): make them exact zeros.
        if constexpr (SEL) {
            bool all_live = true;
#pragma unroll
            for (int j = 0; j < 4; ++j) all_live = all_live && block_cell_live(cur.id[j], 3, pos);
            if (!all_live) {
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    if (!block_cell_live(cur.id[i >> 1], 2 * (i & 1) + hw, pos)) vv.zero(i);
            }
        } else if (pg == n_pages - 1) {
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (pg * kPage + 2 * i + hw > pos) vv.zero(i);
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            float pr[HG];
            const f4* prow = reinterpret_cast<const f4*>(&ps[wave][2 * i + hw][0]);
#pragma unroll
            for (int hq = 0; hq < HQ; ++hq) {
                const f4 t = prow[hq];
                pr[hq * 4 + 0] = t.x, pr[hq * 4 + 1] = t.y, pr[hq * 4 + 2] = t.z,
                            pr[hq * 4 + 3] = t.w;
            }
            if (RowBuf<VENC>::kScaled) {
                // dequantisation folded into the probabilities: p * scale, then * code
                const float vs = vv.scale(i);
#pragma unroll
                for (int h = 0; h < HG; ++h) pr[h] *= vs;
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float vj = vv.elem(i, j);
#pragma unroll
                for (int h = 0; h < HG; ++h) o[h][j] = fmaf(vj, pr[h], o[h][j]);
            }
            load_v(vv, nxt, i);
        }
        wave_lds_sync();

        pg = pg_next;
        cur = nxt;
    }

    __builtin_amdgcn_s_setprio(0);
    // ---- wave totals ------------------------------------------------------------------
    if (HG == 4) l_run = xor_sum(l_run, 4);
    l_run = sum_bits345(l_run);
    if ((lane >> 3) == 0 && (HG == 8 || (lane & 4) == 0)) {
        wave_m[wave][my_head] = m_run;
        wave_l[wave][my_head] = l_run;
    }
    float* ow = reinterpret_cast<float*>(&xs[wave][0]);  // [HG][256] floats = 8 KiB at HG 8
    // The two half-waves hold partial sums over different rows of the same 8 elements.
    // Swapping the upper half of o[h][j] with the lower half of o[h][j+4] leaves, after one
    // add, element j's total in lanes 0-31 and element j+4's total in lanes 32-63.
#pragma unroll
    for (int h = 0; h < HG; ++h) {
        f4 t;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float a = o[h][j], c = o[h][j + 4];
            permlane32_swap(a, c);
            t[j] = a + c;
        }
        *reinterpret_cast<f4*>(ow + h * kHd + dl * 8 + hw * 4) = t;
    }
    __syncthreads();

    // ---- merge the four waves; thread = head-dim element ----------------------------
    const int d = threadIdx.x;
#pragma unroll
    for (int h = 0; h < HG; ++h) {
        float mx = wave_m[0][h];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) mx = fmaxf(mx, wave_m[w][h]);
        float acc = 0.0f, lsum = 0.0f;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            const float mw = wave_m[w][h];
            const float f = mw == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(mw - mx);
            acc = fmaf(f, reinterpret_cast<const float*>(&xs[w][0])[h * kHd + d], acc);
            lsum = fmaf(f, wave_l[w][h], lsum);
        }
        P.part_o[((size_t)wg * HG + h) * kHd + d] = acc;
        if (d == 0) {
            P.part_ml[((size_t)wg * HG + h) * 2 + 0] = mx;
            P.part_ml[((size_t)wg * HG + h) * 2 + 1] = lsum;
        }
    }
}

// ---- decode attention on the matrix cores -----------------------------------------------------
// The same split-K decomposition and the same partial-result layout as decode_attn_kernel, for
// f16 pools and head groups the 8- or 4-head VALU kernel would have to walk in several chunks
// (the reference's own 24 q / 2 kv heads = 12 per group; 32 / 2 = 16): a 16-column MFMA tile
// holds up to 16 heads of a kv head at once, every K/V row is still read once, and the VALU
// only does the softmax.  Lane (c = lane % 16, g = lane / 16) of a wave owns head c; per page:
//   S^T[cell][head] = K[cell][:] . q[head][:]          v_mfma_f32_16x16x32_f16, A = K, B = q
//   O^T[d][head]   += V^T[d][cell] . P^T[cell][head]   v_mfma_f32_16x16x32_f16, A = V regrouped
// with q and p split into a high and a low f16 part (K and V are exact f16), as in the prefill
// kernel: two MFMAs per K fragment, and for P.V one MFMA whose 32-deep contraction runs over the
// page's 16 cells twice, against p's high parts and against its low parts.  K fragment m of a lane is the 16 bytes at element 32 m + 8 g of row c; V fragments
// are the 16 bytes at element 128 h + 8 c of rows 4 g + r.  Every fragment register is
// refilled with the next page's data right after its last use.
typedef _Float16 h4m __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void split_hi_lo(float x, _Float16& hi, _Float16& lo) {
    hi = (_Float16)x;
    lo = (_Float16)(x - (float)hi);
}

constexpr int kOwStride = kHd + 4;  // floats per head in the wave-merge staging

// Shared tail of the MFMA decode kernels: wave totals, then every wave stages its scaled O in
// LDS and each wave sums one quarter of the columns over the four stagings and writes it as the
// work-group's partial (m, l, O) in the layout the merge kernel reads.
// o[h][t][r] of lane (c, g) is out[head c][128 h + 8 (4 g + r) + t].
struct MfmaFoldLds {
    float ow[kWaves][16][kOwStride];
    float wave_m[kWaves][16];
    float wave_l[kWaves][16];
};

__device__ __forceinline__ void mfma_fold_and_store(const AttnKernelParams& P, MfmaFoldLds& L, int wg, int wave,
                                                    int c, int g, f4 (&o)[2][8], float m_run, float l_run) {
    auto& ow = L.ow;
    auto& wave_m = L.wave_m;
    auto& wave_l = L.wave_l;
    l_run = sum_over_lane_groups(l_run);
    if (g == 0) {
        wave_m[wave][c] = m_run;
        wave_l[wave][c] = l_run;
    }
    __syncthreads();
    float mx = wave_m[0][c];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) mx = fmaxf(mx, wave_m[w][c]);
    float lsum = 0.0f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
        const float mw = wave_m[w][c];
        lsum = fmaf(mw == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(mw - mx), wave_l[w][c], lsum);
    }
    {
        const float f = m_run == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(m_run - mx);
        // element (h, r, t) of a lane is out[head c][128 h + 8 (4 g + r) + t]: 8 consecutive floats per (h, r)
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float* d = &ow[wave][c][128 * h + 8 * (4 * g + r)];
                *reinterpret_cast<f4*>(d) = f4{o[h][0][r] * f, o[h][1][r] * f, o[h][2][r] * f, o[h][3][r] * f};
                *reinterpret_cast<f4*>(d + 4) = f4{o[h][4][r] * f, o[h][5][r] * f, o[h][6][r] * f, o[h][7][r] * f};
            }
    }
    __syncthreads();
    // wave w sums columns [64 w, 64 w + 64): lane (c, g) takes 4 columns at 4 c of heads g, g + 4, ...
    const int hg = P.group;
#pragma unroll
    for (int hp = 0; hp < 16; hp += 4) {
        const int head = hp + g;
        if (hp >= hg) break;
        if (head < hg) {
            const int col = 64 * wave + 4 * c;
            f4 acc = *reinterpret_cast<const f4*>(&ow[0][head][col]);
#pragma unroll
            for (int w = 1; w < kWaves; ++w) acc += *reinterpret_cast<const f4*>(&ow[w][head][col]);
            *reinterpret_cast<f4*>(P.part_o + ((size_t)wg * hg + head) * kHd + col) = acc;
        }
    }
    if (wave == 0 && g == 0 && c < hg) {
        P.part_ml[((size_t)wg * hg + c) * 2 + 0] = mx;
        P.part_ml[((size_t)wg * hg + c) * 2 + 1] = lsum;
    }
}

// STEP: the row of cell pos comes from the caller's f32 K/V (stored under the f16 rule into the
// pool on the way), as in decode_attn_kernel<..., STEP = true>.
// SEL: the 16 rows of an iteration are four listed 4-cell blocks instead of a page, as in
// decode_attn_kernel<..., SEL = true> (block g supplies the V rows of lane group g, block c / 4
// the K row of lane c).
template <bool STEP, bool SEL = false>
__global__ __launch_bounds__(kBlock, 2) void decode_attn_mfma_kernel(const AttnKernelParams P) {
    static_assert(!(STEP && SEL), "the fused step attends the dense selection");
    __shared__ __attribute__((aligned(16))) MfmaFoldLds lds;

    // ---- which (entry, kv head, page range); one work-group per unit (no head chunks) --------
    const int unit = blockIdx.x;
    int e = 0;
    while (e + 1 < P.b.n && unit >= P.b.wg_base[e + 1]) ++e;
    const int rem = unit - P.b.wg_base[e];
    const int split = rem / P.n_kv;
    const int kvh = rem - split * P.n_kv;
    const int wg = unit;
    const int pos = P.b.pos[e];
    typedef const __attribute__((address_space(4))) int32_t* table_ptr;
    typedef const __attribute__((address_space(4))) uint32_t* list_ptr;
    const table_ptr bt = (table_ptr)(uintptr_t)(P.tables + (size_t)P.b.row[e] * (size_t)P.max_pages_per_seq);
    uint32_t n_sel = 0;
    list_ptr sel = nullptr;
    if constexpr (SEL) {
        n_sel = min(((list_ptr)(uintptr_t)P.counts)[e], (uint32_t)P.max_ids);
        sel = (list_ptr)(uintptr_t)(P.ids + (size_t)e * (size_t)P.id_stride);
    }
    // loop iterations of this entry: pages, or groups of four selected blocks
    const int n_pages = SEL ? (int)((n_sel + 3u) >> 2) : pos / kPage + 1;
    const int pps = P.b.pps[e];
    const int pg0 = split * pps;
    const int pg1 = min(pg0 + pps, n_pages);

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int c = lane & 15;
    const int g = lane >> 4;
    const size_t page_bytes = (size_t)P.n_kv * kPage * kHd * 2;
    const size_t head_off = (size_t)kvh * kPage * kHd * 2;

    // Row runs of iteration i (see decode_attn_kernel): a page, or four listed blocks whose ids
    // are clamped to the blocks at or below `pos` before any address is formed.
    const auto locate = [&](int i, RowRuns<SEL>& rr) {
        if constexpr (SEL) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t at = (uint32_t)i * 4u + (uint32_t)j;
                const uint32_t id = sel[min(at, n_sel - 1u)];
                rr.id[j] = at < n_sel ? id : 0xffffffffu;
                const uint32_t idc = min(id, (uint32_t)pos >> 2);
                const size_t off = (size_t)bt[idc >> 2] * page_bytes + head_off + (size_t)(idc & 3u) * 4u * (kHd * 2);
                rr.k[j] = P.kpool + off;
                rr.v[j] = P.vpool + off;
            }
        } else {
            const size_t off = (size_t)bt[i] * page_bytes + head_off;
            rr.k[0] = P.kpool + off;
            rr.v[0] = P.vpool + off;
            rr.id[0] = 0;
        }
    };
    const auto pick = [](const auto (&a)[SEL ? 4 : 1], int j) {
        if constexpr (SEL) return j == 0 ? a[0] : j == 1 ? a[1] : j == 2 ? a[2] : a[3]; else return a[0];
    };
    // this lane's K row (row c of the iteration) and the first of its four V rows (row 4 g)
    const auto k_row = [&](const RowRuns<SEL>& rr) {
        return SEL ? pick(rr.k, c >> 2) + (size_t)(c & 3) * (kHd * 2) : rr.k[0] + (size_t)c * (kHd * 2);
    };
    const auto v_rows = [&](const RowRuns<SEL>& rr) {
        return SEL ? pick(rr.v, g) : rr.v[0] + (size_t)(4 * g) * (kHd * 2);
    };
    const auto k_addr = [&](const uint8_t* row, int m) {
        return reinterpret_cast<const v4u*>(row + (size_t)(m * 32 + g * 8) * 2);
    };
    const auto v_addr = [&](const uint8_t* rows, int h, int r) {
        return reinterpret_cast<const v4u*>(rows + (size_t)r * (kHd * 2) + (size_t)(h * 128 + c * 8) * 2);
    };

    int pg = pg0 + wave;
    v4u kf[8], vf[2][4];
    RowRuns<SEL> cur{};
    if (pg < pg1) {
        locate(pg, cur);
        const uint8_t* kp = k_row(cur);
        const uint8_t* vp = v_rows(cur);
#pragma unroll
        for (int m = 0; m < 8; ++m) kf[m] = __builtin_nontemporal_load(k_addr(kp, m));
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int r = 0; r < 4; ++r) vf[h][r] = __builtin_nontemporal_load(v_addr(vp, h, r));
    }

    // ---- q fragments of head c (heads past the group stay zero) ----------------------------------
    half8 qhi[8], qlo[8];
    {
        const bool head_live = c < P.group;
        const float* qp = P.q + ((size_t)e * P.n_q + (size_t)kvh * P.group + (head_live ? c : 0)) * kHd + g * 8;
#pragma unroll
        for (int m = 0; m < 8; ++m) {
            float x[8];
            const float4 a = *reinterpret_cast<const float4*>(qp + m * 32);
            const float4 b = *reinterpret_cast<const float4*>(qp + m * 32 + 4);
            x[0] = a.x, x[1] = a.y, x[2] = a.z, x[3] = a.w;
            x[4] = b.x, x[5] = b.y, x[6] = b.z, x[7] = b.w;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                _Float16 hi, lo;
                split_hi_lo(head_live ? x[j] : 0.0f, hi, lo);
                qhi[m][j] = hi;
                qlo[m][j] = lo;
            }
        }
    }

    // O^T accumulators: o[h][t][r] = out[head c][128 h + 8 (4 g + r) + t]
    f4 o[2][8];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int t = 0; t < 8; ++t) o[h][t] = f4{0.0f, 0.0f, 0.0f, 0.0f};
    float m_run = -INFINITY;  // running max of head c (base-2 logits), equal in the 4 g lanes
    float l_run = 0.0f;       // this lane's share (its 4 cells per page) of the denominator

    while (pg < pg1) {
        // the rows of this wave's next iteration, if it has one, are requested into the fragment
        // registers as these are used up (the last iteration requests nothing)
        const int pg_next = pg + kWaves;
        const bool more = pg_next < pg1;
        RowRuns<SEL> nxt{};
        const uint8_t* kp_next = nullptr;
        const uint8_t* vp_next = nullptr;
        if (more) {
            locate(pg_next, nxt);
            kp_next = k_row(nxt);
            vp_next = v_rows(nxt);
        }

        if constexpr (STEP) {
            if (pg == n_pages - 1) {
                // This wave holds the page of cell pos; its pool row is stale.  Every lane converts
                // its slices of the new row; the lanes whose fragments are that row keep and store them.
                const int r = pos & (kPage - 1);
                const size_t here = (size_t)(cur.k[0] - P.kpool) + (size_t)r * (kHd * 2);
                const float* nk = P.new_k + ((size_t)e * P.n_kv + (size_t)kvh) * kHd;
                const float* nv = P.new_v + ((size_t)e * P.n_kv + (size_t)kvh) * kHd;
                const auto row_slice = [](const float* src) {
                    const float4 a = *reinterpret_cast<const float4*>(src);
                    const float4 b = *reinterpret_cast<const float4*>(src + 4);
                    v4u w;
                    w.x = f16_store_pair(a.x, a.y), w.y = f16_store_pair(a.z, a.w);
                    w.z = f16_store_pair(b.x, b.y), w.w = f16_store_pair(b.z, b.w);
                    return w;
                };
#pragma unroll
                for (int m = 0; m < 8; ++m) {
                    const v4u w = row_slice(nk + m * 32 + g * 8);
                    if (c == r) {
                        kf[m] = w;
                        *reinterpret_cast<v4u*>(P.kpool_w + here + (size_t)(m * 32 + g * 8) * 2) = w;
                    }
                }
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const v4u w = row_slice(nv + h * 128 + c * 8);
                    if (g == (r >> 2)) {
#pragma unroll
                        for (int rr = 0; rr < 4; ++rr)
                            if (rr == (r & 3)) vf[h][rr] = w;
                        *reinterpret_cast<v4u*>(P.vpool_w + here + (size_t)(h * 128 + c * 8) * 2) = w;
                    }
                }
            }
        }

        // ---- S^T = K . q^T: four independent accumulation chains ------------------------------
        f4 s0 = f4{0.0f, 0.0f, 0.0f, 0.0f}, s1 = s0, s2 = s0, s3 = s0;
#pragma unroll
        for (int m = 0; m < 8; m += 2) {
            const half8 ka = __builtin_bit_cast(half8, kf[m]);
            const half8 kb = __builtin_bit_cast(half8, kf[m + 1]);
            s0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka, qhi[m], s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka, qlo[m], s1, 0, 0, 0);
            s2 = __builtin_amdgcn_mfma_f32_16x16x32_f16(kb, qhi[m + 1], s2, 0, 0, 0);
            s3 = __builtin_amdgcn_mfma_f32_16x16x32_f16(kb, qlo[m + 1], s3, 0, 0, 0);
            if (more) {
                kf[m] = __builtin_nontemporal_load(k_addr(kp_next, m));
                kf[m + 1] = __builtin_nontemporal_load(k_addr(kp_next, m + 1));
            }
        }
        const f4 s = (s0 + s1) + (s2 + s3);  // s[r] = q[head c] . k[cell 4 g + r]

        // ---- online softmax of head c ---------------------------------------------------------------
        float t4[4];
        float pm = -INFINITY;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            bool live;
            if constexpr (SEL)
                live = block_cell_live(pick(cur.id, g), r, pos);
            else
                live = pg * kPage + 4 * g + r <= pos;
            t4[r] = live ? s[r] * P.scale_log2e : -INFINITY;
            pm = fmaxf(pm, t4[r]);
        }
        pm = max_over_lane_groups(pm);
        // dense: finite, every page of a range holds a live cell; a group of listed blocks may be
        // dead as a whole, and exp2(-inf - -inf) would be NaN
        const float m_new = fmaxf(m_run, pm);
        const bool none_yet = SEL && m_new == -INFINITY;
        const float alpha = none_yet ? 1.0f : __builtin_amdgcn_exp2f(m_run - m_new);
        h4m phi, plo;
        float psum = 0.0f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float p = none_yet ? 0.0f : __builtin_amdgcn_exp2f(t4[r] - m_new);
            psum += p;
            _Float16 hi, lo;
            split_hi_lo(p, hi, lo);
            phi[r] = hi;
            plo[r] = lo;
        }
        const half8 phl = half8{phi[0], phi[1], phi[2], phi[3], plo[0], plo[1], plo[2], plo[3]};
        l_run = l_run * alpha + psum;
        if (__builtin_amdgcn_ballot_w64(m_new > m_run) != 0) {
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int t = 0; t < 8; ++t) o[h][t] *= alpha;
        }
        m_run = m_new;

        // Rows that are not attended may hold anything (even NaN): make them exact zeros.
        if constexpr (SEL) {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (!block_cell_live(pick(cur.id, g), r, pos)) {
                    vf[0][r] = v4u{0u, 0u, 0u, 0u};
                    vf[1][r] = v4u{0u, 0u, 0u, 0u};
                }
        } else if (pg == n_pages - 1) {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (pg * kPage + 4 * g + r > pos) {
                    vf[0][r] = v4u{0u, 0u, 0u, 0u};
                    vf[1][r] = v4u{0u, 0u, 0u, 0u};
                }
        }

        // ---- O^T += V^T . P^T ------------------------------------------------------------------------
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const half8 v0 = __builtin_bit_cast(half8, vf[h][0]), v1 = __builtin_bit_cast(half8, vf[h][1]);
            const half8 v2 = __builtin_bit_cast(half8, vf[h][2]), v3 = __builtin_bit_cast(half8, vf[h][3]);
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                // the 32-deep MFMA runs over the page's 16 cells twice: against the high parts of p
                // and against the low parts
                const half8 vv = half8{v0[t], v1[t], v2[t], v3[t], v0[t], v1[t], v2[t], v3[t]};
                o[h][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vv, phl, o[h][t], 0, 0, 0);
            }
            if (more) {
#pragma unroll
                for (int r = 0; r < 4; ++r) vf[h][r] = __builtin_nontemporal_load(v_addr(vp_next, h, r));
            }
        }
        pg = pg_next;
        cur = nxt;
    }

    mfma_fold_and_store(P, lds, wg, wave, c, g, o, m_run, l_run);
}

// ---- decode attention on the matrix cores, int8 rows with f16 block scales ---------------------
// The I8H layout ([256 x i8][8 x f16 scale] per row) through the same MFMA decomposition as
// decode_attn_mfma_kernel.  An int8 code is exactly representable in f16, so codes enter the
// MFMAs as they are and the block scales are applied where a block's sum is complete:
//   scores: one 32-deep MFMA pair per 32-value block m (the block is the contraction), then
//           s[cell] += scale_k[cell][m] * partial[cell]           (4 FMAs per block and lane)
//   P.V   : the dequantised value code * scale (7 + 11 significant bits) is split exactly into
//           two f16 terms, hi = f16(code * scale) and lo = fma(code, scale, -hi) (the remainder
//           has at most 7 significant bits and its lowest bit is 2^(e - 10) >= 2^-24 for a normal
//           scale 2^e * f, so it is a representable f16 number, subnormal at worst); the three
//           products (hi + lo).(p_hi + p_lo) then carry the result to f32 accuracy.  A lane's 8 columns lie in one block (4 h + c / 4), so it
//           needs one scale per V row and half.
// The VALU formulation of this layout is bound by instruction issue (conversions and FMAs, 40 %
// of the HBM roofline on long contexts); here the VALU only converts and scales.
typedef _Float16 h2m __attribute__((ext_vector_type(2)));

// four int8 codes (one dword) -> four exact f16 values: 0x6400 | (code ^ 0x80) is 1024 + (code + 128)
__device__ __forceinline__ void codes_to_f16(unsigned w, h2m& lo, h2m& hi) {
    const unsigned u = w ^ 0x80808080u;
    const h2m bias = h2m{(_Float16)1152.0f, (_Float16)1152.0f};
    lo = __builtin_bit_cast(h2m, __builtin_amdgcn_perm(0x64646464u, u, 0x04010400u)) - bias;
    hi = __builtin_bit_cast(h2m, __builtin_amdgcn_perm(0x64646464u, u, 0x04030402u)) - bias;
}
// the same for codes that already carry the ^ 0x80 bias
__device__ __forceinline__ void biased_to_f16(unsigned u, h2m& lo, h2m& hi) {
    const h2m bias = h2m{(_Float16)1152.0f, (_Float16)1152.0f};
    lo = __builtin_bit_cast(h2m, __builtin_amdgcn_perm(0x64646464u, u, 0x04010400u)) - bias;
    hi = __builtin_bit_cast(h2m, __builtin_amdgcn_perm(0x64646464u, u, 0x04030402u)) - bias;
}
// 4 x 4 byte transpose: t[j] = { w[0].byte j, w[1].byte j, w[2].byte j, w[3].byte j }
__device__ __forceinline__ void transpose4x4_bytes(const unsigned (&w)[4], unsigned (&t)[4]) {
    const unsigned a_lo = __builtin_amdgcn_perm(w[1], w[0], 0x05010400u);  // w0.0 w1.0 w0.1 w1.1
    const unsigned a_hi = __builtin_amdgcn_perm(w[1], w[0], 0x07030602u);  // w0.2 w1.2 w0.3 w1.3
    const unsigned b_lo = __builtin_amdgcn_perm(w[3], w[2], 0x05010400u);
    const unsigned b_hi = __builtin_amdgcn_perm(w[3], w[2], 0x07030602u);
    t[0] = __builtin_amdgcn_perm(b_lo, a_lo, 0x05040100u);
    t[1] = __builtin_amdgcn_perm(b_lo, a_lo, 0x07060302u);
    t[2] = __builtin_amdgcn_perm(b_hi, a_hi, 0x05040100u);
    t[3] = __builtin_amdgcn_perm(b_hi, a_hi, 0x07060302u);
}
// whether either f16 of a dword has exponent field 0 (the values the cache reads as zero)
__device__ __forceinline__ bool has_zero_exponent(unsigned two_halves) {
    const unsigned t = two_halves & 0x7c007c00u;
    return (t & 0xffffu) == 0 || (t >> 16) == 0;
}
__device__ __forceinline__ half8 codes8_to_f16(v2u w) {
    h2m a, b, c2, d;
    codes_to_f16(w.x, a, b);
    codes_to_f16(w.y, c2, d);
    return half8{a[0], a[1], b[0], b[1], c2[0], c2[1], d[0], d[1]};
}
// f16 scale under the cache's load rule (exponent field 0 reads as zero)
__device__ __forceinline__ float scale_of(_Float16 h) {
    const unsigned short bits = __builtin_bit_cast(unsigned short, h);
    return (bits & 0x7c00u) == 0 ? 0.0f : (float)h;
}

// Data path: rows reach the matrix cores through LDS, not through registers.  Every wave owns two
// slots of 2 x 4352 bytes (the K unit and the V unit of one page and kv head, scales included)
// and fills them with 16-byte global->LDS loads, 64 lanes x 16 contiguous bytes per instruction
// (whole cache lines, nothing fetched twice), two pages ahead of the page it computes: the K half
// of a slot is refilled right after the scores that read it, the V half right after P.V.  A
// wave has 20 such loads in flight in a fixed order (K, V of the next page, K, V of the one
// after), so "the oldest five have landed" is s_waitcnt vmcnt(15) at both points of use.
constexpr int kI8hUnit = kPage * row_bytes_of(kRowI8H);  // 4352
constexpr int kI8hSlot = 2 * kI8hUnit;                    // K unit, then V unit

// 4352 bytes = 4 x 1024 + 256: four full instructions and one of 16 lanes.  `real` false issues the
// same five instructions on one 16-byte location (the data is never used): the number of loads
// in flight, which the waits count, then does not depend on where in its range a wave is.
__device__ __forceinline__ void i8h_unit_to_lds(const uint8_t* src, bool real, uint8_t* dst, int lane) {
    typedef const __attribute__((address_space(1))) void* gptr;
    typedef __attribute__((address_space(3))) void* lptr;
    const uint8_t* lane_src = src + (real ? lane * 16 : 0);
    const int step = real ? 1024 : 0;
#pragma unroll
    for (int n = 0; n < 4; ++n)
        __builtin_amdgcn_global_load_lds((gptr)(lane_src + n * step), (lptr)(dst + n * 1024), 16, 0, 0);
    if (lane < 16) __builtin_amdgcn_global_load_lds((gptr)(lane_src + 4 * step), (lptr)(dst + 4096), 16, 0, 0);
}

__global__ __launch_bounds__(kBlock, 2) void decode_attn_mfma_i8h_kernel(const AttnKernelParams P) {
    // slot 0 and slot 1 of the four waves; the fold staging of the epilogue reuses their memory
    __shared__ __attribute__((aligned(16))) uint8_t ring[2 * kWaves * kI8hSlot];
    static_assert(sizeof(MfmaFoldLds) <= sizeof(ring), "fold staging must fit the slots");
    uint8_t* const ring0 = ring;
    uint8_t* const ring1 = ring + kWaves * kI8hSlot;
    constexpr int kRow = row_bytes_of(kRowI8H);  // 272

    const int unit = blockIdx.x;
    int e = 0;
    while (e + 1 < P.b.n && unit >= P.b.wg_base[e + 1]) ++e;
    const int rem = unit - P.b.wg_base[e];
    const int split = rem / P.n_kv;
    const int kvh = rem - split * P.n_kv;
    const int wg = unit;
    const int pos = P.b.pos[e];
    const int n_pages = pos / kPage + 1;
    const int pps = P.b.pps[e];
    const int pg0 = split * pps;
    const int pg1 = min(pg0 + pps, n_pages);
    typedef const __attribute__((address_space(4))) int32_t* table_ptr;
    const table_ptr bt = (table_ptr)(uintptr_t)(P.tables + (size_t)P.b.row[e] * (size_t)P.max_pages_per_seq);

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int c = lane & 15;
    const int g = lane >> 4;
    const int my_block = c >> 2;  // which of the 4 blocks of a half this lane's 8 columns lie in
    const size_t page_bytes = (size_t)P.n_kv * kI8hUnit;
    const size_t head_off = (size_t)kvh * kI8hUnit;
    uint8_t* const slot0 = ring0 + wave * kI8hSlot;
    uint8_t* const slot1 = ring1 + wave * kI8hSlot;

    // unit of pipeline step i of this wave; steps past the wave's last are requested all the same,
    // as loads of one location, so that the number of loads in flight stays what the waits assume
    const int n_steps = pg0 + wave < pg1 ? (pg1 - pg0 - wave + kWaves - 1) / kWaves : 0;
    const auto unit_off = [&](int i) -> size_t {
        return (size_t)bt[min(pg0 + wave + kWaves * i, pg1 - 1)] * page_bytes + head_off;
    };
    i8h_unit_to_lds(P.kpool + unit_off(0), n_steps > 0, slot0, lane);
    i8h_unit_to_lds(P.vpool + unit_off(0), n_steps > 0, slot0 + kI8hUnit, lane);
    i8h_unit_to_lds(P.kpool + unit_off(1), n_steps > 1, slot1, lane);
    i8h_unit_to_lds(P.vpool + unit_off(1), n_steps > 1, slot1 + kI8hUnit, lane);

    // ---- q fragments of head c (heads past the group stay zero) ----------------------------------
    half8 qhi[8], qlo[8];
    {
        const bool head_live = c < P.group;
        const float* qp = P.q + ((size_t)e * P.n_q + (size_t)kvh * P.group + (head_live ? c : 0)) * kHd + g * 8;
#pragma unroll
        for (int m = 0; m < 8; ++m) {
            float x[8];
            const float4 a = *reinterpret_cast<const float4*>(qp + m * 32);
            const float4 b = *reinterpret_cast<const float4*>(qp + m * 32 + 4);
            x[0] = a.x, x[1] = a.y, x[2] = a.z, x[3] = a.w;
            x[4] = b.x, x[5] = b.y, x[6] = b.z, x[7] = b.w;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                _Float16 hi, lo;
                split_hi_lo(head_live ? x[j] : 0.0f, hi, lo);
                qhi[m][j] = hi;
                qlo[m][j] = lo;
            }
        }
    }

    f4 o[2][8];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int t = 0; t < 8; ++t) o[h][t] = f4{0.0f, 0.0f, 0.0f, 0.0f};
    float m_run = -INFINITY;
    float l_run = 0.0f;

    // One page: step i of the wave, resident in `slot`; the slot is refilled with step i + 2.
    const auto one_page = [&](uint8_t* slot, int i) __attribute__((always_inline)) {
        const int pg = pg0 + wave + kWaves * i;
        const uint8_t* ks = slot;
        const uint8_t* vs = slot + kI8hUnit;
        const size_t off_next = unit_off(i + 2);

        // ---- scores: per block, codes . q on the matrix core, then the block's scale ----------------
        __builtin_amdgcn_s_waitcnt(0x0F7F);  // vmcnt(15): this page's K unit has landed
        f4 s = f4{0.0f, 0.0f, 0.0f, 0.0f};
        // all fragments of the unit are requested from LDS in one batch, ahead of the first use
        half8 ksc[4];
        v2u kc[8];
#pragma unroll
        for (int m = 0; m < 8; ++m) kc[m] = *reinterpret_cast<const v2u*>(ks + c * kRow + m * 32 + g * 8);
#pragma unroll
        for (int r = 0; r < 4; ++r)
            ksc[r] = __builtin_bit_cast(half8, *reinterpret_cast<const v4u*>(ks + (4 * g + r) * kRow + kHd));
        const unsigned k_screen = *reinterpret_cast<const unsigned*>(ks + (lane >> 2) * kRow + kHd + 4 * (lane & 3));
        __builtin_amdgcn_sched_barrier(0);
        // A scale with exponent field 0 reads as zero.  The store rule never writes one, so the
        // unit's 64 scale dwords are screened one per lane, and only a unit that holds such a scale
        // (foreign data, rows never written) pays for the per-value rule.
        if (__builtin_amdgcn_ballot_w64(has_zero_exponent(k_screen)) != 0) {
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int m = 0; m < 8; ++m)
                    if ((__builtin_bit_cast(unsigned short, ksc[r][m]) & 0x7c00u) == 0) ksc[r][m] = (_Float16)0.0f;
        }
#pragma unroll
        for (int m = 0; m < 8; ++m) {
            const half8 ka = codes8_to_f16(kc[m]);
            f4 part = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka, qhi[m], f4{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
            part = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka, qlo[m], part, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 4; ++r) s[r] = fmaf((float)ksc[r][m], part[r], s[r]);
        }
        i8h_unit_to_lds(P.kpool + off_next, i + 2 < n_steps, slot, lane);

        // ---- online softmax of head c ---------------------------------------------------------------
        float t4[4];
        float pm = -INFINITY;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const bool live = pg * kPage + 4 * g + r <= pos;
            t4[r] = live ? s[r] * P.scale_log2e : -INFINITY;
            pm = fmaxf(pm, t4[r]);
        }
        pm = max_over_lane_groups(pm);
        const float m_new = fmaxf(m_run, pm);  // finite: every page of a range holds a live cell
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        float p[4];
        float psum = 0.0f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            p[r] = __builtin_amdgcn_exp2f(t4[r] - m_new);
            psum += p[r];
        }
        l_run = l_run * alpha + psum;
        if (__builtin_amdgcn_ballot_w64(m_new > m_run) != 0) {
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int t = 0; t < 8; ++t) o[h][t] *= alpha;
        }
        m_run = m_new;
        h4m phi, plo;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            _Float16 hi, lo;
            split_hi_lo(p[r], hi, lo);
            phi[r] = hi;
            plo[r] = lo;
        }
        const half8 phh = half8{phi[0], phi[1], phi[2], phi[3], phi[0], phi[1], phi[2], phi[3]};
        const half8 pll = half8{plo[0], plo[1], plo[2], plo[3], plo[0], plo[1], plo[2], plo[3]};
        // ---- P.V: dequantise into the exact (hi, lo) pair, two 32-deep MFMAs per 16 columns ---------------
        __builtin_amdgcn_s_waitcnt(0x0F7F);  // vmcnt(15): this page's V unit has landed
        // Scales of the lane's rows 4 g + r for its block of either half.  Rows past `pos` may hold
        // anything: their probabilities are exact zeros already, and their scales are made zeros
        // too, so that 0 * (garbage scale) cannot produce a NaN (any int8 code is a finite number).
        unsigned vsb[2][4];
        v2u vc[2][4];
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                vc[h][r] = *reinterpret_cast<const v2u*>(vs + (4 * g + r) * kRow + h * 128 + c * 8);
                vsb[h][r] = *reinterpret_cast<const unsigned short*>(vs + (4 * g + r) * kRow + kHd + 2 * (4 * h + my_block));
            }
        const unsigned v_screen = *reinterpret_cast<const unsigned*>(vs + (lane >> 2) * kRow + kHd + 4 * (lane & 3));
        __builtin_amdgcn_sched_barrier(0);
        const bool last_page = pg == n_pages - 1;
        if (last_page || __builtin_amdgcn_ballot_w64(has_zero_exponent(v_screen)) != 0) {
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if ((vsb[h][r] & 0x7c00u) == 0 || pg * kPage + 4 * g + r > pos) vsb[h][r] = 0;
        }
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const h2m s01 = __builtin_bit_cast(h2m, vsb[h][0] | (vsb[h][1] << 16));
            const h2m s23 = __builtin_bit_cast(h2m, vsb[h][2] | (vsb[h][3] << 16));
            // the lane's 4 rows x 8 codes, transposed as bytes so that a dword holds one column's
            // four rows: converted, it is the A fragment of that column's MFMA
            unsigned wx[4], wy[4], col[8];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                wx[r] = vc[h][r].x ^ 0x80808080u;
                wy[r] = vc[h][r].y ^ 0x80808080u;
            }
            {
                unsigned t0[4], t1[4];
                transpose4x4_bytes(wx, t0);
                transpose4x4_bytes(wy, t1);
#pragma unroll
                for (int t = 0; t < 4; ++t) col[t] = t0[t], col[4 + t] = t1[t];
            }
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                h2m c01, c23;
                biased_to_f16(col[t], c01, c23);
                const h2m hi01 = c01 * s01, hi23 = c23 * s23;
                const h2m lo01 = __builtin_elementwise_fma(c01, s01, -hi01);
                const h2m lo23 = __builtin_elementwise_fma(c23, s23, -hi23);
                // (hi + lo) . p_hi and (hi + lo) . p_lo as two 32-deep MFMAs: the contraction runs
                // over the 16 cells twice, a lane's eight slots being its four cells' hi parts and then
                // their lo parts
                const half8 ahl = half8{hi01[0], hi01[1], hi23[0], hi23[1], lo01[0], lo01[1], lo23[0], lo23[1]};
                o[h][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ahl, phh, o[h][t], 0, 0, 0);
                o[h][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ahl, pll, o[h][t], 0, 0, 0);
            }
        }
        i8h_unit_to_lds(P.vpool + off_next, i + 2 < n_steps, slot + kI8hUnit, lane);
    };

    for (int i = 0; i < n_steps; ++i) one_page((i & 1) ? slot1 : slot0, i);

    // no load may still be on its way into the slots when the fold staging takes their place
    __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0)
    __syncthreads();
    mfma_fold_and_store(P, *reinterpret_cast<MfmaFoldLds*>(ring), wg, wave, c, g, o, m_run, l_run);
}

// ---- decode attention on the matrix cores, f16 K and q8_0 V -----------------------------------
// The MFMA decomposition of decode_attn_mfma_kernel with both operands staged through LDS like the
// int8 kernel's units (every load of the loop is then a global->LDS load, which keeps the count of
// loads in flight, and with it every wait, exact): the f16 K unit of the next page is requested
// when the scores have used this page's, the V units ([f32 scale][32 x i8] blocks, 288 bytes a
// row) two pages ahead.  A q8_0 value is code * scale with an f32 scale, so it takes a per-cell
// power of two out first to stay inside f16:
//   E[cell]  = exponent of the largest of the cell's 8 block scales (clamped to +-120),
//   a[cell][d] = code * (scale * 2^-E[cell])       |a| < 256; split into hi + lo f16 as below,
//   weight   = exp2(logit + E[cell] - M)            M the running maximum of logit + E,
// so that weight * a is the term softmax-weight * value up to the common factor 2^-M, the largest
// terms have weights near 1 whatever the magnitudes of their values, and what falls off the f16
// range is small against the largest term.  The denominator sums exp2(logit - M) in f32.
// scale' = scale * 2^-E is split into two f16 (s_hi + s_lo, 22 bits); code * s_hi is split exactly
// into hi = f16(.) and its remainder (at most 7 significant bits, a representable f16 number),
// and lo = remainder + code * s_lo; (hi + lo) . (w_hi + w_lo) on two 32-deep MFMAs as in the int8
// kernel.
constexpr int kQ8vRow = row_bytes_of(kRowQ8);  // 288
constexpr int kQ8vUnit = kPage * kQ8vRow;      // 4608

// K unit in LDS: 8 instructions of 1024 bytes (two rows each), 32 bytes apart so that the rows a
// fragment read touches spread over the banks.
constexpr int kQ8vKStep = 1024 + 32;
constexpr int kQ8vKSlot = 8 * kQ8vKStep;  // 8448
__device__ __forceinline__ void q8v_k_unit_to_lds(const uint8_t* src, bool real, uint8_t* dst, int lane) {
    typedef const __attribute__((address_space(1))) void* gptr;
    typedef __attribute__((address_space(3))) void* lptr;
    const uint8_t* lane_src = src + (real ? lane * 16 : 0);
    const int step = real ? 1024 : 0;
#pragma unroll
    for (int n = 0; n < 8; ++n)
        __builtin_amdgcn_global_load_lds((gptr)(lane_src + n * step), (lptr)(dst + n * kQ8vKStep), 16, 0, 0);
}

// 4608 bytes = 4 x 1024 + 512: four full instructions and one of 32 lanes.  `real` false issues the
// same five instructions on one 16-byte location (the data is never used): the number of loads
// in flight, which the waits count, then does not depend on where in its range a wave is.
__device__ __forceinline__ void q8v_unit_to_lds(const uint8_t* src, bool real, uint8_t* dst, int lane) {
    typedef const __attribute__((address_space(1))) void* gptr;
    typedef __attribute__((address_space(3))) void* lptr;
    const uint8_t* lane_src = src + (real ? lane * 16 : 0);
    const int step = real ? 1024 : 0;
#pragma unroll
    for (int n = 0; n < 4; ++n)
        __builtin_amdgcn_global_load_lds((gptr)(lane_src + n * step), (lptr)(dst + n * 1024), 16, 0, 0);
    if (lane < 32) __builtin_amdgcn_global_load_lds((gptr)(lane_src + 4 * step), (lptr)(dst + 4096), 16, 0, 0);
}

template <int CTRL>
__device__ __forceinline__ float dpp_mov(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, false));
}

__global__ __launch_bounds__(kBlock, 2) void decode_attn_mfma_q8v_kernel(const AttnKernelParams P) {
    // per wave one K slot and two V slots during the loop, the fold staging after it
    constexpr int kWaveLds = kQ8vKSlot + 2 * kQ8vUnit;
    constexpr int kLds = kWaves * kWaveLds > (int)sizeof(MfmaFoldLds) ? kWaves * kWaveLds : (int)sizeof(MfmaFoldLds);
    __shared__ __attribute__((aligned(16))) uint8_t smem[kLds];

    const int unit = blockIdx.x;
    int e = 0;
    while (e + 1 < P.b.n && unit >= P.b.wg_base[e + 1]) ++e;
    const int rem = unit - P.b.wg_base[e];
    const int split = rem / P.n_kv;
    const int kvh = rem - split * P.n_kv;
    const int wg = unit;
    const int pos = P.b.pos[e];
    const int n_pages = pos / kPage + 1;
    const int pps = P.b.pps[e];
    const int pg0 = split * pps;
    const int pg1 = min(pg0 + pps, n_pages);
    typedef const __attribute__((address_space(4))) int32_t* table_ptr;
    const table_ptr bt = (table_ptr)(uintptr_t)(P.tables + (size_t)P.b.row[e] * (size_t)P.max_pages_per_seq);

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int c = lane & 15;
    const int g = lane >> 4;
    const size_t k_page_bytes = (size_t)P.n_kv * kPage * kHd * 2;
    const size_t k_head_off = (size_t)kvh * kPage * kHd * 2;
    const size_t v_page_bytes = (size_t)P.n_kv * kQ8vUnit;
    const size_t v_head_off = (size_t)kvh * kQ8vUnit;
    uint8_t* const kslot = smem + wave * kWaveLds;
    uint8_t* const slots = kslot + kQ8vKSlot;

    // pipeline steps of this wave: pages pg0 + wave, + kWaves, ...
    const int n_steps = pg0 + wave < pg1 ? (pg1 - pg0 - wave + kWaves - 1) / kWaves : 0;
    // physical page of step i; past the wave's last step the answer is not used for its data
    const auto phys = [&](int i) -> size_t { return (size_t)bt[min(pg0 + wave + kWaves * i, pg1 - 1)]; };

    // Loads complete in order.  Issue order per step: K(i+1) when the scores of step i are done,
    // V(i+2) at its end; the prologue keeps that order (V0, K0, V1).  Behind K(i) at the top of step
    // i there is V(i+1) = 5 loads; behind V(i) where step i needs it there are K(i), V(i+1), K(i+1)
    // = 8 + 5 + 8.  Steps that do not exist are requested all the same, as loads of one location,
    // so that these counts hold everywhere.
    const auto k_unit = [&](int i) { return P.kpool + phys(i) * k_page_bytes + k_head_off; };
    const auto v_unit = [&](int i) { return P.vpool + phys(i) * v_page_bytes + v_head_off; };
    q8v_unit_to_lds(v_unit(0), n_steps > 0, slots, lane);
    q8v_k_unit_to_lds(k_unit(0), n_steps > 0, kslot, lane);
    q8v_unit_to_lds(v_unit(1), n_steps > 1, slots + kQ8vUnit, lane);

    // ---- q fragments of head c (heads past the group stay zero) ----------------------------------
    half8 qhi[8], qlo[8];
    {
        const bool head_live = c < P.group;
        const float* qp = P.q + ((size_t)e * P.n_q + (size_t)kvh * P.group + (head_live ? c : 0)) * kHd + g * 8;
#pragma unroll
        for (int m = 0; m < 8; ++m) {
            float x[8];
            const float4 a = *reinterpret_cast<const float4*>(qp + m * 32);
            const float4 b = *reinterpret_cast<const float4*>(qp + m * 32 + 4);
            x[0] = a.x, x[1] = a.y, x[2] = a.z, x[3] = a.w;
            x[4] = b.x, x[5] = b.y, x[6] = b.z, x[7] = b.w;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                _Float16 hi, lo;
                split_hi_lo(head_live ? x[j] : 0.0f, hi, lo);
                qhi[m][j] = hi;
                qlo[m][j] = lo;
            }
        }
    }

    f4 o[2][8];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int t = 0; t < 8; ++t) o[h][t] = f4{0.0f, 0.0f, 0.0f, 0.0f};
    float m_run = -INFINITY;  // running maximum of logit + E (base 2)
    float l_run = 0.0f;       // this lane's share of sum exp2(logit - m_run)
    const int my_block = c >> 2;  // which of the 4 blocks of a half this lane's 8 columns lie in

    for (int i = 0; i < n_steps; ++i) {
        const int pg = pg0 + wave + kWaves * i;
        const uint8_t* vs = slots + (i & 1) * kQ8vUnit;
        const int behind = n_steps - 1 - i;  // steps after this one

        // ---- S^T = K . q^T: four independent accumulation chains ------------------------------
        __builtin_amdgcn_s_waitcnt(0x0F75);  // vmcnt(5): this page's K unit has landed
        v4u kf[8];
        {
            // row c: two rows per 1056-byte step; fragment m of lane group g at 64 m + 16 g
            const uint8_t* kr = kslot + (c >> 1) * kQ8vKStep + (c & 1) * 512 + g * 16;
#pragma unroll
            for (int m = 0; m < 8; ++m) kf[m] = *reinterpret_cast<const v4u*>(kr + m * 64);
        }
        __builtin_amdgcn_sched_barrier(0);
        f4 s0 = f4{0.0f, 0.0f, 0.0f, 0.0f}, s1 = s0, s2 = s0, s3 = s0;
#pragma unroll
        for (int m = 0; m < 8; m += 2) {
            const half8 ka = __builtin_bit_cast(half8, kf[m]);
            const half8 kb = __builtin_bit_cast(half8, kf[m + 1]);
            s0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka, qhi[m], s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka, qlo[m], s1, 0, 0, 0);
            s2 = __builtin_amdgcn_mfma_f32_16x16x32_f16(kb, qhi[m + 1], s2, 0, 0, 0);
            s3 = __builtin_amdgcn_mfma_f32_16x16x32_f16(kb, qlo[m + 1], s3, 0, 0, 0);
        }
        const f4 s = (s0 + s1) + (s2 + s3);  // s[r] = q[head c] . k[cell 4 g + r]
        q8v_k_unit_to_lds(k_unit(i + 1), behind >= 1, kslot, lane);

        // ---- this page's V unit: scales first -------------------------------------------------
        __builtin_amdgcn_s_waitcnt(0x4F75);  // vmcnt(21): K(i), V(i+1), K(i+1) behind V(i)
        // lane (c, g): scale of blocks 2 (c / 4), + 1 of row 4 g + c % 4, the row's maximum over the
        // lanes c, c ^ 4, c ^ 8, c ^ 12, then the four rows' maxima from the lanes of the quad
        const bool last_page = pg == n_pages - 1;
        float smax;
        {
            const uint8_t* rp = vs + (4 * g + (c & 3)) * kQ8vRow + (c >> 2) * 72;
            const float a = *reinterpret_cast<const float*>(rp);
            const float b = *reinterpret_cast<const float*>(rp + 36);
            smax = fmaxf(a, b);
            // rows past `pos` may hold anything: they count as scale 1 here and as zeros below
            if (last_page && pg * kPage + 4 * g + (c & 3) > pos) smax = 1.0f;
            smax = fmaxf(smax, dpp_mov<0x124>(smax));  // row_ror:4
            smax = fmaxf(smax, dpp_mov<0x128>(smax));  // row_ror:8
        }
        int ex[4];
        float down[4];  // 2^-E
        {
            const float m0 = dpp_mov<0x00>(smax), m1 = dpp_mov<0x55>(smax);
            const float m2 = dpp_mov<0xAA>(smax), m3 = dpp_mov<0xFF>(smax);
            const float mr[4] = {m0, m1, m2, m3};
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                int ee = (int)((__builtin_bit_cast(unsigned, mr[r]) >> 23) & 0xffu) - 127;
                ee = min(max(ee, -120), 120);
                ex[r] = ee;
                down[r] = __builtin_bit_cast(float, (unsigned)(127 - ee) << 23);
            }
        }

        // ---- online softmax of head c over logit + E ------------------------------------------------
        float t4[4], tw[4];
        float pm = -INFINITY;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const bool live = pg * kPage + 4 * g + r <= pos;
            t4[r] = live ? s[r] * P.scale_log2e : -INFINITY;
            tw[r] = t4[r] + (float)ex[r];
            pm = fmaxf(pm, tw[r]);
        }
        pm = max_over_lane_groups(pm);
        const float m_new = fmaxf(m_run, pm);  // finite: every page of a range holds a live cell
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        h4m whi, wlo;
        float psum = 0.0f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float w = __builtin_amdgcn_exp2f(tw[r] - m_new);
            psum += __builtin_amdgcn_exp2f(t4[r] - m_new);
            _Float16 hi, lo;
            split_hi_lo(w, hi, lo);
            whi[r] = hi;
            wlo[r] = lo;
        }
        l_run = l_run * alpha + psum;
        if (__builtin_amdgcn_ballot_w64(m_new > m_run) != 0) {
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int t = 0; t < 8; ++t) o[h][t] *= alpha;
        }
        m_run = m_new;
        const half8 whh = half8{whi[0], whi[1], whi[2], whi[3], whi[0], whi[1], whi[2], whi[3]};
        const half8 wll = half8{wlo[0], wlo[1], wlo[2], wlo[3], wlo[0], wlo[1], wlo[2], wlo[3]};

        // ---- P.V ----------------------------------------------------------------------------------
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            unsigned wx[4], wy[4], col[8];
            _Float16 shi[4], slo[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const uint8_t* blk = vs + (4 * g + r) * kQ8vRow + (4 * h + my_block) * 36;
                float sc = *reinterpret_cast<const float*>(blk) * down[r];
                if (last_page && pg * kPage + 4 * g + r > pos) sc = 0.0f;
                split_hi_lo(sc, shi[r], slo[r]);
                const unsigned* cw = reinterpret_cast<const unsigned*>(blk + 4 + (c & 3) * 8);
                wx[r] = cw[0] ^ 0x80808080u;
                wy[r] = cw[1] ^ 0x80808080u;
            }
            const h2m s01 = h2m{shi[0], shi[1]}, s23 = h2m{shi[2], shi[3]};
            const h2m l01 = h2m{slo[0], slo[1]}, l23 = h2m{slo[2], slo[3]};
            {
                unsigned t0[4], t1[4];
                transpose4x4_bytes(wx, t0);
                transpose4x4_bytes(wy, t1);
#pragma unroll
                for (int t = 0; t < 4; ++t) col[t] = t0[t], col[4 + t] = t1[t];
            }
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                h2m c01, c23;
                biased_to_f16(col[t], c01, c23);
                const h2m hi01 = c01 * s01, hi23 = c23 * s23;
                const h2m lo01 = __builtin_elementwise_fma(c01, l01, __builtin_elementwise_fma(c01, s01, -hi01));
                const h2m lo23 = __builtin_elementwise_fma(c23, l23, __builtin_elementwise_fma(c23, s23, -hi23));
                const half8 ahl = half8{hi01[0], hi01[1], hi23[0], hi23[1], lo01[0], lo01[1], lo23[0], lo23[1]};
                o[h][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ahl, whh, o[h][t], 0, 0, 0);
                o[h][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ahl, wll, o[h][t], 0, 0, 0);
            }
        }
        q8v_unit_to_lds(v_unit(i + 2), behind >= 2, slots + (i & 1) * kQ8vUnit, lane);
    }

    // no load may still be on its way into the slots when the fold staging takes their place
    __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0)
    __syncthreads();
    mfma_fold_and_store(P, *reinterpret_cast<MfmaFoldLds*>(smem), wg, wave, c, g, o, m_run, l_run);
}

struct MergeParams {
    AttnBatch b;
    const float* part_o;
    const float* part_ml;
    const float* gate;
    float* out;
    int64_t gate_seq_stride, gate_head_stride;
    int32_t n_kv, n_q, group, hg;
};

constexpr int kMergeGroups = 4;   // split ranges summed side by side, then folded in LDS
constexpr int kMergeInFlight = 8; // partial rows a thread requests before it needs the factors

// One work-group per (entry, q head): kMergeGroups x 256 threads.  Thread (g, d) owns head-dim
// element d of splits g, g + 4, ...; it requests its first 8 partial values straight away, and
// only then are the per-split (m, l) pairs staged in LDS and the maximum agreed, so the two
// round trips to memory overlap.
__global__ __launch_bounds__(kHd * kMergeGroups) void decode_attn_merge_kernel(const MergeParams P) {
    constexpr int kMaxStaged = 1024;
    __shared__ float sm[kMaxStaged];
    __shared__ float sl[kMaxStaged];
    __shared__ float red[kMergeGroups][kHd];
    __shared__ float red_l[kMergeGroups];
    __shared__ float wave_max[kHd * kMergeGroups / 64];
    const int e = blockIdx.x / P.n_q;
    const int h = blockIdx.x % P.n_q;
    const int kvh = h / P.group;
    const int hl = h % P.group;
    const int hc = hl / P.hg;
    const int hh = hl % P.hg;
    const int splits = P.b.splits[e];
    const int wg0 = P.b.wg_base[e] + hc * splits * P.n_kv + kvh;
    const int d = threadIdx.x & (kHd - 1);
    const int g = threadIdx.x >> 8;
    const size_t ostride = (size_t)P.n_kv * P.hg * kHd;  // floats between consecutive splits
    const float* po = P.part_o + ((size_t)wg0 * P.hg + hh) * kHd + d;
    const float* pml = P.part_ml + ((size_t)wg0 * P.hg + hh) * 2;
    const size_t mlstride = (size_t)P.n_kv * P.hg * 2;

    float v[kMergeInFlight];
#pragma unroll
    for (int u = 0; u < kMergeInFlight; ++u) {
        const int s = g + u * kMergeGroups;
        v[u] = s < splits ? po[(size_t)s * ostride] : 0.0f;
    }
    // stage (m, l) and agree on the maximum: per-thread max over its splits, wave reduction,
    // then one LDS slot per wave (a serial scan over the splits would cost a dependent LDS
    // round trip per split)
    constexpr int kThreads = kHd * kMergeGroups;
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
    if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6] = my_m;
    __syncthreads();
    const auto m_of = [&](int s) { return s < kMaxStaged ? sm[s] : pml[(size_t)s * mlstride]; };
    const auto l_of = [&](int s) { return s < kMaxStaged ? sl[s] : pml[(size_t)s * mlstride + 1]; };
    float mx = wave_max[0];
#pragma unroll
    for (int w = 1; w < kThreads / 64; ++w) mx = fmaxf(mx, wave_max[w]);
    float acc = 0.0f, lsum = 0.0f;
#pragma unroll
    for (int u = 0; u < kMergeInFlight; ++u) {
        const int s = g + u * kMergeGroups;
        if (s < splits) {
            const float ms = m_of(s);
            const float f = ms == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(ms - mx);
            acc = fmaf(f, v[u], acc);
            lsum = fmaf(f, l_of(s), lsum);
        }
    }
    // further rounds of kMergeInFlight requests for long split lists
    for (int s0 = g + kMergeInFlight * kMergeGroups; s0 < splits;
         s0 += kMergeInFlight * kMergeGroups) {
#pragma unroll
        for (int u = 0; u < kMergeInFlight; ++u) {
            const int s = s0 + u * kMergeGroups;
            v[u] = s < splits ? po[(size_t)s * ostride] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < kMergeInFlight; ++u) {
            const int s = s0 + u * kMergeGroups;
            if (s < splits) {
                const float ms = m_of(s);
                const float f = ms == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(ms - mx);
                acc = fmaf(f, v[u], acc);
                lsum = fmaf(f, l_of(s), lsum);
            }
        }
    }
    red[g][d] = acc;
    if (d == 0) red_l[g] = lsum;
    __syncthreads();
    if (g != 0) return;
#pragma unroll
    for (int k = 1; k < kMergeGroups; ++k) {
        acc += red[k][d];
        lsum += red_l[k];
    }
    float r = lsum > 0.0f ? acc / lsum : 0.0f;
    if (P.gate) {
        const float gt = P.gate[(size_t)e * P.gate_seq_stride + (size_t)h * P.gate_head_stride + d];
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

// Heads one work-group carries for a given q-heads-per-kv-head group.
int32_t attn_heads_per_wave(int32_t group) { return group % 8 == 0 ? 8 : 4; }

// Whether a call on this pool goes to the MFMA kernel: f16 rows, unless the pool was
// created with BKV_POOL_ATTN_VALU (the VALU formulation, kept for comparison).
bool attn_on_mfma(const bkv_pool* p, int32_t group, bool dense) {
    if (group > 16 || (p->desc.flags & BKV_POOL_ATTN_VALU) != 0) return false;
    // f16 rows: every call; the quantised layouts: the dense selection
    return p->g.layout == BKV_LAYOUT_F16 || dense;
}

int32_t plan_attn(const bkv_pool* p, int32_t n_q_head, AttnBatch& b, int32_t sel_groups, bool mfma) {
    const int32_t n_kv = p->g.n_kv;
    const int32_t group = n_q_head / n_kv;
    const int32_t hg = mfma ? group : attn_heads_per_wave(group);
    const int32_t n_hc = (group + hg - 1) / hg;
    const int64_t per_page = (int64_t)n_kv * n_hc;
    int64_t total_pages = 0;
    // loop iterations of an entry: its pages, or (selection lists, whose true lengths only the
    // device knows) the most groups of four blocks a list can hold
    const auto iters = [&](int i) -> int64_t { return sel_groups > 0 ? sel_groups : b.pos[i] / kPage + 1; };
    for (int i = 0; i < b.n; ++i) total_pages += iters(i);
    // All work-groups should be resident at once (one generation): a handful of left-over
    // work-groups would run alone after the rest and double the kernel's time.  `resident`
    // follows from the register budget of the kernel variant that will run.
    const int64_t resident = (mfma || hg == 8) ? 2 : 3;
    int64_t target = (int64_t)(p->n_cu > 0 ? p->n_cu : 256) * resident;
    if (target > p->max_wgs) target = p->max_wgs;
    int64_t pps = (total_pages * per_page + target - 1) / target;
    pps = ((pps + kWaves - 1) / kWaves) * kWaves;
    if (pps < kWaves) pps = kWaves;
    for (;;) {
        int64_t total = 0;
        for (int i = 0; i < b.n; ++i) {
            const int64_t pages = iters(i);
            const int64_t splits = (pages + pps - 1) / pps;
            // even the ranges out inside the entry, keeping whole groups of kWaves pages
            int64_t each = (pages + splits - 1) / splits;
            each = ((each + kWaves - 1) / kWaves) * kWaves;
            b.splits[i] = (int32_t)((pages + each - 1) / each);
            b.pps[i] = (int32_t)each;
            b.wg_base[i] = (int32_t)total;
            total += (int64_t)b.splits[i] * per_page;
        }
        b.wg_base[b.n] = (int32_t)total;
        if (total <= target) return (int32_t)total;
        pps += kWaves;
    }
}

hipError_t launch_decode_attn(bkv_pool* p, int32_t layer, const AttnBatch& b, const AttnArgs& a,
                              hipStream_t stream) {
    const int32_t n_kv = p->g.n_kv;
    const int32_t group = a.n_q_head / n_kv;
    const int32_t hg = a.mfma ? group : attn_heads_per_wave(group);
    AttnKernelParams kp;
    kp.b = b;
    kp.kpool = p->k_layer[(size_t)layer];
    kp.vpool = p->v_layer[(size_t)layer];
    kp.tables = p->table_dev;
    kp.q = a.q;
    kp.part_o = p->part_o;
    kp.part_ml = p->part_ml;
    kp.max_pages_per_seq = p->desc.max_pages_per_seq;
    kp.n_kv = n_kv;
    kp.n_q = a.n_q_head;
    kp.group = group;
    kp.n_hc = (group + hg - 1) / hg;
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
    const int32_t total = b.wg_base[b.n];
    const int32_t n_units = total / kp.n_hc;
    const int32_t grid = (n_units + 7) / 8 * 8 * kp.n_hc;
    {
        StageScope timed(p, BKV_STAGE_ATTN_SPLIT, stream);
        const int layout = p->g.layout;
#define BKV_LAUNCH(HGV, KE, VE)                                                  \
    do {                                                                        \
        if (sel)                                                                \
            decode_attn_kernel<HGV, KE, VE, true><<<grid, kBlock, 0, stream>>>(kp);  \
        else                                                                    \
            decode_attn_kernel<HGV, KE, VE, false><<<grid, kBlock, 0, stream>>>(kp); \
    } while (0)
        if (a.mfma) {
            // f16 pools, dense selection, one work-group per unit (checked by the caller)
            if (layout == BKV_LAYOUT_I8H)
                decode_attn_mfma_i8h_kernel<<<total, kBlock, 0, stream>>>(kp);
            else if (layout == BKV_LAYOUT_Q8V)
                decode_attn_mfma_q8v_kernel<<<total, kBlock, 0, stream>>>(kp);
            else if (step)
                decode_attn_mfma_kernel<true><<<total, kBlock, 0, stream>>>(kp);
            else if (sel)
                decode_attn_mfma_kernel<false, true><<<total, kBlock, 0, stream>>>(kp);
            else
                decode_attn_mfma_kernel<false><<<total, kBlock, 0, stream>>>(kp);
        } else if (step) {
            // f16 pools, dense selection (checked by the caller)
            if (hg == 8)
                decode_attn_kernel<8, kRowF16, kRowF16, false, true><<<grid, kBlock, 0, stream>>>(kp);
            else
                decode_attn_kernel<4, kRowF16, kRowF16, false, true><<<grid, kBlock, 0, stream>>>(kp);
        } else if (layout == BKV_LAYOUT_F16) {
            if (hg == 8) BKV_LAUNCH(8, kRowF16, kRowF16); else BKV_LAUNCH(4, kRowF16, kRowF16);
        } else if (layout == BKV_LAYOUT_Q8V) {
            if (hg == 8) BKV_LAUNCH(8, kRowF16, kRowQ8); else BKV_LAUNCH(4, kRowF16, kRowQ8);
        } else {
            if (hg == 8) BKV_LAUNCH(8, kRowI8H, kRowI8H); else BKV_LAUNCH(4, kRowI8H, kRowI8H);
        }
#undef BKV_LAUNCH
    }
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) return err;
    MergeParams mp;
    mp.b = b;
    mp.part_o = p->part_o;
    mp.part_ml = p->part_ml;
    mp.gate = a.gate;
    mp.out = a.out;
    mp.gate_seq_stride = a.gate_seq_stride;
    mp.gate_head_stride = a.gate_head_stride;
    mp.n_kv = n_kv;
    mp.n_q = a.n_q_head;
    mp.group = group;
    mp.hg = hg;
    {
        StageScope timed(p, BKV_STAGE_ATTN_MERGE, stream);
        decode_attn_merge_kernel<<<b.n * a.n_q_head, kHd * kMergeGroups, 0, stream>>>(mp);
    }
    return hipGetLastError();
}

}  // namespace bkv
