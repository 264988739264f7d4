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
#include "decode_attn_common.hpp"
#include "f16_rule.hpp"

namespace bkv {

namespace {

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

struct MergeParams {
    AttnBatch b;
    const AttnBatch* bd;  // DESC: the batch is read from this device-resident copy
    const float* part_o;
    const float* part_ml;
    const float* gate;
    float* out;
    int64_t gate_seq_stride, gate_head_stride;
    int32_t n_kv, n_q, group, hg;
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
    const int e = blockIdx.x / P.n_q;
    const int h = blockIdx.x % P.n_q;
    const int kvh = h / P.group;
    const int hl = h % P.group;
    const int hc = hl / P.hg;
    const int hh = hl % P.hg;
    int splits, base;
    if constexpr (DESC) {
        const batch_desc_ptr D = (batch_desc_ptr)(uintptr_t)P.bd;
        splits = D->splits[e];
        base = D->wg_base[e];
    } else {
        splits = P.b.splits[e];
        base = P.b.wg_base[e];
    }
    const int wg0 = base + hc * splits * P.n_kv + kvh;
    const int d4 = threadIdx.x & 63;
    const int g = threadIdx.x >> 6;
    const size_t ostride = (size_t)P.n_kv * P.hg * kHd;  // floats between consecutive splits
    const float* po = P.part_o + ((size_t)wg0 * P.hg + hh) * kHd + 4 * d4;
    const float* pml = P.part_ml + ((size_t)wg0 * P.hg + hh) * 2;
    const size_t mlstride = (size_t)P.n_kv * P.hg * 2;

    f4 v[kMergeInFlight];
#pragma unroll
    for (int u = 0; u < kMergeInFlight; ++u) {
        const int s = g + u * kMergeGroups;
        v[u] = s < splits ? *reinterpret_cast<const f4*>(po + (size_t)s * ostride) : f4{0.0f, 0.0f, 0.0f, 0.0f};
    }
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
    (void)dense;
    return true;
}

// The limits a plan of this pool geometry works under.  The partial-result workspace holds
// max_wgs x 8 head rows: a work-group of the matrix-core kernels writes `group` rows, one of the
// VALU kernel 8 or 4.
AttnPlanLimits attn_plan_limits(int32_t n_cu, int32_t max_wgs, int32_t n_kv, int32_t group, bool mfma) {
    const int32_t hg = mfma ? group : attn_heads_per_wave(group);
    const int32_t n_hc = (group + hg - 1) / hg;
    AttnPlanLimits lim;
    lim.per_page = n_kv * n_hc;
    lim.gran = kWaves;
    // All work-groups should be resident at once (one generation): a handful of left-over
    // work-groups would run alone after the rest and double the kernel's time.  `resident`
    // follows from the register budget of the kernel variant that will run.
    const int32_t resident = (mfma || hg == 8) ? 2 : 3;
    lim.target = (n_cu > 0 ? n_cu : 256) * resident;
    lim.max_wgs = hg > 8 ? (int32_t)((int64_t)max_wgs * 8 / hg) : max_wgs;
    return lim;
}

int32_t plan_attn(const bkv_pool* p, int32_t n_q_head, AttnBatch& b, int32_t sel_groups, bool mfma,
                  int32_t max_wgs) {
    const AttnPlanLimits lim =
        attn_plan_limits(p->n_cu, max_wgs > 0 ? max_wgs : p->max_wgs, p->g.n_kv, n_q_head / p->g.n_kv, mfma);
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
static void* g_scratch_ptr[kMaxDevices] = {};

hipError_t attn_static_scratch_init(int device) {
    if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
    if (g_scratch_ptr[device]) return hipSuccess;
    int current = -1;
    hipError_t e = hipGetDevice(&current);
    if (e != hipSuccess) return e;
    if (current != device) return hipErrorInvalidDevice;
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    g_scratch_ptr[device] = ptr;
    return hipSuccess;
}

bool attn_static_scratch(int device, float** o, float** ml) {
    if (device < 0 || device >= kMaxDevices || !g_scratch_ptr[device]) return false;
    AttnStaticScratch* s = static_cast<AttnStaticScratch*>(g_scratch_ptr[device]);
    *o = s->o;
    *ml = s->ml;
    return true;
}

hipError_t launch_decode_attn(bkv_pool* p, int32_t layer, const AttnBatch& b, const AttnArgs& a,
                              hipStream_t stream) {
    const int32_t n_kv = p->g.n_kv;
    const int32_t group = a.n_q_head / n_kv;
    const int32_t hg = a.mfma ? group : attn_heads_per_wave(group);
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
    const int32_t total = a.desc ? a.desc_grid : b.wg_base[b.n];
    const int32_t n_units = total / kp.n_hc;
    const int32_t grid = (n_units + 7) / 8 * 8 * kp.n_hc;
    if (a.mfma) {
        // one work-group per unit, every head of the kv head in it (checked by the caller); while the
        // pool times its kernels, the events ride on the dispatch
        hipEvent_t ev_start = nullptr, ev_stop = nullptr;
        if (a.timed) (void)timer_dispatch_events(p, BKV_STAGE_ATTN_SPLIT, &ev_start, &ev_stop);
        const hipError_t e = launch_decode_attn_mfma(kp, p->g.layout, step, sel, total, stream, ev_start, ev_stop);
        if (e != hipSuccess) return e;
    } else {
        const int layout = p->g.layout;
        const auto go = [&](auto kernel) {
            if (a.timed)
                launch_staged(p, BKV_STAGE_ATTN_SPLIT, kernel, dim3((unsigned)grid), dim3(kBlock), 0, stream, kp);
            else
                hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(kBlock), 0, stream, kp);
        };
#define BKV_LAUNCH(HGV, KE, VE)                              \
    do {                                                    \
        if (sel)                                            \
            go(decode_attn_kernel<HGV, KE, VE, true, false>);  \
        else                                                \
            go(decode_attn_kernel<HGV, KE, VE, false, false>); \
    } while (0)
        if (step) {
            // f16 pools, dense selection (checked by the caller)
            if (hg == 8)
                go(decode_attn_kernel<8, kRowF16, kRowF16, false, true>);
            else
                go(decode_attn_kernel<4, kRowF16, kRowF16, false, true>);
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
    mp.hg = hg;
    const dim3 mgrid((unsigned)(b.n * a.n_q_head)), mblock(64 * kMergeGroups);
    if (a.desc)
        hipLaunchKernelGGL(decode_attn_merge_kernel<true>, mgrid, mblock, 0, stream, mp);
    else if (a.timed)
        launch_staged(p, BKV_STAGE_ATTN_MERGE, decode_attn_merge_kernel<false>, mgrid, mblock, 0, stream, mp);
    else
        hipLaunchKernelGGL(decode_attn_merge_kernel<false>, mgrid, mblock, 0, stream, mp);
    return hipGetLastError();
}

// ---- a decode step that re-plans itself on the device ------------------------------------------
// One thread: every entry moves on by one cell and the batch is cut again, by the same function the
// host uses, so that a replayed launch reads what a fresh call would have been given.  An entry
// that would pass the last cell the plan was checked for stops the advance (nothing moves, the
// status word says so).
__global__ void step_advance_kernel(StepDesc* d, AttnPlanLimits lim, int32_t page_cells) {
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    AttnBatch b = d->b;
    for (int i = 0; i < b.n; ++i)
        if (b.pos[i] + 1 > d->horizon[i]) {
            d->status = 1;
            return;
        }
    for (int i = 0; i < b.n; ++i) b.pos[i] += 1;
    (void)plan_attn_ranges(lim, page_cells, 0, b);
    d->b = b;
    d->steps += 1u;
}

hipError_t launch_step_advance(StepDesc* d, const AttnPlanLimits& lim, int32_t page_cells, hipStream_t stream) {
    hipLaunchKernelGGL(step_advance_kernel, dim3(1), dim3(64), 0, stream, d, lim, page_cells);
    return hipGetLastError();
}

}  // namespace bkv
