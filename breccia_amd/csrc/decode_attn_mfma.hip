// Paged decode attention for gfx950: the split-K online-softmax kernels, on the matrix cores, for
// f16 pools, for int8 K/V with f16 block scales and for f16 K + q8_0 V.  The cut into work-groups,
// the merge kernel and the launch are in decode_attn.hip; results must agree with the reference's
// f64 CPU attend (crates/breccia-kernels/src/qsa/cpu.rs:197-246).
#include <hip/hip_ext.h>

#include "decode_attn_common.hpp"
#include "f16_rule.hpp"
#include "lane_groups.hpp"
#include "quant_decode.hpp"
#include "quant_encode.hpp"

namespace bkv {

namespace {

// ---- decode attention on the matrix cores -----------------------------------------------------
// Decode attention is an HBM-bound stream (every K/V row is read once and used by the `group` q
// heads of its kv head), but at the edge of the HBM roofline a formulation that multiplies on the
// VALU is co-limited by instruction issue -- and has to walk the rows once per chunk of 8 or 4
// heads (the reference's own 24 q / 2 kv heads = 12 per group).  A 16-column MFMA tile holds up
// to 16 heads of a kv head at once, every K/V row is read once whatever the group, and the VALU
// only does the softmax.  Lane (c = lane % 16, g = lane / 16) of a wave owns head c; per page:
//   S^T[cell][head] = K[cell][:] . q[head][:]          v_mfma_f32_16x16x32_f16, A = K, B = q
//   O^T[d][head]   += V^T[d][cell] . P^T[cell][head]   v_mfma_f32_16x16x32_f16, A = V regrouped
// with q and p split into a high and a low f16 part (K and V are exact f16), as in the prefill
// kernel: two MFMAs per K fragment, and for P.V one MFMA whose 32-deep contraction runs over the
// page's 16 cells twice, against p's high parts and against its low parts.  K fragment m of a
// lane is the 16 bytes at element 32 m + 8 g of row c; V fragments are the 16 bytes at element
// 128 h + 8 c of rows 4 g + r.  Every fragment register is refilled with the next page's data
// right after its last use.
typedef _Float16 h4m __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void split_hi_lo(float x, _Float16& hi, _Float16& lo) {
    hi = (_Float16)x;
    lo = (_Float16)(x - (float)hi);
}

// q fragments of head c of the kv head (heads past the group stay zero): lane (c, g) holds
// q[head][32 m + 8 g + 0..7], m = 0..7, as a high and a low f16 part
__device__ __forceinline__ void load_q_fragments(const AttnKernelParams& P, int e, int kvh, int c, int g,
                                                 half8 (&qhi)[8], half8 (&qlo)[8]) {
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

// K fragments as fetched (see k_addr in the kernel): of the pair (2 p, 2 p + 1), lane c < 8 holds its own
// fragment 2 p and fragment 2 p of lane c + 8, lane c >= 8 holds fragment 2 p + 1 of lane c - 8 and its own
// fragment 2 p + 1.  One masked DPP move per register (row_ror:8 is lane ^ 8 inside a row of 16; the bank
// mask picks the half of the row that takes the neighbour's value) puts every fragment where its MFMA reads it.
__device__ __forceinline__ void k_pair_home(const v4u& lo_rows, const v4u& hi_rows, half8& even, half8& odd) {
    v4u e, o;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int a = (int)lo_rows[j], b = (int)hi_rows[j];
        e[j] = (unsigned)__builtin_amdgcn_update_dpp(a, b, 0x128, 0xf, 0xc, false);
        o[j] = (unsigned)__builtin_amdgcn_update_dpp(b, a, 0x128, 0xf, 0x3, false);
    }
    even = __builtin_bit_cast(half8, e);
    odd = __builtin_bit_cast(half8, o);
}

// STEP: the row of cell pos comes from the caller's f32 K/V (stored under the f16 rule into the
// pool on the way): the pool ends up as bkv_append would leave it, the output as append + attend.
// SEL: the 16 rows of an iteration are four listed 4-cell blocks instead of a page (block g
// supplies the V rows of lane group g, block c / 4 the K row of lane c).
template <bool STEP, bool SEL = false, bool DESC = false>
__global__ __launch_bounds__(kBlock, 2) void decode_attn_mfma_kernel(const AttnKernelParams P) {
    static_assert(!(STEP && SEL), "the fused step attends the dense selection");
    __shared__ __attribute__((aligned(16))) MfmaFoldLds lds;

    // ---- which (entry, kv head, page range); one work-group per unit (no head chunks) --------
    const int unit = blockIdx.x;
    int e, rem, pos, row, pps;
    if (!unit_of_work_group<DESC>(P, unit, e, rem, pos, row, pps)) return;
    const int split = small_div(rem, P.inv_kv16);
    const int kvh = rem - split * P.n_kv;
    const int wg = unit;
    typedef const __attribute__((address_space(4))) int32_t* table_ptr;
    typedef const __attribute__((address_space(4))) uint32_t* list_ptr;
    const table_ptr bt = (table_ptr)(uintptr_t)(P.tables + (size_t)row * (size_t)P.max_pages_per_seq);
    uint32_t n_sel = 0;
    list_ptr sel = nullptr;
    if constexpr (SEL) {
        n_sel = min(((list_ptr)(uintptr_t)P.counts)[e], (uint32_t)P.max_ids);
        sel = (list_ptr)(uintptr_t)(P.ids + (size_t)e * (size_t)P.id_stride);
    }
    // loop iterations of this entry: pages, or groups of four selected blocks
    const int n_pages = SEL ? (int)((n_sel + 3u) >> 2) : pos / kPage + 1;
    const int pg0 = split * pps;
    const int pg1 = min(pg0 + pps, n_pages);

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int c = lane & 15;
    const int g = lane >> 4;
    const size_t page_bytes = (size_t)P.n_kv * kPage * kHd * 2;
    const size_t head_off = (size_t)kvh * kPage * kHd * 2;

    // Row runs of iteration i: a page, or four listed blocks whose ids
    // are clamped to the blocks at or below `pos` before any address is formed.
    const auto locate = [&](int i, RowRuns<SEL>& rr) {
        if constexpr (SEL) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t at = (uint32_t)i * 4u + (uint32_t)j;
                // the slot is read whether or not the list reaches it (the buffer holds max_ids slots per
                // entry): the read then does not wait for the list's length, one trip to memory less
                const uint32_t id = sel[min(at, (uint32_t)P.max_ids - 1u)];
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
    // K rows are fetched in whole 128-byte cache lines: for the pair of fragments (2 p, 2 p + 1) -- bytes
    // 128 p .. 128 p + 127 of a row -- one instruction reads rows 0..7 and one rows 8..15 of the iteration,
    // eight lanes to a row (lane (c, g) takes segment g + 4 (c / 8) of row c % 8, or of row 8 + c % 8).
    // Half of what a lane receives is its neighbour's eight columns away (c ^ 8); the two trade
    // places before use (k_fragments_home).  Fetched four lanes to a row, fragment by fragment, every
    // line was requested twice, half a line at a time, and the kernel streamed 4 to 7 % slower.
    const int c7 = c & 7;
    const auto k_row_of = [&](const RowRuns<SEL>& rr, int row) {
        return SEL ? pick(rr.k, row >> 2) + (size_t)(row & 3) * (kHd * 2) : rr.k[0] + (size_t)row * (kHd * 2);
    };
    const auto k_addr = [&](const uint8_t* row, int p) {
        return reinterpret_cast<const v4u*>(row + (size_t)(128 * p + 16 * (g + 4 * (c >> 3))));
    };
    // the first of this lane's four V rows (row 4 g)
    const auto v_rows = [&](const RowRuns<SEL>& rr) {
        return SEL ? pick(rr.v, g) : rr.v[0] + (size_t)(4 * g) * (kHd * 2);
    };
    const auto v_addr = [&](const uint8_t* rows, int h, int r) {
        return reinterpret_cast<const v4u*>(rows + (size_t)r * (kHd * 2) + (size_t)(h * 128 + c * 8) * 2);
    };

    int pg = pg0 + wave;
    v4u kf[8], vf[2][4];
    RowRuns<SEL> cur{};
    // a selection list's first rows are requested before its length is known (every address is clamped
    // to the sequence's own blocks, so rows past the list's end are merely unused)
    if (SEL || pg < pg1) {
        locate(pg, cur);
        const uint8_t* kp_lo = k_row_of(cur, c7);
        const uint8_t* kp_hi = k_row_of(cur, 8 + c7);
        const uint8_t* vp = v_rows(cur);
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            kf[2 * p] = __builtin_nontemporal_load(k_addr(kp_lo, p));
            kf[2 * p + 1] = __builtin_nontemporal_load(k_addr(kp_hi, p));
        }
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int r = 0; r < 4; ++r) vf[h][r] = __builtin_nontemporal_load(v_addr(vp, h, r));
    }

    // STEP: the wave that will hold the page of cell pos (in its last iteration) takes the new row now,
    // while its first pages are on their way: lane l < 32 converts slice l (8 values) of the K row, lane
    // 32 + l slice l of the V row, stores it into the pool (whole rows, 16 bytes a lane) and parks it in
    // the wave's part of the fold staging, which nothing else uses before the loop is over.  Fetched at
    // the last page instead, the row would add a trip to memory to the end of that work-group's walk.
    v4u* const new_row = reinterpret_cast<v4u*>(&lds.ow[wave][0][0]);
    if constexpr (STEP) {
        const int last = n_pages - 1;
        if (last >= pg0 && last < pg1 && ((last - pg0) & (kWaves - 1)) == wave) {
            const bool is_k = lane < 32;
            const int sl = lane & 31;
            const float* src = (is_k ? P.new_k : P.new_v) + ((size_t)e * P.n_kv + (size_t)kvh) * kHd + sl * 8;
            const float4 a = *reinterpret_cast<const float4*>(src);
            const float4 b = *reinterpret_cast<const float4*>(src + 4);
            v4u w;
            w.x = f16_store_pair(a.x, a.y), w.y = f16_store_pair(a.z, a.w);
            w.z = f16_store_pair(b.x, b.y), w.w = f16_store_pair(b.z, b.w);
            const size_t here = (size_t)bt[last] * page_bytes + head_off + (size_t)(pos & (kPage - 1)) * (kHd * 2);
            *reinterpret_cast<v4u*>((is_k ? P.kpool_w : P.vpool_w) + here + (size_t)sl * 16) = w;
            new_row[lane] = w;
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        }
    }

    half8 qhi[8], qlo[8];
    load_q_fragments(P, e, kvh, c, g, qhi, qlo);

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
        const uint8_t* kp_lo_next = nullptr;
        const uint8_t* kp_hi_next = nullptr;
        const uint8_t* vp_next = nullptr;
        if (more) {
            locate(pg_next, nxt);
            kp_lo_next = k_row_of(nxt, c7);
            kp_hi_next = k_row_of(nxt, 8 + c7);
            vp_next = v_rows(nxt);
        }

        if constexpr (STEP) {
            if (pg == n_pages - 1) {
                // This wave holds the page of cell pos; its pool row was stale when it was fetched.  The
                // lanes whose fragments are that row take the slices parked before the loop.
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                const int r = pos & (kPage - 1);
                // K registers hold rows as fetched: row r sits in the lanes with c % 8 == r % 8, in the
                // register of rows 0..7 or of rows 8..15, segment g + 4 (c / 8) of each 128-byte line
                const int seg = g + 4 * (c >> 3);
#pragma unroll
                for (int p = 0; p < 4; ++p) {
                    const v4u w = new_row[p * 8 + seg];
                    if (c7 == (r & 7)) {
                        if (r < 8) kf[2 * p] = w; else kf[2 * p + 1] = w;
                    }
                }
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const v4u w = new_row[32 + h * 16 + c];
                    if (g == (r >> 2)) {
#pragma unroll
                        for (int rr = 0; rr < 4; ++rr)
                            if (rr == (r & 3)) vf[h][rr] = w;
                    }
                }
            }
        }

        // ---- S^T = K . q^T: four independent accumulation chains ------------------------------
        f4 s0 = f4{0.0f, 0.0f, 0.0f, 0.0f}, s1 = s0, s2 = s0, s3 = s0;
#pragma unroll
        for (int m = 0; m < 8; m += 2) {
            half8 ka, kb;
            k_pair_home(kf[m], kf[m + 1], ka, kb);
            s0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka, qhi[m], s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka, qlo[m], s1, 0, 0, 0);
            s2 = __builtin_amdgcn_mfma_f32_16x16x32_f16(kb, qhi[m + 1], s2, 0, 0, 0);
            s3 = __builtin_amdgcn_mfma_f32_16x16x32_f16(kb, qlo[m + 1], s3, 0, 0, 0);
            if (more) {
                kf[m] = __builtin_nontemporal_load(k_addr(kp_lo_next, m >> 1));
                kf[m + 1] = __builtin_nontemporal_load(k_addr(kp_hi_next, m >> 1));
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
// (Multiplied on the VALU, this layout is bound by instruction issue: conversions and FMAs, 40 %
// of the HBM roofline on long contexts; here the VALU only converts and scales.)
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

// Data path: rows reach the matrix cores through LDS, because a lane's MFMA fragments are scattered
// over a row of codes and scales, but they travel there through registers: a wave fetches the K
// unit and the V unit of its next page (2 x 4352 bytes: one page and kv head, scales included) with
// ordinary coalesced loads -- 64 lanes x 16 contiguous bytes per instruction, whole cache lines, 17
// registers a unit -- while it multiplies the page before, and deposits them into its one LDS slot
// when it gets there.  (Direct global->LDS loads save the registers and the deposit, and stream
// 10 % slower on this chip: 6.0 against 6.7 TB/s for the same random 4 KiB chunks in this launch
// shape, measured with a probe; the kernel had been bound by that, not by its arithmetic.)
constexpr int kI8hUnit = kPage * row_bytes_of(kRowI8H);  // 4352
constexpr int kI8hSlot = 2 * kI8hUnit;                    // K unit, then V unit

// Where the 16 rows of one K or V unit come from: one run (a page's rows of one kv head), or, for a
// selection list, four runs of four rows (the listed blocks; crates/breccia-kernels/src/qsa/cpu.rs:
// 248-257).  In LDS the unit looks the same either way: a 16-byte piece at byte `off` of the unit
// comes from run off / RUN (row lengths are multiples of 16 bytes, so a piece never straddles runs).
template <bool SEL>
struct UnitSrc {
    const uint8_t* run[SEL ? 4 : 1];
};
template <bool SEL, int RUN>
__device__ __forceinline__ const uint8_t* unit_piece(const UnitSrc<SEL>& u, int off) {
    if constexpr (SEL) {
        const uint8_t* base = off >= 3 * RUN ? u.run[3] : off >= 2 * RUN ? u.run[2] : off >= RUN ? u.run[1] : u.run[0];
        const int j = (off >= RUN) + (off >= 2 * RUN) + (off >= 3 * RUN);
        return base + (off - j * RUN);
    } else {
        return u.run[0] + off;
    }
}
// The four listed blocks of loop iteration `it` of a selection list: ids for the causal test
// (0xffffffff past the end of the list) and, clamped to the blocks at or below `pos` before any
// address is formed, the byte offset of each block's rows inside a pool whose pages are
// `page_bytes` long and whose rows are `row_bytes` long.
typedef const __attribute__((address_space(4))) uint32_t* sel_list_ptr;
typedef const __attribute__((address_space(4))) int32_t* block_table_ptr;
__device__ __forceinline__ void listed_blocks(sel_list_ptr sel, uint32_t n_sel, uint32_t max_ids, block_table_ptr bt,
                                              int it, int pos, size_t page_bytes, size_t head_off, int row_bytes,
                                              uint32_t (&id)[4], size_t (&off)[4]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t at = (uint32_t)it * 4u + (uint32_t)j;
        // read whether or not the list reaches the slot (the buffer holds max_ids slots per entry): the
        // read does not wait for the list's length
        const uint32_t raw = sel[min(at, max_ids - 1u)];
        id[j] = at < n_sel ? raw : 0xffffffffu;
        const uint32_t idc = min(raw, (uint32_t)pos >> 2);
        off[j] = (size_t)bt[idc >> 2] * page_bytes + head_off + (size_t)(idc & 3u) * 4u * (size_t)row_bytes;
    }
}
__device__ __forceinline__ uint32_t pick4(const uint32_t (&a)[4], int j) {
    return j == 0 ? a[0] : j == 1 ? a[1] : j == 2 ? a[2] : a[3];
}

// One unit between memory and LDS: 4352 bytes = 64 lanes x (4 x 16 + 4).
struct I8hUnitRegs {
    v4u q[4];
    unsigned tail;
};
template <bool SEL>
__device__ __forceinline__ void i8h_unit_fetch(const UnitSrc<SEL>& src, int lane, I8hUnitRegs& r) {
    constexpr int kRun = 4 * row_bytes_of(kRowI8H);
#pragma unroll
    for (int n = 0; n < 4; ++n)
        r.q[n] = __builtin_nontemporal_load(reinterpret_cast<const v4u*>(unit_piece<SEL, kRun>(src, n * 1024 + lane * 16)));
    r.tail = __builtin_nontemporal_load(reinterpret_cast<const unsigned*>(unit_piece<SEL, kRun>(src, 4096 + lane * 4)));
}
__device__ __forceinline__ void i8h_unit_deposit(const I8hUnitRegs& r, uint8_t* dst, int lane) {
#pragma unroll
    for (int n = 0; n < 4; ++n) *reinterpret_cast<v4u*>(dst + n * 1024 + lane * 16) = r.q[n];
    *reinterpret_cast<unsigned*>(dst + 4096 + lane * 4) = r.tail;
}

// SEL: an iteration's 16 rows are four listed 4-cell blocks (see decode_attn_mfma_kernel); the
// work is planned for max_ids blocks, a work-group past the end of the list has nothing to do.
template <bool STEP, bool DESC = false, bool SEL = false>
__global__ __launch_bounds__(kBlock, 2) void decode_attn_mfma_i8h_kernel(const AttnKernelParams P) {
    static_assert(!(STEP && SEL), "the fused step attends the dense selection");
    // one slot per wave; the fold staging of the epilogue reuses the memory
    constexpr int kRing = kWaves * kI8hSlot > (int)sizeof(MfmaFoldLds) ? kWaves * kI8hSlot : (int)sizeof(MfmaFoldLds);
    __shared__ __attribute__((aligned(16))) uint8_t ring[kRing];
    constexpr int kRow = row_bytes_of(kRowI8H);  // 272
    // STEP: the new K row and the new V row of the entry, encoded; one wave of a work-group at most
    __shared__ __attribute__((aligned(16))) uint8_t parked[STEP ? 2 * kRow : 16];

    const int unit = blockIdx.x;
    int e, rem, pos, row, pps;
    if (!unit_of_work_group<DESC>(P, unit, e, rem, pos, row, pps)) return;
    const int split = small_div(rem, P.inv_kv16);
    const int kvh = rem - split * P.n_kv;
    const int wg = unit;
    const block_table_ptr bt = (block_table_ptr)(uintptr_t)(P.tables + (size_t)row * (size_t)P.max_pages_per_seq);
    uint32_t n_sel = 0;
    sel_list_ptr sel = nullptr;
    if constexpr (SEL) {
        n_sel = min(((sel_list_ptr)(uintptr_t)P.counts)[e], (uint32_t)P.max_ids);
        sel = (sel_list_ptr)(uintptr_t)(P.ids + (size_t)e * (size_t)P.id_stride);
    }
    // loop iterations of this entry: pages, or groups of four selected blocks
    const int n_pages = SEL ? (int)((n_sel + 3u) >> 2) : pos / kPage + 1;
    const int pg0 = split * pps;
    const int pg1 = min(pg0 + pps, n_pages);

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int c = lane & 15;
    const int g = lane >> 4;
    const int my_block = c >> 2;  // which of the 4 blocks of a half this lane's 8 columns lie in
    const size_t page_bytes = (size_t)P.n_kv * kI8hUnit;
    const size_t head_off = (size_t)kvh * kI8hUnit;
    uint8_t* const slot = ring + wave * kI8hSlot;

    // pipeline steps of this wave: pages pg0 + wave, + kWaves, ...
    const int n_steps = pg0 + wave < pg1 ? (pg1 - pg0 - wave + kWaves - 1) / kWaves : 0;
    const auto unit_off = [&](int i) -> size_t {
        return (size_t)bt[min(pg0 + wave + kWaves * i, pg1 - 1)] * page_bytes + head_off;
    };
    // the K and the V unit of step i (both pools have the same geometry in this layout)
    const auto unit_src = [&](int i, const uint8_t* pool, UnitSrc<SEL>& u) {
        if constexpr (SEL) {
            // whatever the step, listed or past the list's end: every address is clamped to the sequence's
            // own blocks, and nothing here waits for the list's length
            uint32_t id[4];
            size_t off[4];
            listed_blocks(sel, n_sel, (uint32_t)P.max_ids, bt, pg0 + wave + kWaves * i, pos, page_bytes, head_off, kRow, id, off);
#pragma unroll
            for (int j = 0; j < 4; ++j) u.run[j] = pool + off[j];
        } else {
            u.run[0] = pool + (n_steps > 0 ? unit_off(i) : 0);
        }
    };
    // the page in flight: requested while the page before is multiplied
    I8hUnitRegs k_regs, v_regs;
    const auto fetch = [&](int i) {
        UnitSrc<SEL> u;
        unit_src(i, P.kpool, u);
        i8h_unit_fetch<SEL>(u, lane, k_regs);
        unit_src(i, P.vpool, u);
        i8h_unit_fetch<SEL>(u, lane, v_regs);
    };
    if (SEL || n_steps > 0) fetch(0);  // a selection list's first units before its length is known

    // STEP: the wave that will hold the page of cell pos (in its last step) takes the new rows before the
    // loop, while its first units are on their way: the raw values are requested ahead of the q fragments
    // (one wait covers both), then lanes 0..7 encode the K row and lanes 8..15 the V row with the append
    // kernel's encoder, one lane per 32-value block, into the pool and into two parking rows in LDS.  In
    // its last step the wave copies a parked row into the unit that has just landed (an LDS move instead
    // of a trip to memory and an encode at the end of the work-group's walk).
    const auto wave_lds_fence = [&]() {
        // the wave's own LDS writes are in order with its later reads; keep the compiler from
        // moving those reads up
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };
    const bool takes_new_row = STEP && n_steps > 0 && pg0 + wave + kWaves * (n_steps - 1) == n_pages - 1;
    float new_x[32];
    if constexpr (STEP) {
        if (takes_new_row && lane < 16) {
            const float* src = (lane < 8 ? P.new_k : P.new_v) + ((size_t)e * P.n_kv + (size_t)kvh) * kHd + (lane & 7) * 32;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float4 a = *reinterpret_cast<const float4*>(src + 4 * j);
                new_x[4 * j] = a.x, new_x[4 * j + 1] = a.y, new_x[4 * j + 2] = a.z, new_x[4 * j + 3] = a.w;
            }
        }
    }

    half8 qhi[8], qlo[8];
    load_q_fragments(P, e, kvh, c, g, qhi, qlo);

    if constexpr (STEP) {
        if (takes_new_row) {
            if (lane < 16) {
                uint32_t w[8], hb;
                i8h_block_words(new_x, w, hb);
                const int r = pos & (kPage - 1);
                const int blk = lane & 7;
                uint8_t* const pool_row = (lane < 8 ? P.kpool_w : P.vpool_w) + unit_off(n_steps - 1) + (size_t)r * kRow;
                uint8_t* const rows[2] = {parked + (lane < 8 ? 0 : kRow), pool_row};
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    *reinterpret_cast<v4u*>(rows[t] + blk * 32) = v4u{w[0], w[1], w[2], w[3]};
                    *reinterpret_cast<v4u*>(rows[t] + blk * 32 + 16) = v4u{w[4], w[5], w[6], w[7]};
                    *reinterpret_cast<unsigned short*>(rows[t] + kHd + 2 * blk) = (unsigned short)hb;
                }
            }
            wave_lds_fence();
        }
    }

    f4 o[2][8];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int t = 0; t < 8; ++t) o[h][t] = f4{0.0f, 0.0f, 0.0f, 0.0f};
    float m_run = -INFINITY;
    float l_run = 0.0f;

    // the parked row `which` (0 = K, 1 = V) into row pos % 16 of the unit that has just landed
    const auto take_new_row = [&](int which, uint8_t* lds_unit) {
        const int r = pos & (kPage - 1);
        if (lane < kRow / 16)
            *reinterpret_cast<v4u*>(lds_unit + r * kRow + lane * 16) =
                *reinterpret_cast<const v4u*>(parked + which * kRow + lane * 16);
        wave_lds_fence();
    };

    // One page: step i of the wave.  Its units arrive in the registers; they go into the slot and the
    // registers take the request for step i + 1.
    const auto one_page = [&](int i) __attribute__((always_inline)) {
        const int pg = pg0 + wave + kWaves * i;
        const uint8_t* ks = slot;
        const uint8_t* vs = slot + kI8hUnit;
        i8h_unit_deposit(k_regs, slot, lane);
        i8h_unit_deposit(v_regs, slot + kI8hUnit, lane);
        if (i + 1 < n_steps) fetch(i + 1);
        wave_lds_fence();
        if constexpr (STEP) {
            if (pg == n_pages - 1) {
                take_new_row(0, slot);
                take_new_row(1, slot + kI8hUnit);
            }
        }
        // which of the lane's four cells are attended: up to `pos`, or the live cells of listed blocks
        bool live[4];
        if constexpr (SEL) {
            uint32_t id[4];
            size_t unused[4];
            listed_blocks(sel, n_sel, (uint32_t)P.max_ids, bt, pg, pos, page_bytes, head_off, kRow, id, unused);
            const uint32_t mine = pick4(id, g);
#pragma unroll
            for (int r = 0; r < 4; ++r) live[r] = block_cell_live(mine, r, pos);
        } else {
#pragma unroll
            for (int r = 0; r < 4; ++r) live[r] = pg * kPage + 4 * g + r <= pos;
        }

        // ---- scores: per block, codes . q on the matrix core, then the block's scale ----------------
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

        // ---- this page's V fragments are requested before the softmax, whose chain of dependent
        // instructions then has the dequantisation to overlap with -----------------------------------
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

        // ---- online softmax of head c ---------------------------------------------------------------
        float t4[4];
        float pm = -INFINITY;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            t4[r] = live[r] ? s[r] * P.scale_log2e : -INFINITY;
            pm = fmaxf(pm, t4[r]);
        }
        pm = max_over_lane_groups(pm);
        // dense: finite, every page of a range holds a live cell; a group of listed blocks may be dead
        // as a whole, and exp2(-inf - -inf) would be NaN
        const float m_new = fmaxf(m_run, pm);
        const bool none_yet = SEL && m_new == -INFINITY;
        const float alpha = none_yet ? 1.0f : __builtin_amdgcn_exp2f(m_run - m_new);
        float p[4];
        float psum = 0.0f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            p[r] = none_yet ? 0.0f : __builtin_amdgcn_exp2f(t4[r] - m_new);
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
        const bool last_page = SEL || pg == n_pages - 1;
        if (last_page || __builtin_amdgcn_ballot_w64(has_zero_exponent(v_screen)) != 0) {
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if ((vsb[h][r] & 0x7c00u) == 0 || !live[r]) vsb[h][r] = 0;
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
    };

    for (int i = 0; i < n_steps; ++i) one_page(i);

    // every wave is done with its slot before the fold staging takes their place
    __syncthreads();
    mfma_fold_and_store(P, *reinterpret_cast<MfmaFoldLds*>(ring), wg, wave, c, g, o, m_run, l_run);
}

// ---- decode attention on the matrix cores, f16 K and q8_0 V -----------------------------------
// The MFMA decomposition of decode_attn_mfma_kernel.  K is f16 and takes that kernel's way: whole
// 128-byte lines straight into the fragment registers (k_pair_home), refilled with the next page's
// as they are used up.  The V unit ([f32 scale][32 x i8] blocks, 288 bytes a row) is staged through
// LDS like the int8 kernel's units: the next page's unit is fetched into registers with coalesced
// loads while this page is multiplied, and deposited into the wave's slot when the page is reached.
// A q8_0 value is code * scale with an f32 scale, so it takes a per-cell
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

// A V unit: 4608 bytes = 64 lanes x (4 x 16 + 8).
struct Q8vUnitRegs {
    v4u q[4];
    v2u tail;
};
template <bool SEL>
__device__ __forceinline__ void q8v_unit_fetch(const UnitSrc<SEL>& src, int lane, Q8vUnitRegs& r) {
    constexpr int kRun = 4 * kQ8vRow;
#pragma unroll
    for (int n = 0; n < 4; ++n)
        r.q[n] = __builtin_nontemporal_load(reinterpret_cast<const v4u*>(unit_piece<SEL, kRun>(src, n * 1024 + lane * 16)));
    r.tail = __builtin_nontemporal_load(reinterpret_cast<const v2u*>(unit_piece<SEL, kRun>(src, 4096 + lane * 8)));
}
__device__ __forceinline__ void q8v_unit_deposit(const Q8vUnitRegs& r, uint8_t* dst, int lane) {
#pragma unroll
    for (int n = 0; n < 4; ++n) *reinterpret_cast<v4u*>(dst + n * 1024 + lane * 16) = r.q[n];
    *reinterpret_cast<v2u*>(dst + 4096 + lane * 8) = r.tail;
}

// SEL: an iteration's 16 rows are four listed 4-cell blocks, as in the int8 kernel.
template <bool STEP, bool DESC = false, bool SEL = false>
__global__ __launch_bounds__(kBlock, 2) void decode_attn_mfma_q8v_kernel(const AttnKernelParams P) {
    static_assert(!(STEP && SEL), "the fused step attends the dense selection");
    // per wave one V slot during the loop, the fold staging after it
    constexpr int kWaveLds = kQ8vUnit;
    constexpr int kLds = kWaves * kWaveLds > (int)sizeof(MfmaFoldLds) ? kWaves * kWaveLds : (int)sizeof(MfmaFoldLds);
    __shared__ __attribute__((aligned(16))) uint8_t smem[kLds];
    // STEP: the new row of the entry, encoded (512 bytes of K, 288 of V); one wave of a work-group at most
    __shared__ __attribute__((aligned(16))) uint8_t parked[STEP ? 512 + kQ8vRow : 16];

    const int unit = blockIdx.x;
    int e, rem, pos, row, pps;
    if (!unit_of_work_group<DESC>(P, unit, e, rem, pos, row, pps)) return;
    const int split = small_div(rem, P.inv_kv16);
    const int kvh = rem - split * P.n_kv;
    const int wg = unit;
    const block_table_ptr bt = (block_table_ptr)(uintptr_t)(P.tables + (size_t)row * (size_t)P.max_pages_per_seq);
    uint32_t n_sel = 0;
    sel_list_ptr sel = nullptr;
    if constexpr (SEL) {
        n_sel = min(((sel_list_ptr)(uintptr_t)P.counts)[e], (uint32_t)P.max_ids);
        sel = (sel_list_ptr)(uintptr_t)(P.ids + (size_t)e * (size_t)P.id_stride);
    }
    const int n_pages = SEL ? (int)((n_sel + 3u) >> 2) : pos / kPage + 1;
    const int pg0 = split * pps;
    const int pg1 = min(pg0 + pps, n_pages);

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int c = lane & 15;
    const int g = lane >> 4;
    const size_t k_page_bytes = (size_t)P.n_kv * kPage * kHd * 2;
    const size_t k_head_off = (size_t)kvh * kPage * kHd * 2;
    const size_t v_page_bytes = (size_t)P.n_kv * kQ8vUnit;
    const size_t v_head_off = (size_t)kvh * kQ8vUnit;
    uint8_t* const slots = smem + wave * kWaveLds;

    // pipeline steps of this wave: pages pg0 + wave, + kWaves, ...
    const int n_steps = pg0 + wave < pg1 ? (pg1 - pg0 - wave + kWaves - 1) / kWaves : 0;
    // physical page of step i; past the wave's last step the answer is not used for its data
    const auto phys = [&](int i) -> size_t { return (size_t)bt[min(pg0 + wave + kWaves * i, pg1 - 1)]; };

    const auto unit_src = [&](int i, bool is_k, UnitSrc<SEL>& u) {
        const uint8_t* pool = is_k ? P.kpool : P.vpool;
        if constexpr (SEL) {
            // whatever the step, listed or past the list's end: every address is clamped to the sequence's
            // own blocks, and nothing here waits for the list's length
            uint32_t id[4];
            size_t off[4];
            listed_blocks(sel, n_sel, (uint32_t)P.max_ids, bt, pg0 + wave + kWaves * i, pos, is_k ? k_page_bytes : v_page_bytes,
                          is_k ? k_head_off : v_head_off, is_k ? kHd * 2 : kQ8vRow, id, off);
#pragma unroll
            for (int j = 0; j < 4; ++j) u.run[j] = pool + off[j];
        } else {
            u.run[0] = n_steps > 0 ? pool + phys(i) * (is_k ? k_page_bytes : v_page_bytes) + (is_k ? k_head_off : v_head_off)
                                   : pool;
        }
    };
    // K rows are fetched in whole 128-byte lines, as in decode_attn_mfma_kernel: for the pair of fragments
    // (2 p, 2 p + 1) one instruction reads rows 0..7 and one rows 8..15 of the page, eight lanes to a row
    // (lane (c, g) takes segment g + 4 (c / 8) of row c % 8, or of row 8 + c % 8); k_pair_home puts the
    // halves where their MFMAs read them.
    const int c7 = c & 7;
    const int kseg = g + 4 * (c >> 3);
    const auto k_rows = [&](const UnitSrc<SEL>& u, const uint8_t*& lo, const uint8_t*& hi) {
        if constexpr (SEL) {
            // rows 4 j .. 4 j + 3 of the iteration are listed block j
            const int at = (c7 & 3) * (kHd * 2) + kseg * 16;
            lo = (c7 >> 2 ? u.run[1] : u.run[0]) + at;
            hi = (c7 >> 2 ? u.run[3] : u.run[2]) + at;
        } else {
            lo = u.run[0] + c7 * (kHd * 2) + kseg * 16;
            hi = lo + 8 * (kHd * 2);
        }
    };
    // the page in flight: K in the fragment registers, refilled as they are used up; the V unit requested
    // while the page before is multiplied
    v4u kf[8];
    Q8vUnitRegs v_regs;
    if (SEL || n_steps > 0) {  // a selection list's first units before its length is known
        UnitSrc<SEL> u;
        const uint8_t *lo, *hi;
        unit_src(0, true, u);
        k_rows(u, lo, hi);
#pragma unroll
        for (int pp = 0; pp < 4; ++pp) {
            kf[2 * pp] = __builtin_nontemporal_load(reinterpret_cast<const v4u*>(lo + 128 * pp));
            kf[2 * pp + 1] = __builtin_nontemporal_load(reinterpret_cast<const v4u*>(hi + 128 * pp));
        }
        unit_src(0, false, u);
        q8v_unit_fetch<SEL>(u, lane, v_regs);
    }

    // STEP: the wave that will hold the page of cell pos (in its last step) encodes the new row before
    // the loop, while its first units are on their way, as the append kernel does -- K under the f16
    // rule, 8 values a lane; V as q8_0 blocks, one lane per block -- into the pool and into a parking
    // row in LDS; in its last step it copies the parked row into the unit that has just landed (two LDS
    // moves instead of a trip to memory and an encode at the end of the work-group's walk).
    const auto wave_lds_fence = [&]() {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };
    // the raw values are requested ahead of the q fragments (one wait covers both) and encoded after them
    const bool takes_new_row = STEP && n_steps > 0 && pg0 + wave + kWaves * (n_steps - 1) == n_pages - 1;
    float new_x[32];
    if constexpr (STEP) {
        if (takes_new_row) {
            if (lane < 32) {
                const float* src = P.new_k + ((size_t)e * P.n_kv + (size_t)kvh) * kHd + lane * 8;
                const float4 a = *reinterpret_cast<const float4*>(src);
                const float4 b = *reinterpret_cast<const float4*>(src + 4);
                new_x[0] = a.x, new_x[1] = a.y, new_x[2] = a.z, new_x[3] = a.w;
                new_x[4] = b.x, new_x[5] = b.y, new_x[6] = b.z, new_x[7] = b.w;
            } else if (lane < 40) {
                const float* src = P.new_v + ((size_t)e * P.n_kv + (size_t)kvh) * kHd + (lane - 32) * 32;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float4 a = *reinterpret_cast<const float4*>(src + 4 * j);
                    new_x[4 * j] = a.x, new_x[4 * j + 1] = a.y, new_x[4 * j + 2] = a.z, new_x[4 * j + 3] = a.w;
                }
            }
        }
    }

    half8 qhi[8], qlo[8];
    load_q_fragments(P, e, kvh, c, g, qhi, qlo);

    if constexpr (STEP) {
        if (takes_new_row) {
            const int r = pos & (kPage - 1);
            const int i = n_steps - 1;
            if (lane < 32) {
                v4u w;
                w.x = f16_store_pair(new_x[0], new_x[1]), w.y = f16_store_pair(new_x[2], new_x[3]);
                w.z = f16_store_pair(new_x[4], new_x[5]), w.w = f16_store_pair(new_x[6], new_x[7]);
                *reinterpret_cast<v4u*>(parked + lane * 16) = w;
                *reinterpret_cast<v4u*>(P.kpool_w + phys(i) * k_page_bytes + k_head_off + (size_t)r * 512 + lane * 16) = w;
            } else if (lane < 40) {
                const int blk = lane - 32;
                uint32_t w[9];
                q8v_block_words(new_x, w);
                uint32_t* const ld = reinterpret_cast<uint32_t*>(parked + 512 + blk * 36);
                uint32_t* const gd = reinterpret_cast<uint32_t*>(P.vpool_w + phys(i) * v_page_bytes + v_head_off +
                                                                  (size_t)r * kQ8vRow + blk * 36);
#pragma unroll
                for (int j = 0; j < 9; ++j) {
                    ld[j] = w[j];
                    gd[j] = w[j];
                }
            }
            wave_lds_fence();
        }
    }
    // K registers hold rows as fetched: row r sits in the lanes with c % 8 == r % 8, in the register of
    // rows 0..7 or of rows 8..15, segment g + 4 (c / 8) of each 128-byte line
    const auto take_new_k = [&]() {
        const int r = pos & (kPage - 1);
#pragma unroll
        for (int pp = 0; pp < 4; ++pp) {
            const v4u w = *reinterpret_cast<const v4u*>(parked + (pp * 8 + kseg) * 16);
            if (c7 == (r & 7)) {
                if (r < 8) kf[2 * pp] = w; else kf[2 * pp + 1] = w;
            }
        }
    };
    const auto take_new_v = [&](uint8_t* lds_unit) {
        const int r = pos & (kPage - 1);
        if (lane < kQ8vRow / 16)
            *reinterpret_cast<v4u*>(lds_unit + r * kQ8vRow + lane * 16) =
                *reinterpret_cast<const v4u*>(parked + 512 + lane * 16);
        wave_lds_fence();
    };

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
        const uint8_t* vs = slots;
        // this page's V unit arrives in the registers: into the slot with it, and the registers take the
        // request for the next page's
        q8v_unit_deposit(v_regs, slots, lane);
        const bool more = i + 1 < n_steps;
        const uint8_t* klo_next = nullptr;
        const uint8_t* khi_next = nullptr;
        if (more) {
            UnitSrc<SEL> u;
            unit_src(i + 1, false, u);
            q8v_unit_fetch<SEL>(u, lane, v_regs);
            unit_src(i + 1, true, u);
            k_rows(u, klo_next, khi_next);
        }
        wave_lds_fence();
        if constexpr (STEP) {
            if (pg == n_pages - 1) {
                take_new_k();
                take_new_v(slots);
            }
        }
        bool live[4];       // the lane's cells 4 g + r
        bool live_mine;     // cell 4 g + c % 4
        if constexpr (SEL) {
            uint32_t id[4];
            size_t unused[4];
            listed_blocks(sel, n_sel, (uint32_t)P.max_ids, bt, pg, pos, k_page_bytes, k_head_off, kHd * 2, id, unused);
            const uint32_t mine = pick4(id, g);
#pragma unroll
            for (int r = 0; r < 4; ++r) live[r] = block_cell_live(mine, r, pos);
            live_mine = block_cell_live(mine, c & 3, pos);
        } else {
#pragma unroll
            for (int r = 0; r < 4; ++r) live[r] = pg * kPage + 4 * g + r <= pos;
            live_mine = pg * kPage + 4 * g + (c & 3) <= pos;
        }

        // ---- S^T = K . q^T: four independent accumulation chains ------------------------------
        f4 s0 = f4{0.0f, 0.0f, 0.0f, 0.0f}, s1 = s0, s2 = s0, s3 = s0;
#pragma unroll
        for (int m = 0; m < 8; m += 2) {
            half8 ka, kb;
            k_pair_home(kf[m], kf[m + 1], ka, kb);
            s0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka, qhi[m], s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka, qlo[m], s1, 0, 0, 0);
            s2 = __builtin_amdgcn_mfma_f32_16x16x32_f16(kb, qhi[m + 1], s2, 0, 0, 0);
            s3 = __builtin_amdgcn_mfma_f32_16x16x32_f16(kb, qlo[m + 1], s3, 0, 0, 0);
            if (more) {
                kf[m] = __builtin_nontemporal_load(reinterpret_cast<const v4u*>(klo_next + 64 * m));
                kf[m + 1] = __builtin_nontemporal_load(reinterpret_cast<const v4u*>(khi_next + 64 * m));
            }
        }
        const f4 s = (s0 + s1) + (s2 + s3);  // s[r] = q[head c] . k[cell 4 g + r]

        // ---- this page's V unit: scales first -------------------------------------------------
        // lane (c, g): scale of blocks 2 (c / 4), + 1 of row 4 g + c % 4, the row's maximum over the
        // lanes c, c ^ 4, c ^ 8, c ^ 12, then the four rows' maxima from the lanes of the quad
        const bool last_page = SEL || pg == n_pages - 1;
        float smax;
        {
            const uint8_t* rp = vs + (4 * g + (c & 3)) * kQ8vRow + (c >> 2) * 72;
            const float a = *reinterpret_cast<const float*>(rp);
            const float b = *reinterpret_cast<const float*>(rp + 36);
            smax = fmaxf(a, b);
            // rows past `pos` may hold anything: they count as scale 1 here and as zeros below
            if (last_page && !live_mine) smax = 1.0f;
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
            t4[r] = live[r] ? s[r] * P.scale_log2e : -INFINITY;
            tw[r] = t4[r] + (float)ex[r];
            pm = fmaxf(pm, tw[r]);
        }
        pm = max_over_lane_groups(pm);
        // dense: finite, every page of a range holds a live cell; a group of listed blocks may be dead
        // as a whole, and exp2(-inf - -inf) would be NaN
        const float m_new = fmaxf(m_run, pm);
        const bool none_yet = SEL && m_new == -INFINITY;
        const float alpha = none_yet ? 1.0f : __builtin_amdgcn_exp2f(m_run - m_new);
        h4m whi, wlo;
        float psum = 0.0f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float w = none_yet ? 0.0f : __builtin_amdgcn_exp2f(tw[r] - m_new);
            psum = fmaf(w, down[r], psum);  // exp2(logit - m_new) = w * 2^-E: no second exponential
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
                if (last_page && !live[r]) sc = 0.0f;
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
    }

    // every wave is done with its slots before the fold staging takes their place
    __syncthreads();
    mfma_fold_and_store(P, *reinterpret_cast<MfmaFoldLds*>(smem), wg, wave, c, g, o, m_run, l_run);
}

}  // namespace

// With `start` / `stop` the two events are attached to the dispatch itself (they take the kernel's
// own begin and end time stamps, what a profiler's kernel trace reports), otherwise a plain launch.
template <typename K>
static void launch_one(K kernel, const AttnKernelParams& kp, int32_t total, hipStream_t stream, hipEvent_t start,
                       hipEvent_t stop) {
    if (start && stop)
        hipExtLaunchKernelGGL(kernel, dim3((unsigned)total), dim3(kBlock), 0, stream, start, stop, 0, kp);
    else
        kernel<<<total, kBlock, 0, stream>>>(kp);
}

hipError_t launch_decode_attn_mfma(const AttnKernelParams& kp, int layout, bool step, bool sel, int32_t total,
                                   hipStream_t stream, hipEvent_t start, hipEvent_t stop) {
    if (kp.bd) {
        // the batch comes from the device-resident descriptor: the fused step only
        if (!step || sel) return hipErrorInvalidValue;
        if (layout == BKV_LAYOUT_I8H)
            launch_one(decode_attn_mfma_i8h_kernel<true, true>, kp, total, stream, start, stop);
        else if (layout == BKV_LAYOUT_Q8V)
            launch_one(decode_attn_mfma_q8v_kernel<true, true>, kp, total, stream, start, stop);
        else
            launch_one(decode_attn_mfma_kernel<true, false, true>, kp, total, stream, start, stop);
        return hipGetLastError();
    }
    if (layout == BKV_LAYOUT_I8H) {
        if (step)
            launch_one(decode_attn_mfma_i8h_kernel<true>, kp, total, stream, start, stop);
        else if (sel)
            launch_one(decode_attn_mfma_i8h_kernel<false, false, true>, kp, total, stream, start, stop);
        else
            launch_one(decode_attn_mfma_i8h_kernel<false>, kp, total, stream, start, stop);
    } else if (layout == BKV_LAYOUT_Q8V) {
        if (step)
            launch_one(decode_attn_mfma_q8v_kernel<true>, kp, total, stream, start, stop);
        else if (sel)
            launch_one(decode_attn_mfma_q8v_kernel<false, false, true>, kp, total, stream, start, stop);
        else
            launch_one(decode_attn_mfma_q8v_kernel<false>, kp, total, stream, start, stop);
    } else if (step)
        launch_one(decode_attn_mfma_kernel<true, false>, kp, total, stream, start, stop);
    else if (sel)
        launch_one(decode_attn_mfma_kernel<false, true>, kp, total, stream, start, stop);
    else
        launch_one(decode_attn_mfma_kernel<false, false>, kp, total, stream, start, stop);
    return hipGetLastError();
}

}  // namespace bkv
