// Paged causal attention for chunks of many query tokens (prefill) on gfx950 matrix cores.
// The reference's counterpart is its GQA pair for T >= 16 (crates/breccia-kernels/shaders/
// qsa_attn_scores_gqa.comp, qsa_attn_apply_gqa.comp; qsa/mod.rs:116-150); the contract is the
// CPU attend (qsa/cpu.rs:197-246) with the dense selection: query token t of a chunk that
// starts at pos0 attends cells 0..pos0+t.
//
// With hundreds of query rows per kv head the work is a real matrix product (each K/V row is
// used by every query row behind it), so it goes to MFMA -- unlike the decode kernel, which
// is a GEMV per sequence.  A work-group of four waves owns 64 consecutive query rows ((token,
// head) pairs of one kv head), 16 per wave, and walks the pages 0..page(pos) together: each
// page's K and V rows are fetched from memory once per work-group into LDS (double-buffered,
// the next page in flight while the current one is multiplied; fetching them per wave ran into
// the L2's bandwidth), and every wave takes its operand fragments from there.  Per page of 16
// cells and per wave:
//   S^T[cell][query] = K[cell][:] . Q[query][:]        v_mfma_f32_16x16x32_f16, A = K, B = Q
//   online softmax per query (base 2), P^T in the layout S^T came out in
//   O^T[d][query]   += V^T[d][cell] . P^T[cell][query]  v_mfma_f32_16x16x32_f16 over the 32 cells of
//                                                       two pages, A = V gathered per lane (four
//                                                       cells of either page), B = P^T, high parts
//                                                       and low parts in one MFMA each
// Both products keep the per-lane query (lane % 16) fixed, so the softmax statistics never
// move between lanes, and P^T feeds the second product straight from registers.  K and V are
// exact f16; q and p are f32 values split into a high and a low f16 part (two MFMAs each), so the
// products carry ~22 significant bits and the result stays at f32-accumulate accuracy.  Pages are
// walked two at a time: one softmax update and one barrier per pair.
// The V operand needs, per lane, four cells of one head-dim column of either page: a column of
// the row-major page image.  gfx950's transposing LDS read (ds_read_b64_tr_b16) delivers exactly
// that: within a group of 16 lanes, lane L receives element L % 4 of the 8-byte pieces that lanes
// L / 4, 4 + L / 4, 8 + L / 4 and 12 + L / 4 addressed.  With lane (c, g) addressing row 4 g + c / 4,
// halves 4 (c % 4) .. of a tile of 16 columns, lane c receives column c of the tile for cells
// 4 g .. 4 g + 3: the MFMA operand, no regrouping on the VALU.  The V images have rows of 544
// bytes (8 banks apart: the 64 lanes' 8-byte pieces of such a read tile the banks exactly).
//
// Pools with q8_0 V ([f32 scale][32 x i8] blocks, qsa_attn_apply_gqa.comp:53-77) take the same
// walk with work-groups of eight waves: the threads that fetch a V page dequantise it once for
// all eight, on its way into LDS, into two f16 images whose sum is the value to 22 bits
//   E[cell]    = exponent of the largest of the cell's 8 block scales (clamped to +-120),
//   a[cell][d] = code * (scale * 2^-E[cell]) = hi + lo,
// and the softmax runs over logit + E with weights exp2(logit + E - M) (the denominator sums
// exp2(logit - M)), as in the decode kernel for this layout: the largest terms have weights near
// 1 whatever the magnitude of their values.  P.V is then hi.p_hi + hi.p_lo + lo.p_hi.
// Int8 pools (codes with an f16 scale per 32 values, K and V alike) are dequantised the same way,
// without the exponent: both K and V become hi/lo image pairs, and the scores are
// K_hi.q_hi + K_hi.q_lo + K_lo.q_hi.
#include <algorithm>

#include "bkv_internal.hpp"
#include "lane_groups.hpp"
#include "quant_decode.hpp"

namespace bkv {

namespace {

constexpr int kHd = 256;
constexpr int kPage = 16;
constexpr int kRowsPerWave = 16;
constexpr int kQ8vRow = kHd / 32 * 36;  // bytes of a q8_0 row
constexpr int kI8hRow = kHd + kHd / 32 * 2;  // bytes of an int8 row: codes, then 8 f16 scales
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLoDown = 1.0f / 2048.0f;  // q's low parts enter the products times 2^11
constexpr int kLdsRow = kHd + 8;    // halves per row of a K page image in LDS (528 bytes)
constexpr int kLdsRowV = kHd + 16;  // of a V page image (544 bytes)

typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));
typedef short tr_s4 __attribute__((__vector_size__(8)));  // what the transposing LDS read returns
typedef __attribute__((address_space(3))) tr_s4* lds_tr_ptr;

struct PrefillKernelParams {
    PrefillBatch b;
    const uint8_t* kpool;
    const uint8_t* vpool;
    const int32_t* tables;
    const float* q;     // [sum n_tok][n_q][256]
    const float* gate;  // optional
    float* out;         // [sum n_tok][n_q][256]
    int64_t gate_tok_stride, gate_head_stride;
    int32_t max_pages_per_seq, n_kv, n_q, group;
    float scale_log2e;
    int32_t by_xcd;  // work-groups are dealt to the chip's 8 dies so that each die sees few (entry, kv head) units
};

// The chip is 8 dies (XCDs), each with an L2 of its own, and work-group i runs on die i % 8.
// Every work-group of one (entry, kv head) unit walks the same K/V pages, so the dies are given
// whole units: with 8 or more units, die x serves units x, x + 8, ...; with fewer, unit u is
// served by dies u, u + U, ...  A unit's pages then stay in one die's L2 (3 MiB for a 3072-token
// chunk) instead of every die fetching every unit through the fabric.
constexpr int kXcds = 8;

// gfx950's double-depth form: 32 contraction steps, 8 halves per lane (k = 8 (lane / 16) + 0..7)
__device__ __forceinline__ f4 mfma32(h8 a, h8 b, f4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ void split_f16(float x, _Float16& hi, _Float16& lo) {
    hi = (_Float16)x;
    lo = (_Float16)(x - (float)hi);
}

// What a thread carries of one page between its fetch and its deposit into LDS.
template <int LAY>
struct PageStage;
template <>
struct PageStage<BKV_LAYOUT_F16> {
    v4u k[2], v[2];  // chunks tid (and, in a work-group of 256 threads, tid + 256) of either image
    int pg;
};
// the quantised layouts: thread tid owns row tid / 32, block tid / 4 % 8, codes 8 (tid % 4) .. + 7 of it
template <>
struct PageStage<BKV_LAYOUT_Q8V> {
    v4u k;                   // chunk tid of the f16 K image
    unsigned scale, c0, c1;  // of V
    int pg;
};
template <>
struct PageStage<BKV_LAYOUT_I8H> {
    unsigned kc0, kc1, vc0, vc1;
    unsigned short kscale, vscale;
    int pg;
};

template <int LAY>
struct PrefillLds {
    // [buffer][image][16 rows][halves]: K (int8 pools: K high parts, K low parts) and V (quantised
    // pools: V high parts, V low parts)
    _Float16 kimg[4][LAY == BKV_LAYOUT_I8H ? 2 : 1][kPage][kLdsRow];
    _Float16 vimg[4][LAY == BKV_LAYOUT_F16 ? 1 : 2][kPage][kLdsRowV];
    float e[LAY == BKV_LAYOUT_Q8V ? 4 : 1][kPage];  // q8_0 V: E of the buffer's cells
};

// WAVES: waves of a work-group, 16 query rows each.  Eight share every page image they put into LDS
// among 128 rows (one work-group per compute unit); four (f16 pools only, two work-groups per
// compute unit) spread a small chunk over twice as many compute units.
template <int LAY, int WAVES = 8>
__global__ __launch_bounds__(64 * WAVES, 8 / WAVES) void prefill_attn_kernel(const PrefillKernelParams P) {
    static_assert(WAVES == 8 || (WAVES == 4 && LAY == BKV_LAYOUT_F16), "the quantised images are dequantised by 512 threads");
    constexpr bool Q8V = LAY == BKV_LAYOUT_Q8V;
    constexpr bool I8H = LAY == BKV_LAYOUT_I8H;
    constexpr bool WIDE = LAY != BKV_LAYOUT_F16;  // V (int8 pools: K too) as two f16 images
    constexpr int kWavesPerWg = WAVES;
    constexpr int kThreads = 64 * kWavesPerWg;
    constexpr int kRowsPerWg = kRowsPerWave * kWavesPerWg;
    // ---- which (entry, kv head, block of 64 query rows) ---------------------------------
    int e = 0, kvh, idx;  // idx: which of the unit's blocks, in dispatch order
    if (P.by_xcd) {
        const int units = P.b.n * P.n_kv;
        const int x = (int)blockIdx.x % kXcds;
        int j = (int)blockIdx.x / kXcds;
        int u;
        if (units >= kXcds) {
            u = x;
            for (;;) {
                if (u >= units) return;  // this die's share of the grid is shorter than the longest
                const int nb = (P.b.n_tok[u / P.n_kv] * P.group + kRowsPerWg - 1) / kRowsPerWg;
                if (j < nb) break;
                j -= nb;
                u += kXcds;
            }
            idx = j;
        } else {
            u = x % units;
            const int dies = (kXcds - u + units - 1) / units;  // dies x with x % units == u
            idx = j * dies + x / units;
        }
        e = u / P.n_kv;
        kvh = u - e * P.n_kv;
    } else {
        while (e + 1 < P.b.n && (int)blockIdx.x >= P.b.wg_base[e + 1]) ++e;
        const int rem = (int)blockIdx.x - P.b.wg_base[e];
        kvh = rem % P.n_kv;
        idx = rem / P.n_kv;
    }
    const int n_rows = P.b.n_tok[e] * P.group;  // query rows of this kv head
    const int n_blocks = (n_rows + kRowsPerWg - 1) / kRowsPerWg;
    if (idx >= n_blocks) return;
    // later rows attend more cells: the heaviest blocks are dispatched first
    const int rb = n_blocks - 1 - idx;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int c = lane & 15;  // query row of the tile / cell of the page / output column group
    const int g = lane >> 4;  // which quarter of the contraction index this lane feeds
    const int row0 = rb * kRowsPerWg + wave * kRowsPerWave;
    // a wave whose rows lie past the end still helps to fetch pages and joins the barriers
    const bool wave_live = row0 < n_rows;

    // this lane's query row
    const int row = row0 + c;
    const bool row_live = wave_live && row < n_rows;
    const int tok = row_live ? row / P.group : 0;
    const int head = kvh * P.group + (row_live ? row % P.group : 0);
    // a lane without a query row (past the end of the chunk) walks along with q = 0 and every cell
    // live: its column of the products is its own, and nothing of it is stored
    const int pos_q = row_live ? P.b.pos0[e] + tok : 0x7fffffff;
    // the first position any row of this wave has: pages wholly at or below it need no causal mask
    const int pos_min = P.b.pos0[e] + (wave_live ? row0 / P.group : 0);
    // the last token any row of this wave belongs to bounds the page walk
    const int last_row = min(row0 + kRowsPerWave, n_rows) - 1;
    const int pos_max = wave_live ? P.b.pos0[e] + last_row / P.group : -1;
    const int n_pages = wave_live ? pos_max / kPage + 1 : 0;
    // pages the work-group walks: those of its last row
    const int wg_last_row = min(rb * kRowsPerWg + kRowsPerWg, n_rows) - 1;
    const int wg_pos_max = P.b.pos0[e] + wg_last_row / P.group;
    const int wg_pages = wg_pos_max / kPage + 1;

    typedef const __attribute__((address_space(4))) int32_t* table_ptr;
    const table_ptr bt = (table_ptr)(uintptr_t)(P.tables + (size_t)P.b.row[e] * (size_t)P.max_pages_per_seq);
    constexpr int kKRow = I8H ? kI8hRow : kHd * 2;  // bytes of a row in the K pool and in the V pool
    constexpr int kVRow = I8H ? kI8hRow : Q8V ? kQ8vRow : kHd * 2;
    const size_t page_bytes = (size_t)P.n_kv * kPage * kKRow;
    const size_t head_off = (size_t)kvh * kPage * kKRow;
    const size_t v_page_bytes = (size_t)P.n_kv * kPage * kVRow;
    const size_t v_head_off = (size_t)kvh * kPage * kVRow;

    // ---- q fragments: lane (c, g) holds q[row][32 m + 8 g + 0..7], m = 0..7, as hi + lo f16 ----
    h8 qhi[8], qlo[8];
    {
        const float* qp = P.q + ((size_t)(P.b.src0[e] + tok) * P.n_q + head) * kHd + g * 8;
#pragma unroll
        for (int m = 0; m < 8; ++m) {
            float x[8];
            if (row_live) {
                const float4 a = *reinterpret_cast<const float4*>(qp + m * 32);
                const float4 b = *reinterpret_cast<const float4*>(qp + m * 32 + 4);
                x[0] = a.x, x[1] = a.y, x[2] = a.z, x[3] = a.w;
                x[4] = b.x, x[5] = b.y, x[6] = b.z, x[7] = b.w;
            } else {
#pragma unroll
                for (int j = 0; j < 8; ++j) x[j] = 0.0f;
            }
            // The softmax scale (and the change to base 2) rides on q: one rounding of q, 2^-24
            // relative.  The low parts are kept times 2^11 and their products scaled back in f32
            // (kLoDown), which keeps them out of the f16 subnormals' few bits.  The product is
            // pinned as one f32 number: left to fuse it into the conversions, the compiler took the
            // remainder against f16(x * c) rounded once and stored a high part rounded twice (x * c to
            // f32, then to f16) -- two numbers that differ by an f16 ulp now and then, which showed as
            // 3e-5 in short contexts.
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                float xs = x[j] * P.scale_log2e;
                asm("" : "+v"(xs));  // the product as one f32 number: no fusing into the conversions below
                const _Float16 hi = (_Float16)xs;
                qhi[m][j] = hi;
                qlo[m][j] = (_Float16)((xs - (float)hi) * 2048.0f);
            }
        }
    }

    // O^T accumulators: o[tile][r] = out[row][16 tile + 4 g + r]
    f4 o[16];
#pragma unroll
    for (int t = 0; t < 16; ++t) o[t] = f4{0.0f, 0.0f, 0.0f, 0.0f};
    float m_run = -INFINITY;  // running max of this lane's query (base-2 logits), same in all 4 g lanes
    float l_run = 0.0f;       // this lane's share (its 4 cells per page) of the denominator

    // ---- pages through LDS -----------------------------------------------------------------------
    // Rows are padded to 528 bytes so that the 16-byte fragment reads of the 64 lanes spread
    // evenly over the banks.  An f16 page image is 512 chunks of 16 bytes: thread t moves chunk
    // t (+ 256) of it.  Pages are taken two at a time (one softmax update, one
    // barrier and P.V MFMAs that contract over the 32 cells of the pair): four buffers, the pair
    // being multiplied and the pair being filled.
    __shared__ __attribute__((aligned(16))) PrefillLds<LAY> L;
    const int tid = threadIdx.x;
    // quantised layouts: this thread's part of a page
    const int v_row = tid >> 5, v_blk = (tid >> 2) & 7, v_j = tid & 3;
    const auto fetch = [&](int pg, PageStage<LAY>& st) {
        const int32_t phys = bt[pg];
        const uint8_t* kp = P.kpool + (size_t)phys * page_bytes + head_off;
        const uint8_t* vp = P.vpool + (size_t)phys * v_page_bytes + v_head_off;
        if constexpr (Q8V) {
            st.k = *reinterpret_cast<const v4u*>(kp + (size_t)tid * 16);
            const uint8_t* blk = vp + v_row * kQ8vRow + v_blk * 36;
            st.scale = *reinterpret_cast<const unsigned*>(blk);
            st.c0 = *reinterpret_cast<const unsigned*>(blk + 4 + v_j * 8);
            st.c1 = *reinterpret_cast<const unsigned*>(blk + 8 + v_j * 8);
            st.pg = pg;
        } else if constexpr (I8H) {
            const uint8_t* kr = kp + v_row * kI8hRow;
            const uint8_t* vr = vp + v_row * kI8hRow;
            st.kc0 = *reinterpret_cast<const unsigned*>(kr + v_blk * 32 + v_j * 8);
            st.kc1 = *reinterpret_cast<const unsigned*>(kr + v_blk * 32 + v_j * 8 + 4);
            st.vc0 = *reinterpret_cast<const unsigned*>(vr + v_blk * 32 + v_j * 8);
            st.vc1 = *reinterpret_cast<const unsigned*>(vr + v_blk * 32 + v_j * 8 + 4);
            st.kscale = *reinterpret_cast<const unsigned short*>(kr + kHd + v_blk * 2);
            st.vscale = *reinterpret_cast<const unsigned short*>(vr + kHd + v_blk * 2);
            st.pg = pg;
        } else {
#pragma unroll
            for (int j = 0; j < 512 / kThreads; ++j) {
                st.k[j] = *reinterpret_cast<const v4u*>(kp + (size_t)(tid + j * kThreads) * 16);
                st.v[j] = *reinterpret_cast<const v4u*>(vp + (size_t)(tid + j * kThreads) * 16);
            }
            st.pg = pg;
        }
    };
    const auto deposit = [&](int buf, const PageStage<LAY>& st) {
        // chunk q of a page image: row q / 32, halves (q % 32) * 8 ..
        if constexpr (Q8V) {
            *reinterpret_cast<v4u*>(&L.kimg[buf][0][tid >> 5][(tid & 31) * 8]) = st.k;
            // Rows past the work-group's last position were never written for these queries and
            // may hold anything: scale 1 for the row's exponent, zeros for its values.
            const bool dead = st.pg * kPage + v_row > wg_pos_max;
            const float sc = __builtin_bit_cast(float, st.scale);
            // the largest scale of the row: over the lanes that differ in the block bits (2..4)
            float smax = dead ? 1.0f : sc;
            smax = fmaxf(smax, dpp_mov<0x124>(smax));  // row_ror:4
            smax = fmaxf(smax, dpp_mov<0x128>(smax));  // row_ror:8
            {
                const LanePair o = swap_rows(smax);
                smax = fmaxf(o.a, o.b);
            }
            int ee = (int)((__builtin_bit_cast(unsigned, smax) >> 23) & 0xffu) - 127;
            ee = min(max(ee, -120), 120);
            const float down = __builtin_bit_cast(float, (unsigned)(127 - ee) << 23);  // 2^-E
            _Float16 s_hi, s_lo;
            split_f16(dead ? 0.0f : sc * down, s_hi, s_lo);
            const h2m sh = h2m{s_hi, s_hi}, sl = h2m{s_lo, s_lo};
            h2m cd[4], hi[4], lo[4];
            codes_to_f16(st.c0, cd[0], cd[1]);
            codes_to_f16(st.c1, cd[2], cd[3]);
#pragma unroll
            for (int i = 0; i < 4; ++i) scaled_hi_lo(cd[i], sh, sl, hi[i], lo[i]);
            const h8 vh = h8{hi[0][0], hi[0][1], hi[1][0], hi[1][1], hi[2][0], hi[2][1], hi[3][0], hi[3][1]};
            const h8 vl = h8{lo[0][0], lo[0][1], lo[1][0], lo[1][1], lo[2][0], lo[2][1], lo[3][0], lo[3][1]};
            *reinterpret_cast<h8*>(&L.vimg[buf][0][v_row][v_blk * 32 + v_j * 8]) = vh;
            *reinterpret_cast<h8*>(&L.vimg[buf][1][v_row][v_blk * 32 + v_j * 8]) = vl;
            if ((tid & 31) == 0) L.e[buf][v_row] = (float)ee;
        } else if constexpr (I8H) {
            // K: code * scale (7 + 11 significant bits) as hi = f16(code * scale) and the exact
            // remainder, like V below.  A scale with exponent field 0 reads as zero, as everywhere.
            {
                const unsigned short ks = (st.kscale & 0x7c00u) == 0 ? (unsigned short)0 : st.kscale;
                const _Float16 ksc = __builtin_bit_cast(_Float16, ks);
                const h2m sh = h2m{ksc, ksc}, sl = h2m{(_Float16)0.0f, (_Float16)0.0f};
                h2m kd[4], hi[4], lo[4];
                codes_to_f16(st.kc0, kd[0], kd[1]);
                codes_to_f16(st.kc1, kd[2], kd[3]);
#pragma unroll
                for (int i = 0; i < 4; ++i) scaled_hi_lo(kd[i], sh, sl, hi[i], lo[i]);
                *reinterpret_cast<h8*>(&L.kimg[buf][0][v_row][v_blk * 32 + v_j * 8]) =
                    h8{hi[0][0], hi[0][1], hi[1][0], hi[1][1], hi[2][0], hi[2][1], hi[3][0], hi[3][1]};
                *reinterpret_cast<h8*>(&L.kimg[buf][1][v_row][v_blk * 32 + v_j * 8]) =
                    h8{lo[0][0], lo[0][1], lo[1][0], lo[1][1], lo[2][0], lo[2][1], lo[3][0], lo[3][1]};
            }
            // V: code * scale (7 + 11 significant bits) as hi = f16(code * scale) and the exact
            // remainder; rows past the work-group's last position become zeros
            const bool dead = st.pg * kPage + v_row > wg_pos_max;
            const unsigned short vs = (dead || (st.vscale & 0x7c00u) == 0) ? (unsigned short)0 : st.vscale;
            const _Float16 vsc = __builtin_bit_cast(_Float16, vs);
            const h2m sh = h2m{vsc, vsc}, sl = h2m{(_Float16)0.0f, (_Float16)0.0f};
            h2m cd[4], hi[4], lo[4];
            codes_to_f16(st.vc0, cd[0], cd[1]);
            codes_to_f16(st.vc1, cd[2], cd[3]);
#pragma unroll
            for (int i = 0; i < 4; ++i) scaled_hi_lo(cd[i], sh, sl, hi[i], lo[i]);
            *reinterpret_cast<h8*>(&L.vimg[buf][0][v_row][v_blk * 32 + v_j * 8]) =
                h8{hi[0][0], hi[0][1], hi[1][0], hi[1][1], hi[2][0], hi[2][1], hi[3][0], hi[3][1]};
            *reinterpret_cast<h8*>(&L.vimg[buf][1][v_row][v_blk * 32 + v_j * 8]) =
                h8{lo[0][0], lo[0][1], lo[1][0], lo[1][1], lo[2][0], lo[2][1], lo[3][0], lo[3][1]};
        } else {
            // V rows past the work-group's last position were never written for these queries and may
            // hold anything (even NaN): exact zeros, before they meet a zero probability.  Only the
            // work-group's last page has such rows.
            const bool last_page = st.pg * kPage + kPage - 1 > wg_pos_max;
#pragma unroll
            for (int j = 0; j < 512 / kThreads; ++j) {
                const int q = tid + j * kThreads;
                v4u vv = st.v[j];
                if (last_page && st.pg * kPage + (q >> 5) > wg_pos_max) vv = v4u{0u, 0u, 0u, 0u};
                *reinterpret_cast<v4u*>(&L.kimg[buf][0][q >> 5][(q & 31) * 8]) = st.k[j];
                *reinterpret_cast<v4u*>(&L.vimg[buf][0][q >> 5][(q & 31) * 8]) = vv;
            }
        }
    };

    // this lane's piece of a transposing V read: row 4 g + c / 4, halves 4 (c % 4) .. of a 16-column tile
    const int tr_off = (4 * g + (c >> 2)) * kLdsRowV + 4 * (c & 3);
    // scores of one page in base 2: s[r] = scale * log2(e) * q[row c] . k[cell 4 g + r], unmasked
    const auto scores = [&](int buf) -> f4 {
        const _Float16* ks = &L.kimg[buf][0][0][0];
        // K: row c, 16 bytes at element 32 m + 8 g (the same split of the head dim as q): the 8
        // halves of a lane are the 8 contraction steps it feeds to the 32-deep MFMA
        h8 kf[8];
#pragma unroll
        for (int m = 0; m < 8; ++m) kf[m] = *reinterpret_cast<const h8*>(ks + c * kLdsRow + m * 32 + g * 8);
        if constexpr (I8H) {
            // K = hi + lo: hi meets q's high and low parts, lo q's high parts; three chains
            const _Float16* kl = &L.kimg[buf][1][0][0];
            f4 s0 = f4{0.0f, 0.0f, 0.0f, 0.0f}, s1 = s0, s2 = s0;
#pragma unroll
            for (int m = 0; m < 8; ++m) {
                const h8 klo = *reinterpret_cast<const h8*>(kl + c * kLdsRow + m * 32 + g * 8);
                s0 = mfma32(kf[m], qhi[m], s0);
                s1 = mfma32(kf[m], qlo[m], s1);
                s2 = mfma32(klo, qhi[m], s2);
            }
            return (s0 + s2) + s1 * kLoDown;
        } else {
            // two accumulation chains, q's high parts and q's low parts: an MFMA adds to the sum of the
            // one before the last, which has left the pipeline by then
            f4 s0 = f4{0.0f, 0.0f, 0.0f, 0.0f}, s1 = s0;
#pragma unroll
            for (int m = 0; m < 8; ++m) {
                s0 = mfma32(kf[m], qhi[m], s0);
                s1 = mfma32(kf[m], qlo[m], s1);
            }
            return s0 + s1 * kLoDown;
        }
    };

    // pages pg and pg + 1 of this wave: scores -> softmax -> accumulate, operands from the LDS
    // buffers buf and buf + 1.  The second page may lie past the wave's last one: it then counts
    // as all dead (its buffer holds some finite page of the work-group, or nothing yet).
    const auto process_pair = [&](int pg, int buf) {
        const bool second = pg + 1 < n_pages;
        float ta[4], tb[4];
        {
            const f4 sa = scores(buf);
            f4 sb = f4{0.0f, 0.0f, 0.0f, 0.0f};
            if (second) sb = scores(buf + 1);
            if (second && (pg + 2) * kPage - 1 <= pos_min) {
                // every cell of the pair is at or below every row's position
#pragma unroll
                for (int r = 0; r < 4; ++r) ta[r] = sa[r], tb[r] = sb[r];
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int cell = pg * kPage + 4 * g + r;
                    ta[r] = cell <= pos_q ? sa[r] : -INFINITY;
                    tb[r] = second && cell + kPage <= pos_q ? sb[r] : -INFINITY;
                }
            }
        }
        // q8_0 V: the softmax runs over logit + E of the cell (wa, wb); dead cells stay at -inf
        float wa[4], wb[4];
        if constexpr (Q8V) {
            const f4 ea = *reinterpret_cast<const f4*>(&L.e[buf][4 * g]);
            f4 eb = f4{0.0f, 0.0f, 0.0f, 0.0f};
            if (second) eb = *reinterpret_cast<const f4*>(&L.e[buf + 1][4 * g]);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                wa[r] = ta[r] + ea[r];
                wb[r] = tb[r] + eb[r];
            }
        } else {
#pragma unroll
            for (int r = 0; r < 4; ++r) wa[r] = ta[r], wb[r] = tb[r];
        }

        // ---- online softmax for this lane's query, over the pair's 32 cells ---------------------------
        // Cell 0 is live for every query, so from the first pair on the reference m_run is finite.
        // It follows the running maximum lazily: it moves only when a pair's maximum passes it by
        // more than kSlack (weights then reach 2^kSlack at most, far inside f16 and f32), which after
        // the first pairs is rare -- and every move costs a rescale of the 64 accumulators.  The
        // q8_0 weights multiply values of up to 2^8, so there the reference is the maximum itself.
        constexpr float kSlack = Q8V ? 0.0f : 6.0f;
        float pm = fmaxf(fmaxf(fmaxf(wa[0], wa[1]), fmaxf(wa[2], wa[3])), fmaxf(fmaxf(wb[0], wb[1]), fmaxf(wb[2], wb[3])));
        pm = max_over_lane_groups(pm);
        const bool moved = pm > m_run + kSlack;  // m_run = -inf at the start: any finite maximum moves it
        const float m_new = moved ? pm : m_run;
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);  // 1, or 0 at the start
        float pv[8];
        float psum = 0.0f;
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            const float ww = r < 4 ? wa[r & 3] : wb[r & 3];
            pv[r] = __builtin_amdgcn_exp2f(ww - m_new);
            if constexpr (Q8V) {
                const float tt = r < 4 ? ta[r & 3] : tb[r & 3];
                psum += __builtin_amdgcn_exp2f(tt - m_new);
            } else {
                psum += pv[r];
            }
        }
        // p = hi + lo, both rounded to nearest (the matrix cores read f16 subnormals as the numbers
        // they are, so small weights keep their low parts' few bits)
        h8 ph, pl;  // slots 0..3: the first page's cells 4 g + r, slots 4..7: the second page's
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            _Float16 hi, lo;
            split_f16(pv[r], hi, lo);
            ph[r] = hi;
            pl[r] = lo;
        }
        l_run = l_run * alpha + psum;
        m_run = m_new;
        if (__builtin_amdgcn_ballot_w64(moved) != 0) {
#pragma unroll
            for (int t = 0; t < 16; ++t) o[t] *= alpha;
        }

        // ---- O^T += V^T . P^T over the 32 cells of the pair ----------------------------------------
        // Per tile of 16 output columns one transposing read from either page's image: lane (c, g)
        // receives column 16 tile + c of cells 4 g .. 4 g + 3 -- slots 0..3 and 4..7 of the operand,
        // the order P^T has.  Rows past the work-group's last position are zeros in the image.  A
        // second page past this wave's last one meets zero probabilities: its buffer holds a page of
        // the work-group all the same (the last one again, past the end), never nothing, so the
        // reads need no condition and the 32 of them can be issued ahead of the MFMAs.
        // quantised V: the image of high parts meets p's high and low parts, the image of low parts
        // p's high parts
#pragma unroll
        for (int img = 0; img < (WIDE ? 2 : 1); ++img) {
            const _Float16* va_s = &L.vimg[buf][img][0][0] + tr_off;
            const _Float16* vb_s = &L.vimg[buf + 1][img][0][0] + tr_off;
#pragma unroll
            for (int t = 0; t < 16; ++t) {
                const tr_s4 fa = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(va_s + t * 16));
                const tr_s4 fb = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(vb_s + t * 16));
                const h8 vv = __builtin_bit_cast(h8, __builtin_shufflevector(fa, fb, 0, 1, 2, 3, 4, 5, 6, 7));
                o[t] = mfma32(vv, ph, o[t]);
                if (img == 0) o[t] = mfma32(vv, pl, o[t]);
            }
        }
    };

    // Two pairs are in flight behind the one being multiplied: one in the other two LDS buffers,
    // one in the staging registers (past the end they carry the last page again).
    PageStage<LAY> stage_a, stage_b;
    const int last_pg = wg_pages - 1;
    fetch(0, stage_a);
    fetch(min(1, last_pg), stage_b);
    deposit(0, stage_a);
    deposit(1, stage_b);
    fetch(min(2, last_pg), stage_a);
    fetch(min(3, last_pg), stage_b);
    __syncthreads();
    for (int pg = 0; pg < wg_pages; pg += 2) {
        const int buf = pg & 2;  // 0 or 2
        if (pg < n_pages) process_pair(pg, buf);
        deposit(buf ^ 2, stage_a);  // pages pg + 2, pg + 3
        deposit((buf ^ 2) + 1, stage_b);
        fetch(min(pg + 4, last_pg), stage_a);
        fetch(min(pg + 5, last_pg), stage_b);
        // after the barrier the other pair of buffers is complete, and nobody reads this one any more
        __syncthreads();
    }

    // ---- normalise, gate, store ---------------------------------------------------------------------
    l_run = sum_over_lane_groups(l_run);
    if (!row_live) return;
    const float inv = l_run > 0.0f ? 1.0f / l_run : 0.0f;
    float* op = P.out + ((size_t)(P.b.src0[e] + tok) * P.n_q + head) * kHd;
    const float* gp = P.gate ? P.gate + (size_t)(P.b.src0[e] + tok) * P.gate_tok_stride +
                                   (size_t)head * P.gate_head_stride
                             : nullptr;
#pragma unroll
    for (int t = 0; t < 16; ++t) {
        const int d0 = 16 * t + 4 * g;
        float y[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            y[r] = o[t][r] * inv;
            if (gp) {
                // sigmoid in the overflow-free form of the reference (qsa/cpu.rs:84-91)
                const float gt = gp[d0 + r];
                float sg;
                if (gt >= 0.0f) {
                    sg = 1.0f / (1.0f + expf(-gt));
                } else {
                    const float ex = expf(gt);
                    sg = ex / (1.0f + ex);
                }
                y[r] *= sg;
            }
        }
        *reinterpret_cast<float4*>(op + d0) = make_float4(y[0], y[1], y[2], y[3]);
    }
}

}  // namespace

// Query rows one work-group owns.  f16 pools: 128 when the chunks make more 64-row work-groups than
// fit the chip at two per compute unit (then sharing the page images among more rows is worth more
// than spreading out), else 64.
int32_t prefill_rows_per_wg(int32_t layout, int64_t wgs_of_64_rows, int32_t n_cu) {
    if (layout != BKV_LAYOUT_F16) return 8 * kRowsPerWave;
    return wgs_of_64_rows > 2 * (int64_t)(n_cu > 0 ? n_cu : 256) ? 8 * kRowsPerWave : 4 * kRowsPerWave;
}

hipError_t launch_prefill_attn(bkv_pool* p, int32_t layer, const PrefillBatch& b, const AttnArgs& a,
                               int32_t rows_per_wg, hipStream_t stream) {
    PrefillKernelParams kp;
    kp.b = b;
    kp.kpool = p->k_layer[(size_t)layer];
    kp.vpool = p->v_layer[(size_t)layer];
    kp.tables = p->table_dev;
    kp.q = a.q;
    kp.gate = a.gate;
    kp.out = a.out;
    kp.gate_tok_stride = a.gate_seq_stride;
    kp.gate_head_stride = a.gate_head_stride;
    kp.max_pages_per_seq = p->desc.max_pages_per_seq;
    kp.n_kv = p->g.n_kv;
    kp.n_q = a.n_q_head;
    kp.group = a.n_q_head / p->g.n_kv;
    kp.scale_log2e = a.scale * kLog2e;
    int32_t grid = b.wg_base[b.n];
    if (grid == 0) return hipSuccess;
    // Deal the work-groups to the dies by unit where that costs little: the grid then holds 8 x the
    // longest die's share, and work-groups past a shorter die's share leave at once.
    kp.by_xcd = 0;
    {
        const int units = b.n * p->g.n_kv;
        int64_t longest = 0;
        if (units >= kXcds) {
            int64_t share[kXcds] = {};
            for (int u = 0; u < units; ++u)
                share[u % kXcds] += ((int64_t)b.n_tok[u / p->g.n_kv] * kp.group + rows_per_wg - 1) / rows_per_wg;
            for (int x = 0; x < kXcds; ++x) longest = std::max(longest, share[x]);
        } else {
            for (int u = 0; u < units; ++u) {
                const int64_t nb = ((int64_t)b.n_tok[u / p->g.n_kv] * kp.group + rows_per_wg - 1) / rows_per_wg;
                const int dies = (kXcds - u + units - 1) / units;
                longest = std::max(longest, (nb + dies - 1) / dies);
            }
        }
        const int64_t by_xcd_grid = longest * kXcds;
        if (by_xcd_grid <= (int64_t)grid + grid / 4 + kXcds) {
            kp.by_xcd = 1;
            grid = (int32_t)by_xcd_grid;
        }
    }
    if (p->g.layout == BKV_LAYOUT_Q8V)
        launch_staged(p, BKV_STAGE_PREFILL_ATTN, prefill_attn_kernel<BKV_LAYOUT_Q8V>, dim3((unsigned)grid), dim3(512), 0,
                      stream, kp);
    else if (p->g.layout == BKV_LAYOUT_I8H)
        launch_staged(p, BKV_STAGE_PREFILL_ATTN, prefill_attn_kernel<BKV_LAYOUT_I8H>, dim3((unsigned)grid), dim3(512), 0,
                      stream, kp);
    else if (rows_per_wg == 8 * kRowsPerWave)
        launch_staged(p, BKV_STAGE_PREFILL_ATTN, prefill_attn_kernel<BKV_LAYOUT_F16, 8>, dim3((unsigned)grid), dim3(512), 0,
                      stream, kp);
    else
        launch_staged(p, BKV_STAGE_PREFILL_ATTN, prefill_attn_kernel<BKV_LAYOUT_F16, 4>, dim3((unsigned)grid), dim3(256), 0,
                      stream, kp);
    return hipGetLastError();
}

}  // namespace bkv
