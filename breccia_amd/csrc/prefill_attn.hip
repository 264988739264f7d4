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
//   O^T[d][query]   += V^T[d][cell] . P^T[cell][query]  v_mfma_f32_16x16x32_f16 over the page's 16
//                                                       cells twice, A = V gathered per lane (the
//                                                       same four cells in both halves of a lane's
//                                                       slots), B = P^T high parts, then low parts
// Both products keep the per-lane query (lane % 16) fixed, so the softmax statistics never
// move between lanes, and P^T feeds the second product straight from registers.  K and V are
// exact f16; q and p are f32 values split into a high and a low f16 part (two MFMAs for the
// scores, the two halves of one for P.V), so the products carry ~22 significant bits and the
// result stays at f32-accumulate accuracy.
// The V operand needs four cells of one head-dim column per lane: each lane loads 16 bytes
// (8 columns) of four rows and regroups them in registers; the 8 MFMAs that use them produce
// columns 8i + t of the output, i = the MFMA row, t = 0..7.
#include "bkv_internal.hpp"
#include "lane_groups.hpp"

namespace bkv {

namespace {

constexpr int kHd = 256;
constexpr int kPage = 16;
constexpr int kRowsPerWave = 16;
constexpr int kWavesPerWg = 4;
constexpr int kThreads = 64 * kWavesPerWg;
constexpr int kChunks = kPage * kHd * 2 / 16 / kThreads;  // 16-byte chunks of a K (or V) page image per thread
constexpr int kRowsPerWg = kRowsPerWave * kWavesPerWg;
constexpr float kLog2e = 1.4426950408889634f;
constexpr int kLdsRow = kHd + 8;  // halves per row of a page image in LDS (528 bytes)

typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));

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
};

// gfx950's double-depth form: 32 contraction steps, 8 halves per lane (k = 8 (lane / 16) + 0..7)
__device__ __forceinline__ f4 mfma32(h8 a, h8 b, f4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ void split_f16(float x, _Float16& hi, _Float16& lo) {
    hi = (_Float16)x;
    lo = (_Float16)(x - (float)hi);
}

__global__ __launch_bounds__(kThreads, 2) void prefill_attn_kernel(const PrefillKernelParams P) {
    // ---- which (entry, kv head, block of 64 query rows) ---------------------------------
    int e = 0;
    while (e + 1 < P.b.n && (int)blockIdx.x >= P.b.wg_base[e + 1]) ++e;
    const int rem = (int)blockIdx.x - P.b.wg_base[e];
    const int kvh = rem % P.n_kv;
    const int n_rows = P.b.n_tok[e] * P.group;  // query rows of this kv head
    const int n_blocks = (n_rows + kRowsPerWg - 1) / kRowsPerWg;
    // later rows attend more cells: the heaviest blocks are dispatched first
    const int rb = n_blocks - 1 - rem / P.n_kv;
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
    const int pos_q = row_live ? P.b.pos0[e] + tok : -1;
    // the last token any row of this wave belongs to bounds the page walk
    const int last_row = min(row0 + kRowsPerWave, n_rows) - 1;
    const int pos_max = wave_live ? P.b.pos0[e] + last_row / P.group : -1;
    const int n_pages = wave_live ? pos_max / kPage + 1 : 0;
    // pages the work-group walks: those of its last row
    const int wg_last_row = min(rb * kRowsPerWg + kRowsPerWg, n_rows) - 1;
    const int wg_pages = (P.b.pos0[e] + wg_last_row / P.group) / kPage + 1;

    typedef const __attribute__((address_space(4))) int32_t* table_ptr;
    const table_ptr bt = (table_ptr)(uintptr_t)(P.tables + (size_t)P.b.row[e] * (size_t)P.max_pages_per_seq);
    const size_t page_bytes = (size_t)P.n_kv * kPage * kHd * 2;
    const size_t head_off = (size_t)kvh * kPage * kHd * 2;

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
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                _Float16 hi, lo;
                split_f16(x[j], hi, lo);
                qhi[m][j] = hi;
                qlo[m][j] = lo;
            }
        }
    }

    // O^T accumulators: o[half][t][r] = out[row][128 half + 8 (4 g + r) + t]
    f4 o[2][8];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int t = 0; t < 8; ++t) o[h][t] = f4{0.0f, 0.0f, 0.0f, 0.0f};
    float m_run = -INFINITY;  // running max of this lane's query (base-2 logits), same in all 4 g lanes
    float l_run = 0.0f;       // this lane's share (its 4 cells per page) of the denominator

    // ---- pages through LDS: [buffer][K | V][16 rows][264 halves] -------------------------------
    // Rows are padded to 528 bytes so that the 16-byte fragment reads of the 64 lanes spread
    // evenly over the banks.  A page image is 2 x 512 chunks of 16 bytes: thread t moves chunk
    // t (+ kThreads, ...) of K and of V.
    __shared__ __attribute__((aligned(16))) _Float16 lds[2][2][kPage][kLdsRow];
    const int tid = threadIdx.x;
    const auto fetch = [&](int pg, v4u (&stage)[2 * kChunks]) {
        const int32_t phys = bt[pg];
        const uint8_t* kp = P.kpool + (size_t)phys * page_bytes + head_off;
        const uint8_t* vp = P.vpool + (size_t)phys * page_bytes + head_off;
#pragma unroll
        for (int j = 0; j < kChunks; ++j) {
            stage[j] = *reinterpret_cast<const v4u*>(kp + (size_t)(tid + j * kThreads) * 16);
            stage[kChunks + j] = *reinterpret_cast<const v4u*>(vp + (size_t)(tid + j * kThreads) * 16);
        }
    };
    const auto deposit = [&](int buf, const v4u (&stage)[2 * kChunks]) {
        // chunk q of a page image: row q / 32, halves (q % 32) * 8 ..
#pragma unroll
        for (int j = 0; j < kChunks; ++j) {
            const int q = tid + j * kThreads;
            *reinterpret_cast<v4u*>(&lds[buf][0][q >> 5][(q & 31) * 8]) = stage[j];
            *reinterpret_cast<v4u*>(&lds[buf][1][q >> 5][(q & 31) * 8]) = stage[kChunks + j];
        }
    };

    // one page of this wave: scores -> softmax -> accumulate, operands from LDS buffer `buf`
    const auto process = [&](int pg, int buf) {
        const _Float16* ks = &lds[buf][0][0][0];
        const _Float16* vs = &lds[buf][1][0][0];
        // ---- S^T = K . Q^T ------------------------------------------------------------------
        // four independent accumulation chains: an MFMA that waits for the previous one's result
        // costs its full latency
        // K: row c, 16 bytes at element 32 m + 8 g (the same split of the head dim as q): the 8
        // halves of a lane are the 8 contraction steps it feeds to the 32-deep MFMA.  All fragments
        // of the page are requested from LDS in one batch; V's follow while the scores are formed.
        h8 kf[8];
#pragma unroll
        for (int m = 0; m < 8; ++m) kf[m] = *reinterpret_cast<const h8*>(ks + c * kLdsRow + m * 32 + g * 8);
        __builtin_amdgcn_sched_barrier(0);
        // V: rows 4 g + r, 16 bytes at element 128 half + 8 c
        v4u vf[2][4];
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                vf[h][r] = *reinterpret_cast<const v4u*>(vs + (4 * g + r) * kLdsRow + h * 128 + c * 8);
        f4 s0 = f4{0.0f, 0.0f, 0.0f, 0.0f}, s1 = s0, s2 = s0, s3 = s0;
#pragma unroll
        for (int m = 0; m < 8; m += 2) {
            s0 = mfma32(kf[m], qhi[m], s0);
            s1 = mfma32(kf[m], qlo[m], s1);
            s2 = mfma32(kf[m + 1], qhi[m + 1], s2);
            s3 = mfma32(kf[m + 1], qlo[m + 1], s3);
        }
        const f4 s = (s0 + s1) + (s2 + s3);
        // s[r] = q[row c] . k[cell 4 g + r]

        // ---- online softmax for this lane's query ------------------------------------------------
        float t4[4];
        float pm = -INFINITY;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int cell = pg * kPage + 4 * g + r;
            t4[r] = cell <= pos_q ? s[r] * P.scale_log2e : -INFINITY;
            pm = fmaxf(pm, t4[r]);
        }
        pm = max_over_lane_groups(pm);
        const float m_new = fmaxf(m_run, pm);
        // a query with no live cell yet keeps m = -inf: exp2(-inf - -inf) would be NaN
        const float alpha = m_new == -INFINITY ? 1.0f : __builtin_amdgcn_exp2f(m_run - m_new);
        h4 phi, plo;
        float psum = 0.0f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float p = m_new == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(t4[r] - m_new);
            psum += p;
            _Float16 hi, lo;
            split_f16(p, hi, lo);
            phi[r] = hi;
            plo[r] = lo;
        }
        const h8 phl = h8{phi[0], phi[1], phi[2], phi[3], plo[0], plo[1], plo[2], plo[3]};
        l_run = l_run * alpha + psum;
        // rescale only on pages where some query's maximum moved (the test is on the maxima, not on
        // alpha != 1: with the latter the compiler multiplies unconditionally, 64 instructions a page)
        const bool moved = m_new > m_run;
        m_run = m_new;
        if (__builtin_amdgcn_ballot_w64(moved) != 0) {
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int t = 0; t < 8; ++t) o[h][t] *= alpha;
        }

        // Rows past the last position of this wave were never written for these queries and may
        // hold anything (even NaN): make them exact zeros before they meet a zero probability.
        if (pg == n_pages - 1) {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (pg * kPage + 4 * g + r > pos_max) {
                    vf[0][r] = v4u{0u, 0u, 0u, 0u};
                    vf[1][r] = v4u{0u, 0u, 0u, 0u};
                }
        }

        // ---- O^T += V^T . P^T ---------------------------------------------------------------------
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const h8 v0 = __builtin_bit_cast(h8, vf[h][0]), v1 = __builtin_bit_cast(h8, vf[h][1]);
            const h8 v2 = __builtin_bit_cast(h8, vf[h][2]), v3 = __builtin_bit_cast(h8, vf[h][3]);
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                // column 128 h + 8 c + t of cells 4 g ..: the 32-deep MFMA runs over the 16 cells twice,
                // against the high parts of p and then the low parts
                const h8 vv = h8{v0[t], v1[t], v2[t], v3[t], v0[t], v1[t], v2[t], v3[t]};
                o[h][t] = mfma32(vv, phl, o[h][t]);
            }
        }
    };

    // Two pages are in flight behind the one being multiplied: staging set A carries the even
    // pages, B the odd ones (past the end they carry the last page again).
    v4u stage_a[2 * kChunks], stage_b[2 * kChunks];
    const int last_pg = wg_pages - 1;
    fetch(0, stage_a);
    fetch(min(1, last_pg), stage_b);
    deposit(0, stage_a);
    fetch(min(2, last_pg), stage_a);
    __syncthreads();
    for (int pg = 0; pg < wg_pages; pg += 2) {
        if (pg < n_pages) process(pg, 0);
        deposit(1, stage_b);                      // page pg + 1
        fetch(min(pg + 3, last_pg), stage_b);
        // after the barrier the other buffer is complete, and nobody reads this one any more
        __syncthreads();
        if (pg + 1 < n_pages) process(pg + 1, 1);
        deposit(0, stage_a);                      // page pg + 2
        fetch(min(pg + 4, last_pg), stage_a);
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
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int d0 = h * 128 + 8 * (4 * g + r);
            float y[8];
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                y[t] = o[h][t][r] * inv;
                if (gp) {
                    // sigmoid in the overflow-free form of the reference (qsa/cpu.rs:84-91)
                    const float gt = gp[d0 + t];
                    float sg;
                    if (gt >= 0.0f) {
                        sg = 1.0f / (1.0f + expf(-gt));
                    } else {
                        const float ex = expf(gt);
                        sg = ex / (1.0f + ex);
                    }
                    y[t] *= sg;
                }
            }
            *reinterpret_cast<float4*>(op + d0) = make_float4(y[0], y[1], y[2], y[3]);
            *reinterpret_cast<float4*>(op + d0 + 4) = make_float4(y[4], y[5], y[6], y[7]);
        }
}

}  // namespace

int32_t prefill_rows_per_wg() { return kRowsPerWg; }

hipError_t launch_prefill_attn(bkv_pool* p, int32_t layer, const PrefillBatch& b, const AttnArgs& a,
                               hipStream_t stream) {
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
    const int32_t grid = b.wg_base[b.n];
    if (grid == 0) return hipSuccess;
    StageScope timed(p, BKV_STAGE_ATTN_SPLIT, stream);
    prefill_attn_kernel<<<grid, kThreads, 0, stream>>>(kp);
    return hipGetLastError();
}

}  // namespace bkv
