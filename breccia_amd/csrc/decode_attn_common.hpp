// Shared by the decode attention translation units: the kernel parameter block, the geometry the
// kernels are built for, the row encodings of the pools and where the rows of one loop iteration
// live.
#pragma once

#include "bkv_internal.hpp"

namespace bkv {

constexpr int kHd = 256;      // head_dim the kernel is built for
constexpr int kPage = 16;     // cells per page
constexpr int kWaves = 4;
constexpr int kBlock = 64 * kWaves;
constexpr float kLog2e = 1.4426950408889634f;

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));

struct AttnKernelParams {
    AttnBatch b;
    // kernels instantiated with DESC read the batch from this device-resident copy instead of `b`: a
    // launch recorded once (in a graph) then serves whatever batch the descriptor holds when it runs
    const AttnBatch* bd;
    const uint8_t* kpool;
    const uint8_t* vpool;
    const int32_t* tables;
    const float* q;
    float* part_o;
    float* part_ml;
    int32_t max_pages_per_seq;
    int32_t n_kv, n_q, group;
    uint32_t inv_kv16;  // small_divisor_inverse(n_kv): a work-group's index splits into (page range, kv head) without a division
    float scale_log2e;
    // selection lists (kernels instantiated with SEL only): entry e attends the 4-cell blocks
    // ids[e * id_stride + 0 .. min(counts[e], max_ids))
    const uint32_t* ids;
    const uint32_t* counts;
    int64_t id_stride;
    int32_t max_ids;
    // fused decode step (kernels instantiated with STEP only): the K/V row of cell pos of entry e
    // comes from new_k / new_v [n][n_kv][head_dim] f32 and is stored into the pool on the way
    const float* new_k;
    const float* new_v;
    uint8_t* kpool_w;
    uint8_t* vpool_w;
};

// x / d for the small numbers of this launch geometry, as a multiplication by ceil(2^16 / d): exact while
// x * d < 2^16 (work-group indices stay below kMaxWgs = 4096, head indices below 256, divisors are kv head
// counts and head groups of at most 16).  An integer division by a run-time value is some forty dependent
// instructions at the head of kernels whose first microsecond is all latency.
static_assert((int64_t)kMaxWgs * BKV_MAX_KV_HEAD <= 65536 && 256 * BKV_MAX_HEAD_GROUP <= 65536,
              "small_div is exact only while x * d < 2^16");
inline uint32_t small_divisor_inverse(int32_t d) { return (65536u + (uint32_t)d - 1u) / (uint32_t)d; }
__device__ __forceinline__ int small_div(int x, uint32_t inv16) { return (int)(((uint32_t)x * inv16) >> 16); }

// Which unit of work a work-group of the matrix-core kernels has: entry e, its rem-th work-group
// (page range x kv head), and the entry's position, block-table row and pages per range.  With DESC the
// batch is read from device memory through the constant address space (uniform addresses: scalar
// loads), and a work-group past the end of the current cut reports false: such a launch has a fixed grid.
typedef const __attribute__((address_space(4))) AttnBatch* batch_desc_ptr;
template <bool DESC>
__device__ __forceinline__ bool unit_of_work_group(const AttnKernelParams& P, int unit, int& e, int& rem, int& pos,
                                                   int& row, int& pps) {
    if constexpr (DESC) {
        const batch_desc_ptr D = (batch_desc_ptr)(uintptr_t)P.bd;
        const int n = D->n;
        if (unit >= D->wg_base[n]) return false;
        e = 0;
        while (e + 1 < n && unit >= D->wg_base[e + 1]) ++e;
        rem = unit - D->wg_base[e];
        pos = D->pos[e];
        row = D->row[e];
        pps = D->pps[e];
    } else {
        // entry 0's fields are asked for alongside n: their cache lines (sixteen entries each) are then on
        // their way before the entry is known
        asm volatile("" ::"s"(P.b.pos[0]), "s"(P.b.pps[0]), "s"(P.b.row[0]), "s"(P.b.wg_base[0]));
        e = 0;
        while (e + 1 < P.b.n && unit >= P.b.wg_base[e + 1]) ++e;
        rem = unit - P.b.wg_base[e];
        pos = P.b.pos[e];
        row = P.b.row[e];
        pps = P.b.pps[e];
    }
    return true;
}

// Row encodings of the K and V pools:
//   kRowF16   256 f16
//   kRowQ8    8 x [f32 scale][32 x i8]         (reference q8_0 V, shaders/qsa_kv_append.comp:
//             38-44; value = i8 * scale, qsa_attn_apply.comp:70-77)
//   kRowI8H   [256 x i8][8 x f16 scale]
constexpr int kRowF16 = 0, kRowQ8 = 1, kRowI8H = 2;
typedef unsigned v4u __attribute__((ext_vector_type(4)));
typedef unsigned v2u __attribute__((ext_vector_type(2)));

__host__ __device__ constexpr int row_bytes_of(int enc) {
    return enc == kRowF16 ? kHd * 2 : enc == kRowQ8 ? (kHd / 32) * 36 : kHd + (kHd / 32) * 2;
}

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

// The split-K kernels on the matrix cores (decode_attn_mfma.hip); `total` work-groups, one per
// (entry, kv head, page range).
// `start` / `stop`: optional events attached to the dispatch (its own begin and end time stamps)
// kp.bd != nullptr: the step kernels that read the batch from the descriptor (`total` is then the fixed grid).
hipError_t launch_decode_attn_mfma(const AttnKernelParams& kp, int layout, bool step, bool sel, int32_t total,
                                   hipStream_t stream, hipEvent_t start = nullptr, hipEvent_t stop = nullptr);

}  // namespace bkv
