// Host-side mirror of the reference's operator interface for the paged-KV path, in C++
// over the C ABI (the reference's own host code is Rust: crates/breccia-kernels/src/qsa/
// mod.rs).  Same names, argument meaning and error behaviour as there, so that a caller or
// a test written against `QsaState` / `Qsa::{kv_append, attend, apply}` reads the same:
//
//   QsaState::with_layout(capacity_cells, max_pos, VLayout)   qsa/mod.rs:399-535
//   QsaState::reset / bytes / release                         qsa/mod.rs:551-602
//   Qsa::workspace(tokens, n_kv_after)                        qsa/mod.rs:928-1048
//   Qsa::kv_append(state, ws, pos0)                           qsa/mod.rs:1105-1131
//   Qsa::attend(state, ws, pos0), Qsa::apply(state, ws, pos0) qsa/mod.rs:1382-1522
//
// As in the reference, one QsaState is the paged K/V cache of one layer of one sequence
// with an identity page table (qsa/mod.rs:477-481); errors are returned before anything is
// launched; every call enqueues on one in-order stream.  Differences, all forced by the
// fused kernel: the score matrix is never materialised, so attend() only validates and
// apply() launches the split-K kernel plus the merge (which applies sigmoid(gate) read in
// place from q_full at h*2*head_dim + head_dim + d, as shaders/qsa_attn_apply.comp does);
// apply() attends the lists in ws.ids / ws.counts once select() or topk_dense() has filled
// them, and every cell 0..=pos otherwise -- through the chunk kernel from GQA_MIN_TOKENS tokens
// on, as the reference switches to its kv-head-group kernels there (qsa/mod.rs:132-143).
#pragma once

#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/breccia_kv.h"
#include "../../include/breccia_kv_bench.h"  // device allocation for the workspace (the reference: its Vulkan context)

namespace breccia {
namespace qsa {

constexpr int MODEL_N_HEAD = 24;      // qsa/mod.rs:69
constexpr int MODEL_N_KV_HEAD = 2;    // qsa/mod.rs:71
constexpr int MODEL_HEAD_DIM = 256;   // qsa/mod.rs:73
constexpr int PAGE_CELLS = 16;        // qsa/mod.rs:116
constexpr int IDX_N_HEAD = 4;         // qsa/mod.rs:77
constexpr int IDX_DIM = 128;          // qsa/mod.rs:79
constexpr int IDX_BLOCK = 4;          // qsa/mod.rs:81
constexpr int IDX_TOPK_BLOCKS = 512;  // qsa/mod.rs:85 (IDX_TOP_K 2048 cells / IDX_BLOCK)
constexpr int GQA_MIN_TOKENS = 16;    // qsa/mod.rs:135: calls of at least this many tokens take the chunk kernels
constexpr int MODEL_N_ROT = 64;       // ops/mod.rs:454
constexpr float MODEL_RMS_EPS = 1e-6f;  // ops/mod.rs:316

enum class VLayout { F16, Q8_0 };  // qsa/mod.rs:242-254

struct Error : std::runtime_error {
    bkv_status status;
    Error(bkv_status st, const std::string& what) : std::runtime_error(what), status(st) {}
};

inline void check(bkv_status st) {
    if (st != BKV_OK) throw Error(st, bkv_last_error());
}

class QsaState {
public:
    // Capacity is rounded up to whole pages; pools start zeroed; the page table is the
    // identity.  capacity_cells == 0 or max_pos == 0 is an error (qsa/mod.rs:405-409).
    static QsaState with_layout(size_t capacity_cells, size_t max_pos, VLayout v_layout) {
        if (capacity_cells == 0 || max_pos == 0)
            throw Error(BKV_ERR_INVALID, "qsa state needs capacity_cells > 0 and max_pos > 0");
        QsaState s;
        const size_t pages = (capacity_cells + PAGE_CELLS - 1) / PAGE_CELLS;
        bkv_pool_desc d{};
        d.n_layers = 1;
        d.n_pages = (int32_t)pages;
        d.n_kv_head = MODEL_N_KV_HEAD;
        d.head_dim = MODEL_HEAD_DIM;
        d.page_cells = PAGE_CELLS;
        d.layout = v_layout == VLayout::F16 ? BKV_LAYOUT_F16 : BKV_LAYOUT_Q8V;
        d.max_seqs = 1;
        d.max_pages_per_seq = (int32_t)pages;
        check(bkv_pool_create(&d, &s.pool));
        try {
            check(bkv_seq_create_identity(s.pool, (int32_t)pages, &s.seq));
        } catch (...) {
            bkv_pool_destroy(s.pool);
            throw;
        }
        s.capacity_cells = pages * PAGE_CELLS;
        s.max_pos = max_pos;
        s.v_layout = v_layout;
        return s;
    }
    static QsaState create(size_t capacity_cells, size_t max_pos) {
        return with_layout(capacity_cells, max_pos, VLayout::F16);
    }

    // Back to construction-time contents (qsa/mod.rs:551-570).
    void reset(void* stream = nullptr) {
        check(bkv_pool_reset(pool, stream));
        check(bkv_seq_create_identity(pool, (int32_t)(capacity_cells / PAGE_CELLS), &seq));
    }
    uint64_t bytes() const { return bkv_pool_bytes(pool); }
    void release() {
        if (pool) check(bkv_pool_destroy(pool));
        pool = nullptr;
    }
    // Device base and size of k_pool (which = 0) / v_pool (which = 1).
    void* pool_ptr(int which, uint64_t* nbytes = nullptr) const {
        void* p = nullptr;
        check(bkv_pool_layer_ptr(pool, 0, which, &p, nbytes));
        return p;
    }

    bkv_pool* pool = nullptr;
    int32_t seq = -1;
    size_t capacity_cells = 0;
    size_t max_pos = 0;
    VLayout v_layout = VLayout::F16;
};

// The device buffers one call reads and writes (the subset of the reference's
// QsaWorkspace that the paged-KV path touches), all f32.
struct QsaWorkspace {
    size_t tokens = 0;
    float* q_full = nullptr;    // [T, n_head, 2*head_dim]  q | gate per head
    float* q = nullptr;         // [T, n_head, head_dim]
    float* k_cur = nullptr;     // [T, n_kv_head, head_dim]
    float* v_cur = nullptr;     // [T, n_kv_head, head_dim]
    float* attn_out = nullptr;  // [T, n_head, head_dim]
    // block selection (qsa/mod.rs:604-660): indexer queries in, id lists out
    float* idx_q = nullptr;     // [T, IDX_N_HEAD, IDX_DIM]
    uint32_t* ids = nullptr;    // [T, max_ids] selected block ids
    uint32_t* counts = nullptr; // [T]
    size_t n_blocks = 0;        // completed (pooled) blocks the selection ranges over
    size_t max_ids = 0;         // topk_blocks + 1
    size_t topk_blocks = 0;
    bool selected = false;      // a selection call has filled ids / counts
};

class Qsa {
public:
    explicit Qsa(int n_head = MODEL_N_HEAD, void* stream = nullptr) : n_head_(n_head), stream_(stream) {}

    // tokens == 0 is an error (qsa/mod.rs:929-931).
    // n_kv_after = cells the cache holds once this call's tokens are appended; it sizes the
    // selection (n_blocks = completed 4-cell blocks, qsa/mod.rs:928-1048).
    QsaWorkspace workspace(size_t tokens, size_t n_kv_after) const {
        if (tokens == 0) throw Error(BKV_ERR_INVALID, "a qsa workspace needs tokens > 0");
        QsaWorkspace ws;
        ws.tokens = tokens;
        ws.n_blocks = n_kv_after / IDX_BLOCK;
        ws.topk_blocks = IDX_TOPK_BLOCKS;
        ws.max_ids = ws.topk_blocks + 1;
        check(bkv_dev_alloc(tokens * IDX_N_HEAD * IDX_DIM * 4, (void**)&ws.idx_q));
        check(bkv_dev_alloc(tokens * ws.max_ids * 4, (void**)&ws.ids));
        check(bkv_dev_alloc(tokens * 4, (void**)&ws.counts));
        const size_t hd = MODEL_HEAD_DIM;
        check(bkv_dev_alloc(tokens * n_head_ * 2 * hd * 4, (void**)&ws.q_full));
        check(bkv_dev_alloc(tokens * n_head_ * hd * 4, (void**)&ws.q));
        check(bkv_dev_alloc(tokens * MODEL_N_KV_HEAD * hd * 4, (void**)&ws.k_cur));
        check(bkv_dev_alloc(tokens * MODEL_N_KV_HEAD * hd * 4, (void**)&ws.v_cur));
        check(bkv_dev_alloc(tokens * n_head_ * hd * 4, (void**)&ws.attn_out));
        return ws;
    }
    void release(QsaWorkspace& ws) const {
        for (float** p : {&ws.q_full, &ws.q, &ws.k_cur, &ws.v_cur, &ws.attn_out, &ws.idx_q}) {
            if (*p) check(bkv_dev_free(*p));
            *p = nullptr;
        }
        if (ws.ids) check(bkv_dev_free(ws.ids));
        if (ws.counts) check(bkv_dev_free(ws.counts));
        ws.ids = ws.counts = nullptr;
    }

    // Append ws.tokens rows of ws.k_cur / ws.v_cur at cells pos0.. (qsa/mod.rs:1107-1131).
    // pos0 + tokens > capacity is an error, never a launch.
    void kv_append(const QsaState& state, const QsaWorkspace& ws, size_t pos0) const {
        const int64_t p0 = (int64_t)pos0;
        const int32_t n = (int32_t)ws.tokens;
        if (pos0 + ws.tokens <= state.capacity_cells) {
            // the allocator's length follows the highest cell written
            const int64_t len = bkv_seq_len(state.pool, state.seq);
            if ((int64_t)(pos0 + ws.tokens) > len)
                check(bkv_seq_reserve(state.pool, state.seq, (int64_t)(pos0 + ws.tokens), nullptr, 0,
                                      nullptr));
        }
        check(bkv_append(state.pool, 0, 1, &state.seq, &p0, &n, ws.k_cur, ws.v_cur, stream_));
    }

    // Qsa::k_norm + Qsa::rope_k + Qsa::kv_append in one launch (qsa/mod.rs:1051-1058,
    // :1079-1089, :1105-1131): ws.k_cur is normalised with k_norm_gamma[head_dim], rotated
    // over the first MODEL_N_ROT dims at positions pos0.. (identity positions, as the
    // reference's state.positions holds), and stored; ws.k_cur itself is left unchanged.
    void k_prep_append(const QsaState& state, const QsaWorkspace& ws, const float* k_norm_gamma,
                       const float* rope_table, int32_t rope_max_pos, size_t pos0) const {
        const int64_t p0 = (int64_t)pos0;
        const int32_t n = (int32_t)ws.tokens;
        if (pos0 + ws.tokens <= state.capacity_cells) {
            const int64_t len = bkv_seq_len(state.pool, state.seq);
            if ((int64_t)(pos0 + ws.tokens) > len)
                check(bkv_seq_reserve(state.pool, state.seq, (int64_t)(pos0 + ws.tokens), nullptr, 0,
                                      nullptr));
        }
        check(bkv_append_kprep(state.pool, 0, 1, &state.seq, &p0, &n, ws.k_cur, ws.v_cur, k_norm_gamma,
                               MODEL_RMS_EPS, rope_table, MODEL_N_ROT, rope_max_pos, nullptr, stream_));
    }

    // Qsa::idx_score + Qsa::topk (qsa/mod.rs:1234-1376): score ws.n_blocks pooled indexer keys
    // (idx_pooled: device f32 [n_blocks, IDX_DIM], the sequence's QsaState::idx_pooled) against
    // every token's ws.idx_q and leave the selected block ids in ws.ids / ws.counts.
    void select(QsaWorkspace& ws, const float* idx_pooled, size_t pos0) const {
        std::vector<int64_t> pos(ws.tokens);
        std::vector<const float*> pooled(ws.tokens, idx_pooled);
        std::vector<int32_t> nb(ws.tokens, (int32_t)ws.n_blocks);
        for (size_t t = 0; t < ws.tokens; ++t) pos[t] = (int64_t)(pos0 + t);
        check(bkv_select_blocks(pool_of_last_state_, (int32_t)ws.tokens, pos.data(), ws.idx_q, pooled.data(),
                                nb.data(), IDX_N_HEAD, IDX_DIM, (int32_t)ws.topk_blocks, ws.ids,
                                (int64_t)ws.max_ids, ws.counts, (int32_t)ws.max_ids, stream_));
        ws.selected = true;
    }
    // Qsa::topk_dense (qsa/mod.rs:1363-1376): every visible block, ascending, no scores read.
    void topk_dense(QsaWorkspace& ws, size_t pos0) const {
        std::vector<int64_t> pos(ws.tokens);
        for (size_t t = 0; t < ws.tokens; ++t) pos[t] = (int64_t)(pos0 + t);
        check(bkv_topk_blocks(pool_of_last_state_, (int32_t)ws.tokens, pos.data(), nullptr,
                              (int32_t)ws.n_blocks, (int32_t)ws.topk_blocks, 1, ws.ids, (int64_t)ws.max_ids,
                              ws.counts, (int32_t)ws.max_ids, stream_));
        ws.selected = true;
    }
    // The selection calls run on the library context of a cache: name it once.
    void bind(const QsaState& state) { pool_of_last_state_ = state.pool; }

    // Range checks of the attention call; nothing is launched (no score matrix exists).
    void attend(const QsaState& state, const QsaWorkspace& ws, size_t pos0) const {
        if (pos0 + ws.tokens > state.capacity_cells)
            throw Error(BKV_ERR_RANGE, "attend: cells " + std::to_string(pos0) + ".." +
                                           std::to_string(pos0 + ws.tokens) + " exceed the cache's " +
                                           std::to_string(state.capacity_cells));
        if (ws.selected && ws.tokens > BKV_MAX_BATCH)
            throw Error(BKV_ERR_INVALID, "attend: selection lists are a decode shape (tokens <= " +
                                             std::to_string(BKV_MAX_BATCH) + ")");
    }

    // out[t][h][:] = sigmoid(gate) * softmax(q.K/sqrt(d)) . V over cells 0..=pos0+t.
    void apply(const QsaState& state, const QsaWorkspace& ws, size_t pos0) const {
        attend(state, ws, pos0);
        std::vector<int32_t> seqs(ws.tokens, state.seq);
        std::vector<int64_t> pos(ws.tokens);
        for (size_t t = 0; t < ws.tokens; ++t) pos[t] = (int64_t)(pos0 + t);
        const int64_t hd = MODEL_HEAD_DIM;
        if (ws.selected) {
            // over the lists a selection call left in ws.ids / ws.counts, as the reference does
            check(bkv_decode_attn_select(state.pool, 0, (int32_t)ws.tokens, seqs.data(), pos.data(), n_head_,
                                         ws.q, ws.q_full + hd, (int64_t)n_head_ * 2 * hd, 2 * hd, 0.0625f,
                                         ws.ids, (int64_t)ws.max_ids, ws.counts, (int32_t)ws.max_ids,
                                         ws.attn_out, stream_));
            return;
        }
        if (ws.tokens >= (size_t)GQA_MIN_TOKENS) {
            // a chunk: the reference's kv-head-group kernels (qsa/mod.rs:132-143), here the
            // matrix-core chunk kernel -- one call, every row of the chunk, K/V read once per block
            // of query rows
            const int64_t p0 = (int64_t)pos0;
            const int32_t n = (int32_t)ws.tokens;
            check(bkv_prefill_attn(state.pool, 0, 1, &state.seq, &p0, &n, n_head_, ws.q, ws.q_full + hd,
                                   (int64_t)n_head_ * 2 * hd, 2 * hd, 0.0625f, ws.attn_out, stream_));
            return;
        }
        check(bkv_decode_attn(state.pool, 0, (int32_t)ws.tokens, seqs.data(), pos.data(), n_head_, ws.q,
                              ws.q_full + hd, (int64_t)n_head_ * 2 * hd, 2 * hd, 0.0625f, ws.attn_out,
                              stream_));
    }

private:
    int n_head_;
    void* stream_;
    bkv_pool* pool_of_last_state_ = nullptr;
};

}  // namespace qsa
}  // namespace breccia
