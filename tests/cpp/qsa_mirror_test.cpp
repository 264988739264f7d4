// Drives the C++ host mirror of the reference interface (breccia_amd/csrc/qsa.hpp) the way
// the reference's own conformance tests drive Qsa (crates/breccia-kernels/tests/
// attn_conformance.rs:1172-1275 for the layout recipe), checking the GPU against the CPU
// oracle.  Built by __graft_entry__.build(); run on the GPU box by tests/test_gpu_cpp_mirror.py.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <vector>

#include "../../breccia_amd/csrc/qsa.hpp"

// CPU oracle (test infrastructure), oracle/bkv_oracle.c
extern "C" {
typedef struct {
    int32_t n_kv, head_dim, page_cells;
} bkvo_geom;
int bkvo_append_f16(const bkvo_geom*, uint16_t*, uint16_t*, const int32_t*, int64_t, int64_t, int64_t,
                    const float*, const float*);
int bkvo_gather(const bkvo_geom*, int, const void*, const void*, const int32_t*, int64_t, int64_t, float*,
                float*);
int bkvo_attend(const float*, const float*, const float*, const uint32_t*, size_t, int64_t, int32_t,
                int32_t, int32_t, const float*, float*, int);
void bkvo_normalish(uint64_t, size_t, float*);
void bkvo_indexer_score(const float*, const float*, size_t, int64_t, size_t, size_t, size_t, double*);
size_t bkvo_topk_blocks(const double*, size_t, size_t, int64_t, uint32_t*);
size_t bkvo_cells_of(const uint32_t*, size_t, uint32_t, uint32_t*);
void bkvo_rmsnorm(const float*, size_t, size_t, size_t, const float*, float, float*);
void bkvo_rope_table(double, size_t, size_t, float*);
void bkvo_rope_apply(const float*, size_t, size_t, size_t, const float*, size_t, const int32_t*, float*);
}

using namespace breccia::qsa;

static int failures = 0;
#define EXPECT(cond, ...)                                  \
    do {                                                   \
        if (!(cond)) {                                     \
            std::printf("FAIL %s:%d: ", __FILE__, __LINE__); \
            std::printf(__VA_ARGS__);                      \
            std::printf("\n");                             \
            ++failures;                                    \
        }                                                  \
    } while (0)

static void upload(float* dev, const std::vector<float>& h) {
    check(bkv_memcpy_h2d(dev, h.data(), h.size() * 4, nullptr));
    check(bkv_stream_sync(nullptr));
}

template <typename T>
static std::vector<T> download(const void* dev, size_t count) {
    std::vector<T> h(count);
    check(bkv_memcpy_d2h(h.data(), dev, count * sizeof(T), nullptr));
    check(bkv_stream_sync(nullptr));
    return h;
}

static void test_errors() {
    bool threw = false;
    try {
        QsaState::create(0, 64);
    } catch (const Error& e) {
        threw = e.status == BKV_ERR_INVALID;
    }
    EXPECT(threw, "capacity 0 must be refused");
    Qsa qsa;
    threw = false;
    try {
        qsa.workspace(0, 1);
    } catch (const Error& e) {
        threw = e.status == BKV_ERR_INVALID;
    }
    EXPECT(threw, "a workspace of 0 tokens must be refused");
}

static void test_layout_recipe() {
    // capacity 40 cells = 3 pages, 33 single-token appends from cell 5
    QsaState state = QsaState::create(40, 64);
    EXPECT(state.capacity_cells == 48, "capacity rounds up to pages, got %zu", state.capacity_cells);
    Qsa qsa;
    QsaWorkspace ws = qsa.workspace(1, 38);
    const bkvo_geom g{2, 256, 16};
    const int32_t table[3] = {0, 1, 2};
    std::vector<uint16_t> want_k(3 * 2 * 16 * 256, 0), want_v(want_k.size(), 0);
    for (int t = 0; t < 33; ++t) {
        const int cell = 5 + t;
        std::vector<float> k(512), v(512);
        for (int i = 0; i < 512; ++i) {
            k[i] = std::sin((float)(cell * 97 + i * 13) * 0.017f) * 3.0f;
            v[i] = std::cos((float)(cell * 61 + i * 7) * 0.031f) * 2.0f;
        }
        upload(ws.k_cur, k);
        upload(ws.v_cur, v);
        qsa.kv_append(state, ws, (size_t)cell);
        bkvo_append_f16(&g, want_k.data(), want_v.data(), table, 48, cell, 1, k.data(), v.data());
    }
    uint64_t nbytes = 0;
    void* kp = state.pool_ptr(0, &nbytes);
    EXPECT(nbytes == want_k.size() * 2, "k_pool is %llu bytes", (unsigned long long)nbytes);
    const auto got_k = download<uint16_t>(kp, want_k.size());
    const auto got_v = download<uint16_t>(state.pool_ptr(1), want_v.size());
    size_t bad = 0;
    for (size_t i = 0; i < want_k.size(); ++i) bad += (got_k[i] != want_k[i]) + (got_v[i] != want_v[i]);
    EXPECT(bad == 0, "%zu of %zu stored halves differ from the cache encoding", bad, 2 * want_k.size());
    std::printf("qsa kv layout+f16   %d K/V elements, %zu differ (33 cells, 3 pages)\n", 33 * 512, bad);

    // append past the capacity is an Err, not a launch (qsa/mod.rs:1108-1116)
    bool threw = false;
    try {
        qsa.kv_append(state, ws, 48);
    } catch (const Error& e) {
        threw = e.status == BKV_ERR_RANGE;
    }
    EXPECT(threw, "append at cell 48 of a 48-cell cache must be refused");

    state.reset();
    const auto zero = download<uint16_t>(state.pool_ptr(0), want_k.size());
    bad = 0;
    for (uint16_t h : zero) bad += h != 0;
    EXPECT(bad == 0, "reset must zero the pool");
    qsa.release(ws);
    state.release();
}

static void test_attention(const int T, const size_t pos0) {
    // 24 heads, gate read in place from q_full: T = 3 decode tokens after a 61-cell prefill, and a
    // chunk of 40 tokens at cells 24.., which apply() sends through the chunk kernel
    const int cells = 64, H = MODEL_N_HEAD, hd = MODEL_HEAD_DIM;
    QsaState state = QsaState::create(cells, 64);
    Qsa qsa;
    const bkvo_geom g{2, 256, 16};
    const int32_t table[4] = {0, 1, 2, 3};
    std::vector<float> k_all(cells * 512), v_all(cells * 512), q(T * H * hd), q_full(T * H * 2 * hd);
    bkvo_normalish(0xF1, k_all.size(), k_all.data());
    bkvo_normalish(0xF2, v_all.size(), v_all.data());
    bkvo_normalish(0xF3, q.size(), q.data());
    bkvo_normalish(0xF4, q_full.size(), q_full.data());
    QsaWorkspace fill = qsa.workspace(cells, cells);
    upload(fill.k_cur, k_all);
    upload(fill.v_cur, v_all);
    qsa.kv_append(state, fill, 0);
    QsaWorkspace ws = qsa.workspace(T, cells);
    upload(ws.q, q);
    upload(ws.q_full, q_full);
    qsa.attend(state, ws, pos0);
    qsa.apply(state, ws, pos0);
    check(bkv_device_sync());
    const auto out = download<float>(ws.attn_out, (size_t)T * H * hd);

    std::vector<uint16_t> pk(4 * 2 * 16 * 256, 0), pv(pk.size(), 0);
    bkvo_append_f16(&g, pk.data(), pv.data(), table, cells, 0, cells, k_all.data(), v_all.data());
    std::vector<float> kf(cells * 512), vf(cells * 512);
    bkvo_gather(&g, 0, pk.data(), pv.data(), table, 0, cells, kf.data(), vf.data());
    std::vector<uint32_t> cell_list(cells);
    for (int c = 0; c < cells; ++c) cell_list[c] = (uint32_t)c;
    double worst = 0.0;
    for (int t = 0; t < T; ++t) {
        std::vector<float> gate(H * hd), want(H * hd);
        for (int h = 0; h < H; ++h)
            std::memcpy(&gate[h * hd], &q_full[((size_t)t * H + h) * 2 * hd + hd], hd * 4);
        bkvo_attend(&q[(size_t)t * H * hd], kf.data(), vf.data(), cell_list.data(), cell_list.size(),
                    (int64_t)(pos0 + t), H, 2, hd, gate.data(), want.data(), 1);
        for (int i = 0; i < H * hd; ++i) {
            const double w = want[i], e = std::fabs((double)out[(size_t)t * H * hd + i] - w);
            worst = std::fmax(worst, e / std::fmax(std::fabs(w), 1.0));
        }
    }
    // the reference's bar: max |g-w| / max(|w|,1) <= 1e-5 (attn_conformance.rs:102-108, :1148-1151)
    EXPECT(worst <= 1e-5, "attention max_rel %.3e exceeds 1e-5", worst);
    std::printf("qsa attend+apply    T=%d, %d heads, gated: max_rel %.3e\n", T, H, worst);

    bool threw = false;
    try {
        qsa.apply(state, ws, pos0 + 1);  // one cell past the cache's 64
    } catch (const Error& e) {
        threw = e.status == BKV_ERR_RANGE;
    }
    EXPECT(threw, "attention past the capacity must be refused");
    qsa.release(ws);
    qsa.release(fill);
    state.release();
}

static void test_k_prep_append() {
    // k_norm -> rope_k -> kv_append in one call: 19 tokens at cells 9..27, the model's table
    const int T = 19, hd = MODEL_HEAD_DIM, max_pos = 64;
    const size_t pos0 = 9;
    QsaState state = QsaState::create(48, max_pos);
    Qsa qsa;
    QsaWorkspace ws = qsa.workspace(T, 28);
    std::vector<float> k(T * 512), v(T * 512), gamma(hd), table((size_t)max_pos * MODEL_N_ROT);
    bkvo_normalish(0xA1, k.size(), k.data());
    bkvo_normalish(0xA2, v.size(), v.data());
    bkvo_normalish(0xFEED, gamma.size(), gamma.data());
    check(bkv_rope_table(1e7, MODEL_N_ROT, max_pos, table.data()));
    std::vector<float> want_table(table.size());
    bkvo_rope_table(1e7, MODEL_N_ROT, max_pos, want_table.data());
    EXPECT(std::memcmp(table.data(), want_table.data(), table.size() * 4) == 0, "rotary table differs");
    float *gamma_dev = nullptr, *table_dev = nullptr;
    check(bkv_dev_alloc(gamma.size() * 4, (void**)&gamma_dev));
    check(bkv_dev_alloc(table.size() * 4, (void**)&table_dev));
    upload(gamma_dev, gamma);
    upload(table_dev, table);
    upload(ws.k_cur, k);
    upload(ws.v_cur, v);
    qsa.k_prep_append(state, ws, gamma_dev, table_dev, max_pos, pos0);
    check(bkv_device_sync());

    std::vector<float> normed(k.size()), rotated(k.size());
    bkvo_rmsnorm(k.data(), (size_t)T * 2, hd, 1, gamma.data(), MODEL_RMS_EPS, normed.data());
    std::vector<int32_t> positions(T * 2);
    for (int r = 0; r < T * 2; ++r) positions[r] = (int32_t)(pos0 + r / 2);
    bkvo_rope_apply(normed.data(), (size_t)T * 2, hd, MODEL_N_ROT, table.data(), max_pos, positions.data(),
                    rotated.data());
    const bkvo_geom g{2, 256, 16};
    const int32_t pages[3] = {0, 1, 2};
    std::vector<uint16_t> want_k(3 * 2 * 16 * 256, 0), want_v(want_k.size(), 0);
    bkvo_append_f16(&g, want_k.data(), want_v.data(), pages, 48, (int64_t)pos0, T, rotated.data(), v.data());
    const auto got_k = download<uint16_t>(state.pool_ptr(0), want_k.size());
    const auto got_v = download<uint16_t>(state.pool_ptr(1), want_v.size());
    size_t bad = 0;
    for (size_t i = 0; i < want_k.size(); ++i) bad += (got_k[i] != want_k[i]) + (got_v[i] != want_v[i]);
    EXPECT(bad == 0, "k_prep_append: %zu halves differ from norm -> rotary -> append on the CPU", bad);
    std::printf("qsa k_prep_append   T=%d at cell %zu: %zu differing halves\n", T, pos0, bad);
    check(bkv_dev_free(gamma_dev));
    check(bkv_dev_free(table_dev));
    qsa.release(ws);
    state.release();
}

static void test_selection_then_attention() {
    // crates/breccia-kernels/tests/attn_conformance.rs:897-1004 through the mirror: 2062 cells,
    // select 512 of 515 blocks + the tail block, then attend exactly that list
    const int cells = 2062, n_blocks = 515, H = MODEL_N_HEAD, hd = MODEL_HEAD_DIM;
    const size_t pos0 = cells - 1;
    QsaState state = QsaState::create(cells, 4096);
    Qsa qsa;
    qsa.bind(state);
    std::vector<float> idx_q(IDX_N_HEAD * IDX_DIM), pooled((n_blocks + 1) * IDX_DIM), k_all((size_t)cells * 512),
        v_all((size_t)cells * 512), q(H * hd), q_full(H * 2 * hd);
    bkvo_normalish(0xE1, idx_q.size(), idx_q.data());
    bkvo_normalish(0xE2, pooled.size(), pooled.data());
    bkvo_normalish(0xE3, k_all.size(), k_all.data());
    bkvo_normalish(0xE4, v_all.size(), v_all.data());
    bkvo_normalish(0xE5, q.size(), q.data());
    bkvo_normalish(0xE6, q_full.size(), q_full.data());
    QsaWorkspace fill = qsa.workspace(cells, cells);
    upload(fill.k_cur, k_all);
    upload(fill.v_cur, v_all);
    qsa.kv_append(state, fill, 0);
    QsaWorkspace ws = qsa.workspace(1, cells);
    EXPECT(ws.n_blocks == (size_t)n_blocks && ws.max_ids == 513, "workspace sizes %zu %zu", ws.n_blocks, ws.max_ids);
    float* pooled_dev = nullptr;
    check(bkv_dev_alloc(pooled.size() * 4, (void**)&pooled_dev));
    upload(pooled_dev, pooled);
    upload(ws.idx_q, idx_q);
    upload(ws.q, q);
    upload(ws.q_full, q_full);
    qsa.select(ws, pooled_dev, pos0);
    qsa.attend(state, ws, pos0);
    qsa.apply(state, ws, pos0);
    check(bkv_device_sync());
    const auto got_ids = download<uint32_t>(ws.ids, ws.max_ids);
    const auto got_count = download<uint32_t>(ws.counts, 1);
    const auto out = download<float>(ws.attn_out, (size_t)H * hd);

    std::vector<double> scores(n_blocks);
    bkvo_indexer_score(idx_q.data(), pooled.data(), n_blocks, (int64_t)pos0, IDX_N_HEAD, IDX_DIM, IDX_BLOCK,
                       scores.data());
    std::vector<uint32_t> want_ids(IDX_TOPK_BLOCKS + 1);
    const size_t want_n = bkvo_topk_blocks(scores.data(), n_blocks, IDX_TOPK_BLOCKS, (int64_t)(pos0 / IDX_BLOCK),
                                           want_ids.data());
    EXPECT(got_count[0] == want_n, "selection length %u vs %zu", got_count[0], want_n);
    EXPECT(std::memcmp(got_ids.data(), want_ids.data(), want_n * 4) == 0, "selection order/set differs");

    const bkvo_geom g{2, 256, 16};
    const int pages = (cells + 15) / 16;
    std::vector<int32_t> table(pages);
    for (int i = 0; i < pages; ++i) table[i] = i;
    std::vector<uint16_t> pk((size_t)pages * 2 * 16 * 256, 0), pv(pk.size(), 0);
    bkvo_append_f16(&g, pk.data(), pv.data(), table.data(), (int64_t)pages * 16, 0, cells, k_all.data(), v_all.data());
    std::vector<float> kf((size_t)cells * 512), vf((size_t)cells * 512);
    bkvo_gather(&g, 0, pk.data(), pv.data(), table.data(), 0, cells, kf.data(), vf.data());
    std::vector<uint32_t> cell_list(want_n * IDX_BLOCK);
    const size_t n_cells = bkvo_cells_of(want_ids.data(), want_n, IDX_BLOCK, cell_list.data());
    std::vector<float> gate(H * hd), want(H * hd);
    for (int h = 0; h < H; ++h) std::memcpy(&gate[h * hd], &q_full[(size_t)h * 2 * hd + hd], hd * 4);
    bkvo_attend(q.data(), kf.data(), vf.data(), cell_list.data(), n_cells, (int64_t)pos0, H, 2, hd, gate.data(),
                want.data(), 4);
    double worst = 0.0;
    for (int i = 0; i < H * hd; ++i) {
        const double w = want[i], e = std::fabs((double)out[i] - w);
        worst = std::fmax(worst, e / std::fmax(std::fabs(w), 1.0));
    }
    EXPECT(worst <= 1e-5, "sparse attention max_rel %.3e exceeds 1e-5", worst);
    std::printf("qsa select+attend   blocks=%d selected=%u: ids exact, max_rel %.3e\n", n_blocks, got_count[0], worst);
    check(bkv_dev_free(pooled_dev));
    qsa.release(ws);
    qsa.release(fill);
    state.release();
}

int main() {
    try {
        test_errors();
        test_layout_recipe();
        test_attention(3, 61);
        test_attention(40, 24);
        test_k_prep_append();
        test_selection_then_attention();
    } catch (const Error& e) {
        std::printf("FAIL: unexpected error %d: %s\n", (int)e.status, e.what());
        return 2;
    }
    std::printf(failures ? "%d check(s) failed\n" : "all checks passed\n", failures);
    return failures ? 1 : 0;
}
