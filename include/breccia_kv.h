/*
 * breccia_kv.h -- C ABI of the MI355X paged-KV library (libbreccia_kv.so).
 *
 * One GPU, one process.  Every entry point returns a bkv_status; on failure
 * bkv_last_error() holds a thread-local message naming the failing check.  Every
 * size / range violation is a host-side error returned BEFORE anything is
 * launched (the reference's contract: crates/breccia-kernels/src/qsa/mod.rs:
 * 1108-1116, :405-409, :929-931) -- never a device fault.
 *
 * Calls that take a `stream` only enqueue work on it (the HIP analogue of the
 * reference recording into a device's open batch, crates/breccia-kernels/src/
 * ops/mod.rs:205-222): results are visible to later work on the same stream.
 * `stream` is a hipStream_t passed as void* (NULL = the default stream).
 * One pool may be driven from several streams, by one host thread at a time: a pool is
 * not thread-safe and takes no lock of its own (the reference guards its queue with a
 * mutex, crates/breccia-vk/src/ctx.rs:565; here that lock belongs to the owner of the pool --
 * a Rust wrapper is Send and not Sync).  Different pools may be used from different threads;
 * bkv_last_error and the wait options are the only process-wide state.  What the pool owns and every call shares --
 * the argument ring, the block tables, the split-K and score workspaces, the swap
 * staging -- it orders across streams by itself with events; the order between the
 * caller's own data (an append before the attention that reads its rows, on another
 * stream) is the caller's to keep, as with any work on streams.
 *
 * Reference items each group replaces are cited per declaration; paths are
 * relative to the reference tree, `qsa/` = crates/breccia-kernels/src/qsa/.
 */
#ifndef BRECCIA_KV_H
#define BRECCIA_KV_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum bkv_status {
    BKV_OK = 0,
    BKV_ERR_INVALID = 1,    /* bad argument / geometry */
    BKV_ERR_RANGE = 2,      /* position, page or sequence out of range */
    BKV_ERR_NO_PAGES = 3,   /* allocator exhausted */
    BKV_ERR_STATE = 4,      /* refcount / ownership / residency rule violated */
    BKV_ERR_NO_DEVICE = 5,  /* pool was created host-only, or HIP is unusable */
    BKV_ERR_HIP = 6,        /* a HIP runtime call failed (message names it) */
    BKV_ERR_NOMEM = 7,      /* host or pinned-host allocation failed */
    BKV_ERR_TIMEOUT = 8     /* a bounded host wait ran out (message names what it waited for);
                               the work is still enqueued, nothing was cancelled */
} bkv_status;

/* How K and V rows are stored.  qsa/mod.rs:242-254 (VLayout). */
typedef enum bkv_layout {
    BKV_LAYOUT_F16 = 0, /* f16 K and V: 2 B / element (reference default)                */
    BKV_LAYOUT_Q8V = 1, /* f16 K; V as q8_0 blocks [f32 scale][32 x i8] = 36 B / 32 values
                           (reference BRECCIA_KV_Q8V, shaders/qsa_kv_append.comp:38-44) */
    BKV_LAYOUT_I8H = 2  /* int8 K and V, row = [head_dim x i8][head_dim/32 x f16 scale],
                           34 B / 32 values (no reference counterpart)                   */
} bkv_layout;

enum {
    BKV_POOL_HOST_ONLY = 1u /* allocator + block tables only; device calls fail with
                               BKV_ERR_NO_DEVICE (for hosts without a GPU) */
};

#define BKV_MAX_BATCH 64      /* (sequence, position) entries per append / attention call */
#define BKV_MAX_HEAD_GROUP 16 /* q heads per kv head */
#define BKV_MAX_KV_HEAD 16    /* kv heads of a pool */

/* Pool geometry.  One pool = n_layers x (K pool, V pool), each laid out exactly as
 * the reference's k_pool / v_pool (qsa/mod.rs:20-35):
 *   row  = (page * n_kv_head + kv_head) * page_cells + cell % page_cells
 *   f16 element index = row * head_dim + d   (u32 word = index / 2, even = low half)
 * plus a device-resident int32 block table per sequence (the reference's
 * `page_table`, one u32 per logical page).  Page ids are shared by all layers. */
typedef struct bkv_pool_desc {
    int32_t n_layers;
    int32_t n_pages;
    int32_t n_kv_head;          /* 1 .. BKV_MAX_KV_HEAD */
    int32_t head_dim;           /* multiple of 32, <= 256; kernels are tuned for 256 */
    int32_t page_cells;         /* 16 */
    int32_t layout;             /* bkv_layout */
    int32_t max_seqs;           /* live sequences the block-table arena holds */
    int32_t max_pages_per_seq;  /* block-table row length */
    uint32_t flags;             /* BKV_POOL_* */
} bkv_pool_desc;

typedef struct bkv_pool bkv_pool;

typedef struct bkv_page_pair {
    int32_t src;
    int32_t dst;
} bkv_page_pair;

/* ---- errors / version ------------------------------------------------------ */
const char *bkv_last_error(void);
const char *bkv_version(void);

/* ---- pool lifecycle ---------------------------------------------------------
 * Replaces QsaState::with_layout / reset / bytes / release (qsa/mod.rs:399-535,
 * :551-570, :572-585, :591-602).  Pools are zeroed at creation and by reset, as in
 * the reference; reset also frees every sequence. */
bkv_status bkv_pool_create(const bkv_pool_desc *desc, bkv_pool **out);
bkv_status bkv_pool_destroy(bkv_pool *pool);
bkv_status bkv_pool_reset(bkv_pool *pool, void *stream);
bkv_status bkv_pool_get_desc(const bkv_pool *pool, bkv_pool_desc *out);
uint64_t bkv_pool_bytes(const bkv_pool *pool);              /* device bytes held */
uint64_t bkv_page_bytes(const bkv_pool *pool, int which);   /* one layer; 0 = K, 1 = V */
/* Fill every K/V pool byte with `byte` (the reference's BRECCIA_FAULT_POISON_QSA
 * knob fills with NaN words, qsa/mod.rs:509-523; 0xff bytes are NaN in f16 and f32). */
bkv_status bkv_pool_fill(bkv_pool *pool, int byte, void *stream);
/* Raw device base of one layer's K (which=0) or V (which=1) pool, for callers that
 * dump or diff pool bytes (the reference's BRECCIA_DUMP_*, graph.rs:2204-2229).
 * Bytes written through this pointer (or swapped in from a foreign dump) bypass the append
 * path's store rule.  One consequence is part of the contract: an f16 code with exponent field 0
 * (a subnormal) is never stored by any append entry point; if foreign bytes hold one, bkv_gather
 * and the int8 layout's scale load read it as zero (the reference's load rule,
 * shaders/f16_storage.glsl:58-69) while the attention kernels multiply it as the IEEE value it
 * encodes.  Pools written only through this library read the same everywhere. */
bkv_status bkv_pool_layer_ptr(const bkv_pool *pool, int32_t layer, int which, void **dev_ptr,
                              uint64_t *bytes);

/* ---- page allocator / block tables (host side) -----------------------------
 * No reference implementation exists (docs/plan/PDF-GAP-ANALYSIS.md:56-60); shaped by
 * the reference's design notes (docs/reference-engines/02-kv-and-context.md:543-548,
 * :566-581, :617-620): 16-token pages, {id, refcount, free queue}, only whole pages
 * move, a page is in exactly one tier.  A sequence handle is a small integer. */
bkv_status bkv_seq_create(bkv_pool *pool, int32_t *seq_out);
/* A sequence whose logical page i is physical page i for i < n_pages: the
 * reference's identity page table (qsa/mod.rs:477-481). */
bkv_status bkv_seq_create_identity(bkv_pool *pool, int32_t n_pages, int32_t *seq_out);
/* Child shares every page of the parent's first `n_tokens` cells (refcount + 1). */
bkv_status bkv_seq_fork(bkv_pool *pool, int32_t parent, int64_t n_tokens, int32_t *child_out);
bkv_status bkv_seq_free(bkv_pool *pool, int32_t seq);
/* Make cells [0, new_len) addressable and cells [len, new_len) privately writable:
 * allocates missing pages; if the page holding cell `len` is shared (refcount > 1)
 * and partially filled, it is replaced by a fresh page and (old, new) is reported in
 * cow_pairs -- the caller must bkv_page_copy those pairs before appending.  A shared
 * page that no other sequence holds any more (refcount back to 1) is written in place.
 * On BKV_ERR_NO_PAGES nothing is changed. */
bkv_status bkv_seq_reserve(bkv_pool *pool, int32_t seq, int64_t new_len, bkv_page_pair *cow_pairs,
                           int32_t cow_capacity, int32_t *n_cow);
/* Set the sequence's length without touching pages (speculative rollback:
 * rejected cells are simply overwritten later, docs/specs/qwen4exp-architecture.md:750-759). */
bkv_status bkv_seq_truncate(bkv_pool *pool, int32_t seq, int64_t new_len);
int64_t bkv_seq_len(const bkv_pool *pool, int32_t seq);           /* -1 on error */
int64_t bkv_seq_capacity(const bkv_pool *pool, int32_t seq);      /* cells addressable */
int32_t bkv_seq_n_pages(const bkv_pool *pool, int32_t seq);
/* Host view of the block table (valid until the next allocator call); entry -1 =
 * page swapped out. */
const int32_t *bkv_seq_block_table(const bkv_pool *pool, int32_t seq);
int32_t bkv_page_refcount(const bkv_pool *pool, int32_t page);    /* -1 on error */
int32_t bkv_pool_free_pages(const bkv_pool *pool);
/* Self-check of the allocator's invariants (sum of refcounts == table entries, free
 * list disjoint from live pages, ...).  BKV_OK or BKV_ERR_STATE with a message. */
bkv_status bkv_pool_check(const bkv_pool *pool);
/* Placement hook: make the free queue hand pages out in `order`, which must be a
 * permutation of the pages that are free right now (fragmentation studies, tests). */
bkv_status bkv_pool_set_free_order(bkv_pool *pool, const int32_t *order, int32_t n);

/* ---- prefix tree: reuse of cached prefixes ------------------------------------
 * No reference implementation; the shape follows its design notes (docs/reference-engines/
 * 02-kv-and-context.md:543-548 page-aligned 16-token hash granularity, :566-581 tier
 * movement rules, :600-603 radix tree with refcount / last_access, eviction as a strategy,
 * pinned read-only subtree).  One tree per pool, one node per COMPLETE page, keyed by that
 * page's token ids; the tree holds one reference on every page it lists, so a listed prefix
 * outlives the sequence that computed it.  Host-side only; nothing is launched.
 *
 * bkv_prefix_insert: list the complete pages of the first n_tokens tokens of `seq` (whose K/V
 *   the caller has appended).  Prefixes already listed keep their pages (first publisher
 *   wins); *new_pages = nodes added.
 * bkv_prefix_match: how many leading tokens of `tokens` are covered by listed pages, in
 *   whatever tier (a multiple of the page size); does not count as a use.
 * bkv_seq_create_from_prefix: a new sequence that shares those pages (refcount + 1 each),
 *   length = *matched_tokens; the caller appends the rest, starting on a fresh page -- a
 *   page-aligned share never needs a copy-on-write copy.
 * bkv_prefix_evict: drop least-recently-used unpinned leaves that nobody else holds until
 *   want_pages went back to the free queue.  bkv_seq_reserve does this by itself when it
 *   runs out of free pages, before it reports BKV_ERR_NO_PAGES.
 * bkv_prefix_pin: pin != 0 pins, 0 unpins the listed chain of `tokens` (injected read-only
 *   context: never evicted while pinned).
 * bkv_pool_reset clears the tree. */
bkv_status bkv_prefix_insert(bkv_pool *pool, int32_t seq, const int32_t *tokens, int64_t n_tokens,
                             int32_t *new_pages);
bkv_status bkv_prefix_match(bkv_pool *pool, const int32_t *tokens, int64_t n_tokens,
                            int64_t *matched_tokens);
bkv_status bkv_seq_create_from_prefix(bkv_pool *pool, const int32_t *tokens, int64_t n_tokens,
                                      int32_t *seq_out, int64_t *matched_tokens);
bkv_status bkv_prefix_evict(bkv_pool *pool, int32_t want_pages, int32_t *freed);
bkv_status bkv_prefix_pin(bkv_pool *pool, const int32_t *tokens, int64_t n_tokens, int32_t pin,
                          int64_t *affected_tokens);
bkv_status bkv_prefix_stats(const bkv_pool *pool, int32_t *nodes, int32_t *evictable_pages,
                            int32_t *pinned_nodes);
bkv_status bkv_prefix_clear(bkv_pool *pool);

/* Lower tiers for evicted prefixes (the design notes' T2 "pinned, hard byte cap" and T3 "NVMe,
 * chunked read", docs/reference-engines/02-kv-and-context.md:594-596, under the movement rules
 * of :566-572: only complete pages move, a page is in exactly one tier, promotion is chunked and
 * never part of a decode step).  No reference implementation.
 * bkv_prefix_tiers: host_bytes of pinned host memory (hipHostMalloc) and, when disk_path is not
 *   NULL, disk_bytes of the file disk_path (created or truncated; it is left in place when the
 *   pool goes) hold whole pages ([layer][K page | V page], bkv_swap_page_bytes each).  From
 *   then on an evicted prefix page is demoted instead of dropped: device -> host; when the host
 *   arena is full its least recently used page goes host -> disk, and when the file is full
 *   its least recently used leaf is dropped.  Demotion works upwards from the leaves, so along
 *   a chain of pages the tiers only go down.  bkv_prefix_match counts the pages of every tier;
 *   bkv_seq_create_from_prefix brings the matched chain's lower part back to fresh device
 *   pages (evicting other cached prefixes if it must) and adopts what is on the device after
 *   that.  bkv_prefix_insert of a sequence that has recomputed a demoted page hands that page
 *   to the tree at no transfer.  Transfers run on the pool's side stream; every later call
 *   that enqueues work on the pool (append, attention, page copy, swap, fill, reset, gather)
 *   waits for them on the device on its own stream -- writes through bkv_pool_layer_ptr are
 *   the caller's to order (bkv_swap_wait) -- and the host does not block except for file I/O
 *   and for the synchronisation before pages leave the device (the streams that wrote them
 *   are not known to the call) -- so with tiers configured bkv_seq_reserve, bkv_prefix_evict
 *   and bkv_seq_create_from_prefix must not be called while a stream is being captured
 *   into a graph.  host_bytes = 0 switches the tiers off and drops what they
 *   hold; calling it again resizes them the same way.  An I/O error on the file drops every
 *   cached prefix and reports BKV_ERR_STATE.
 * bkv_prefix_tier_stats: nodes_by_tier[3] = pages on the device / in host memory / on disk;
 *   moved[4] = pages demoted to host, demoted to disk, promoted, dropped (since creation). */
bkv_status bkv_prefix_tiers(bkv_pool *pool, uint64_t host_bytes, const char *disk_path,
                            uint64_t disk_bytes);
bkv_status bkv_prefix_tier_stats(const bkv_pool *pool, int32_t *nodes_by_tier, uint64_t *moved);
/* Promotion ahead of a request (the notes' "async, never on the decode critical path", :570-572):
 * brings the lower part of the chain that matches `tokens` back to device pages, as
 * bkv_seq_create_from_prefix would, without creating a sequence; the transfers are enqueued on
 * the side stream and not awaited.  Counts as a use of the chain.  *device_tokens = leading
 * tokens whose pages are on the device once the transfers are done. */
bkv_status bkv_prefix_prefetch(bkv_pool *pool, const int32_t *tokens, int64_t n_tokens,
                               int64_t *device_tokens);

/* ---- hot path ---------------------------------------------------------------
 * bkv_append replaces Qsa::kv_append + shaders/qsa_kv_append.comp (qsa/mod.rs:
 * 1105-1156): scatter n_tokens[i] new rows of sequence seqs[i] to cells pos0[i]..
 * through its block table, f32 -> cache encoding (f16 rule of shaders/
 * f16_storage.glsl:26-55; q8_0 rule of qsa_kv_append.comp:87-132).
 * k, v: device f32 [sum n_tokens][n_kv_head][head_dim], sequences concatenated in
 * call order.  Error if pos0+n_tokens exceeds the cells reserved for the sequence.
 * Does not change bkv_seq_len; call bkv_seq_reserve first. */
bkv_status bkv_append(bkv_pool *pool, int32_t layer, int32_t n_seqs, const int32_t *seqs,
                      const int64_t *pos0, const int32_t *n_tokens, const float *k_dev,
                      const float *v_dev, void *stream);
/* The same append from rows that are already binary16 (raw codes, same shape): what a
 * producer that keeps K/V in f16 hands over, half the bytes read.  The codes are widened
 * under the cache's load rule (shaders/f16_storage.glsl:58-69: exponent field 0 reads as a
 * signed zero) and then take the path of bkv_append, so the pool holds exactly what
 * bkv_append of the widened rows would have stored (f16 pools: the codes themselves, with
 * subnormals flushed to zero and NaN stored as infinity). */
bkv_status bkv_append_f16(bkv_pool *pool, int32_t layer, int32_t n_seqs, const int32_t *seqs,
                          const int64_t *pos0, const int32_t *n_tokens, const uint16_t *k_dev,
                          const uint16_t *v_dev, void *stream);

/* K preparation fused into the append: per (token, kv head) row RMSNorm with gamma
 * (Qsa::k_norm, qsa/mod.rs:1051-1058; ops/mod.rs:317-420), the partial NEOX-paired rotary
 * at the token's position (Qsa::rope_k, qsa/mod.rs:1079-1089; ops/mod.rs:634-654), then
 * bkv_append's store; V rows are appended untouched (qsa/cpu.rs:383-397).  One launch
 * instead of three and no f32 round trip of K.  Arithmetic follows the reference CPU path
 * operation for operation (ops/cpu.rs:52-88, :124-154: f64, one f32 rounding per stage).
 *   k_gamma_dev     device f32 [head_dim]
 *   eps             RMSNorm epsilon (the model's is 1e-6, ops/mod.rs:316)
 *   rope_table_dev  device f32 [max_pos][n_rot/2][2] of (cos, sin), see bkv_rope_table
 *   positions_dev   optional device int32 indexed by cell (the reference's positions
 *                   buffer, read at pos0 + token); NULL = the cell index itself.  When
 *                   given it must cover every cell written.  Positions outside the table
 *                   are clamped to its first / last row (shaders/ops_rope.comp).
 * Shapes, errors and ordering are those of bkv_append. */
bkv_status bkv_append_kprep(bkv_pool *pool, int32_t layer, int32_t n_seqs, const int32_t *seqs,
                            const int64_t *pos0, const int32_t *n_tokens, const float *k_dev,
                            const float *v_dev, const float *k_gamma_dev, float eps,
                            const float *rope_table_dev, int32_t n_rot, int32_t max_pos,
                            const int32_t *positions_dev, void *stream);
/* Host-side rotary table, the reference's formula (ops/cpu.rs:103-119, RopeTable::build
 * ops/mod.rs:475-487): table[p][i] = (cos, sin)(p * freq_base^(-2i/n_rot)) evaluated in
 * double and rounded to float.  host_out: max_pos * n_rot floats.  The model's table is
 * freq_base 1e7, n_rot 64. */
bkv_status bkv_rope_table(double freq_base, int32_t n_rot, int32_t max_pos, float *host_out);

/* bkv_decode_attn replaces Qsa::attend + Qsa::apply for decode shapes with the dense
 * selection (qsa/mod.rs:1382-1462, :1466-1522; shaders qsa_attn_scores_small,
 * ops_softmax, qsa_attn_apply_split, qsa_attn_apply_reduce; oracle qsa/cpu.rs:197-246):
 *   out[i][h][:] = sigmoid(gate[i][h][:]) * softmax_c(scale * q[i][h] . K[c]) . V[c],
 *   c over cells 0..pos[i] of sequence seqs[i], kv head = h * n_kv_head / n_q_head.
 * q, out: device f32 [n][n_q_head][head_dim].  gate_dev may be NULL (factor omitted);
 * otherwise gate(i,h,d) = gate_dev[i*gate_seq_stride + h*gate_head_stride + d] (the
 * reference reads it in place from q_full at h*512+256+d, shaders/qsa_attn_apply.comp).
 * The same sequence may appear several times with different pos (T > 1 decode).
 * One split-K online-softmax kernel plus one merge kernel; partials live in a
 * workspace the pool owns.  The split-K kernel multiplies on the matrix cores (all heads of a
 * kv head, up to 16, in one pass over the K/V rows; q and the probabilities as high + low f16
 * parts, quantised values as exact high + low f16 parts, so accuracy is that of f32
 * accumulation), on every layout, for this call, for selection lists and for the fused step. */
bkv_status bkv_decode_attn(bkv_pool *pool, int32_t layer, int32_t n, const int32_t *seqs,
                           const int64_t *pos, int32_t n_q_head, const float *q_dev,
                           const float *gate_dev, int64_t gate_seq_stride,
                           int64_t gate_head_stride, float scale, float *out_dev, void *stream);

/* bkv_decode_attn for callers that cannot allocate device memory (a stream being captured into a
 * graph, a tight serving loop, a harness that forbids hipMalloc).  No counterpart in the
 * reference.  Same arguments, checks, kernels and results (bit for bit) as bkv_decode_attn, but the
 * split-K partial results live in a static device array inside the library instead of a
 * workspace the pool allocated, and the call itself allocates nothing on the device, creates no
 * event and attaches no stage timer.  The array is sized for BKV_STATIC_WGS work-groups of 8 head
 * rows (8.06 MiB, one copy per GPU, held from library load to process end): a batch whose cut
 * needs more -- more than BKV_STATIC_WGS (entry, kv head) pairs at up to 8 q heads per kv head,
 * half as many at 9 to 16 -- is rejected with BKV_ERR_INVALID before anything is enqueued.
 * Every pool and every call on one GPU shares that GPU's array: calls that overlap on one GPU
 * (different streams, different pools) race; calls on one stream are ordered by the stream.
 * Nothing in the array has to start at zero.  Block-table changes still pending from allocator
 * calls are uploaded first, as in every other call (host heap and the pinned argument ring only)
 * -- except on a stream that is being captured, which cannot record that upload: there the call
 * returns BKV_ERR_STATE; make the allocator calls and any eager call before the capture (the rule
 * of step plans). */
#define BKV_STATIC_WGS 1024
bkv_status bkv_decode_attn_static(bkv_pool *pool, int32_t layer, int32_t n, const int32_t *seqs,
                                  const int64_t *pos, int32_t n_q_head, const float *q_dev,
                                  const float *gate_dev, int64_t gate_seq_stride,
                                  int64_t gate_head_stride, float scale, float *out_dev, void *stream);

/* Causal attention for chunks of many query tokens (prefill), on the matrix cores: the
 * reference's GQA pair for T >= 16 (shaders/qsa_attn_scores_gqa.comp, qsa_attn_apply_gqa.comp;
 * qsa/mod.rs:116-150), same contract as bkv_decode_attn (oracle qsa/cpu.rs:197-246, dense
 * selection): token t of chunk i, at position pos0[i] + t, attends cells 0..pos0[i]+t of
 * sequence seqs[i].  The chunk's own K/V must have been appended first.  q, out: device f32
 * [sum n_tokens][n_q_head][head_dim], chunks concatenated in call order; gate(token, h, d) =
 * gate_dev[token*gate_tok_stride + h*gate_head_stride + d] or NULL.  K and V enter the MFMAs
 * as the exact f16 the cache holds; q and the probabilities are f32 split into two f16 parts,
 * so accuracy is that of f32 accumulation.  q8_0 V blocks (BRECCIA_KV_Q8V in
 * qsa_attn_apply_gqa.comp:53-77) are dequantised once per work-group into two f16 terms whose
 * sum carries code * scale to 22 bits, and so are int8 K blocks.  All three layouts, head_dim
 * 256, 16-cell pages.  Written
 * for chunks of tens to thousands of tokens; a handful of tokens is bkv_decode_attn's case. */
bkv_status bkv_prefill_attn(bkv_pool *pool, int32_t layer, int32_t n_seqs, const int32_t *seqs,
                            const int64_t *pos0, const int32_t *n_tokens, int32_t n_q_head,
                            const float *q_dev, const float *gate_dev, int64_t gate_tok_stride,
                            int64_t gate_head_stride, float scale, float *out_dev, void *stream);

/* One decode step in one call: append the new token's K/V row of every listed sequence at cell
 * pos[i] and attend cells 0..pos[i] -- bkv_append of one token per sequence followed by
 * bkv_decode_attn, without the append launch (Qsa::kv_append + Qsa::attend + Qsa::apply of
 * a T = 1 call, qsa/mod.rs:1617-1639).  The work-group that owns the last page of a sequence
 * takes the row from k_new_dev / v_new_dev (f32 [n][n_kv_head][head_dim]), stores it in the
 * pool's layout with the append kernels' own encoders (f16 rule, q8_0 blocks, int8 blocks) --
 * the pool afterwards holds exactly what bkv_append would have written -- and uses it in
 * place of the stale pool row; the output is bit-identical to the two-call sequence.  Every
 * sequence at most once per call; the cell must have been reserved (bkv_seq_reserve) like for
 * bkv_append. */
bkv_status bkv_decode_step(bkv_pool *pool, int32_t layer, int32_t n, const int32_t *seqs,
                           const int64_t *pos, const float *k_new_dev, const float *v_new_dev,
                           int32_t n_q_head, const float *q_dev, const float *gate_dev,
                           int64_t gate_seq_stride, int64_t gate_head_stride, float scale,
                           float *out_dev, void *stream);

/* ---- step plans: a decode step that can be recorded once and replayed ------------------------
 * The reference records every stage of a layer into one open batch and submits once
 * (crates/breccia-kernels/src/ops/mod.rs:205-222, src/dispatch_batch.rs:46-59; contract test
 * tests/batching.rs:27-88: batched == unbatched bit for bit).  The HIP analogue is a graph: the
 * calls of one token are captured from a stream once and replayed for the tokens that follow.
 * bkv_decode_step cannot be captured usefully -- positions, block-table rows and the cut into
 * work-groups travel as kernel arguments, so a replay would repeat one token.  A step plan keeps
 * that batch in device memory instead:
 *   bkv_step_plan_create   checks, for every listed sequence, the `horizon` cells pos[i] ..
 *                          pos[i] + horizon - 1 the way bkv_decode_step checks one (reserved, on
 *                          the device, held by this sequence alone; each sequence once), pushes
 *                          pending block-table changes and writes the descriptor on `stream`.
 *   bkv_step_plan_decode   bkv_decode_step for the plan's batch at its current positions on one
 *                          layer: same kernels, same bytes in the pool, same output bits.  It
 *                          reads positions and the cut from the descriptor, uses a workspace of the
 *                          plan's own, copies nothing from the host, allocates nothing and attaches
 *                          no timer: it can be captured, any number of layers per token.
 *   bkv_step_plan_advance  one small kernel: every position moves on by one cell and the batch is
 *                          cut again on the device by the function the host uses (so a replayed
 *                          step sums its partial results in the order a fresh call would).  An
 *                          advance past the checked cells changes nothing and sets status 1.
 *   bkv_step_plan_state    waits for `stream`, then reports positions, advances done and status.
 * Between creation and the last replay the caller leaves the listed sequences alone (no free,
 * fork, truncate, evict): bkv_step_plan_decode looks at the plan's cells again on every call and
 * returns BKV_ERR_STATE when they are no longer reserved, resident and unshared, but a replayed
 * graph makes no such call.  Allocator calls for OTHER sequences are fine but must be followed by an
 * eager call on the pool before a capture begins, since their block-table changes cannot be
 * recorded.  Streams: the calls of a plan may come on any stream; a call that arrives on another
 * stream than the plan's previous one (creation included) is ordered behind it by the library, with
 * an event recorded there at that moment, and behind the last block-table scatter wherever that
 * ran.  A replayed graph holds none of these host-made orderings: replay on the stream the capture
 * was taken from, or order the streams yourself.  Destroy a pool's plans before the pool
 * (bkv_pool_destroy returns BKV_ERR_STATE while one is alive).  All three layouts. */
typedef struct bkv_step_plan bkv_step_plan;
bkv_status bkv_step_plan_create(bkv_pool *pool, int32_t n, const int32_t *seqs, const int64_t *pos,
                                int32_t horizon, int32_t n_q_head, void *stream, bkv_step_plan **out);
bkv_status bkv_step_plan_destroy(bkv_step_plan *plan);
bkv_status bkv_step_plan_decode(bkv_step_plan *plan, int32_t layer, const float *k_new_dev,
                                const float *v_new_dev, const float *q_dev, const float *gate_dev,
                                int64_t gate_seq_stride, int64_t gate_head_stride, float scale,
                                float *out_dev, void *stream);
bkv_status bkv_step_plan_advance(bkv_step_plan *plan, void *stream);
bkv_status bkv_step_plan_state(bkv_step_plan *plan, void *stream, int64_t *pos_out, uint32_t *steps_out,
                               int32_t *status_out);

/* The same attention over a selection list instead of every cell: the reference's real
 * long-context form (Qsa::attend / Qsa::apply read ws.ids [T, max_ids] and ws.counts [T],
 * qsa/mod.rs:1382-1462; shaders/qsa_attn_scores_small.comp; oracle qsa/cpu.rs:197-257).
 * Entry i attends the cells 4*b .. 4*b+3 of every block id b in
 *   ids_dev[i*id_stride + 0 .. min(counts_dev[i], max_ids)),
 * keeping only cells <= pos[i]; a block listed twice counts twice (as in the oracle); an
 * empty list gives a zero output row.  ids and counts are device u32 buffers (what a
 * top-k kernel leaves behind): their contents are never trusted for addressing -- a block
 * id is clamped to the sequence's blocks at or below pos[i] before any address is formed,
 * and its cells are masked by the causal test -- so no list content can fault.
 * Work is planned for max_ids blocks per entry, the bound the host knows. */
bkv_status bkv_decode_attn_select(bkv_pool *pool, int32_t layer, int32_t n, const int32_t *seqs,
                                  const int64_t *pos, int32_t n_q_head, const float *q_dev,
                                  const float *gate_dev, int64_t gate_seq_stride,
                                  int64_t gate_head_stride, float scale, const uint32_t *ids_dev,
                                  int64_t id_stride, const uint32_t *counts_dev, int32_t max_ids,
                                  float *out_dev, void *stream);

/* Block selection, the step that produces those lists (Qsa::idx_score + Qsa::topk,
 * qsa/mod.rs:1234-1376; shaders qsa_idx_score.comp, qsa_topk*.comp; oracle qsa/cpu.rs:93-152).
 * A block is 4 cells.  For list i (a query at pos[i]):
 *   score[b] = (1/sqrt(idx_dim)) * sum_h relu(idx_q[i][h] . pooled_i[b]),  b < n_blocks[i],
 *              dead when block b starts after pos[i];
 *   ids      = the topk_blocks best live blocks by descending score, ties to the lower block,
 *              then block pos[i]/4 (the query's own) when the selection missed it;
 *   counts[i] = length of the list (<= max_ids; the own block is dropped when there is no room).
 * Scores are computed as the CPU reference computes them (f64, sums in index order) and are
 * kept in a workspace the pool owns, so the emitted list is the reference CPU list exactly,
 * not merely a list of equal quality.
 *   idx_q_dev   device f32 [n][idx_n_head][idx_dim]  (the model: 4 x 128)
 *   pooled_dev  host array of n device pointers, f32 [n_blocks[i]][idx_dim] each (the
 *               sequence's pooled indexer keys, QsaState::idx_pooled)
 *   n_blocks    host array; pos host array.  topk_blocks <= 2048 (the model: 512). */
bkv_status bkv_select_blocks(bkv_pool *pool, int32_t n, const int64_t *pos, const float *idx_q_dev,
                             const float *const *pooled_dev, const int32_t *n_blocks,
                             int32_t idx_n_head, int32_t idx_dim, int32_t topk_blocks,
                             uint32_t *ids_dev, int64_t id_stride, uint32_t *counts_dev,
                             int32_t max_ids, void *stream);
/* The pooled indexer keys bkv_select_blocks scores against: Qsa::idx_pool + Qsa::idx_tail
 * (qsa/mod.rs:1167-1232; shaders qsa_idx_pool.comp, qsa_idx_tail.comp; oracle qsa/cpu.rs:154-185).
 * For every 4-cell block b completed by the tokens at pos0 .. pos0+tokens-1:
 *   pooled[b] = rotary(rmsnorm(mean(raw rows 4b..4b+3)) * gamma, position 4b),
 * rows before pos0 taken from the rolling tail (3 rows, slot = cell % 4) that the previous
 * call left; afterwards the tail holds the rows of the last, incomplete block.  Arithmetic as
 * on the CPU path (f32 mean in cell order, f64 norm and rotary), bit for bit.
 *   pooled_dev  device f32 [max_blocks][idx_dim];  tail_dev device f32 [3][idx_dim]
 *   idx_k_dev   device f32 [tokens][idx_dim] raw indexer keys of this call
 *   gamma_dev   device f32 [idx_dim];  rope_table_dev as for bkv_append_kprep (the model
 *               shares one table: n_rot 64 of idx_dim 128) */
bkv_status bkv_idx_pool(bkv_pool *pool, float *pooled_dev, int32_t max_blocks, float *tail_dev,
                        const float *idx_k_dev, int64_t pos0, int32_t tokens, const float *gamma_dev,
                        float eps, const float *rope_table_dev, int32_t n_rot, int32_t max_pos,
                        int32_t idx_dim, void *stream);
/* The top-k alone over f32 scores the caller already holds: Qsa::topk / Qsa::topk_dense on
 * ws.idx_scores [n][n_blocks] (qsa/mod.rs:1264-1376).  A score is live iff it is finite and
 * greater than -1e29 (the shaders' dead marker is -1e30; NaN and both infinities are dead, as
 * in the CPU path's filter, qsa/cpu.rs:139-143).  The scores are not
 * modified (the reference's serial kernel destroys them).  dense != 0: no scores read, every
 * visible block 0..min(n_blocks, own+1) in ascending order, then the own block if it lies
 * beyond n_blocks. */
bkv_status bkv_topk_blocks(bkv_pool *pool, int32_t n, const int64_t *pos, const float *scores_dev,
                           int32_t n_blocks, int32_t topk_blocks, int32_t dense, uint32_t *ids_dev,
                           int64_t id_stride, uint32_t *counts_dev, int32_t max_ids, void *stream);

/* Copy-on-write page copy: for every pair and every layer, K and V bytes of page
 * `src` -> page `dst`.  No reference implementation (nearest: dispatch_batch.rs:
 * 1130-1150 record_copy).  Pairs are host memory; dst pages must be distinct. */
bkv_status bkv_page_copy(bkv_pool *pool, const bkv_page_pair *pairs, int32_t n_pairs,
                         void *stream);

/* ---- VRAM <-> pinned host swap ------------------------------------------------
 * No reference implementation (nearest: gemv.rs:1023-1071 staging download/upload).
 * Host slab of one page = for each layer: [K page bytes][V page bytes]
 * (bkv_swap_page_bytes).  Device-side gather/scatter runs on `stream`; the PCIe
 * copy is a hipMemcpyAsync on the pool's side stream, fenced with events both ways.
 * bkv_swap_wait blocks the host until the side stream is idle; bkv_swap_fence makes
 * `stream` wait for it without blocking the host. */
uint64_t bkv_swap_page_bytes(const bkv_pool *pool);
bkv_status bkv_host_alloc(bkv_pool *pool, uint64_t bytes, void **host_out); /* hipHostMalloc */
bkv_status bkv_host_free(bkv_pool *pool, void *host);
/* Raw moves of physical pages (no allocator bookkeeping). */
bkv_status bkv_swap_out(bkv_pool *pool, const int32_t *pages, int32_t n, void *pinned_host,
                        void *stream);
bkv_status bkv_swap_in(bkv_pool *pool, const int32_t *pages, int32_t n, const void *pinned_host,
                       void *stream);
bkv_status bkv_swap_wait(bkv_pool *pool); /* bkv_swap_wait_for with the default deadline */
bkv_status bkv_swap_fence(bkv_pool *pool, void *stream);

/* ---- bounded host waits ---------------------------------------------------------
 * The reference never waits on its device without a deadline: crates/breccia-vk/src/ctx.rs:
 * 1545-1553 (WAIT_TIMEOUT_NS = 10 s, then a diagnostic instead of a hang).  The same here: every
 * host-side wait of the library for a stream or an event -- bkv_swap_wait, the transfers between
 * the prefix tiers, a free argument-ring slot, bkv_step_plan_state, bkv_timing_read -- polls the
 * HIP query call up to a deadline and then returns BKV_ERR_TIMEOUT with what it was waiting for.
 * Nothing is aborted or cancelled: the work stays enqueued and a later wait can succeed.
 * bkv_stream_wait is that wait for a caller's stream (timeout_ms < 0: no deadline; 0: a query).
 * bkv_wait_options sets, for the process, the deadline of the library's internal waits
 * (default 10000 ms; negative = none) and how long a wait spins on the query before it starts
 * napping 50 us between queries (default 4000 us: a thread asleep in hipStreamSynchronize is
 * woken tens of microseconds late, which a decode loop that waits per token would pay every
 * time; 0 = never spin).  The exceptions are the device-wide synchronisations HIP offers no
 * query for: pool destruction and reset, growing the selection workspace, and the one before
 * prefix pages leave the device. */
bkv_status bkv_stream_wait(void *stream, int64_t timeout_ms);
bkv_status bkv_swap_wait_for(bkv_pool *pool, int64_t timeout_ms);
bkv_status bkv_wait_options(int64_t timeout_ms, int64_t poll_us);
bkv_status bkv_wait_options_get(int64_t *timeout_ms_out, int64_t *poll_us_out);
/* Allocator-aware eviction of logical pages [lp0, lp0+n) of a sequence: each must be
 * complete and held only by this sequence; bytes go to pinned_host, the physical
 * pages return to the free list and the table entries become -1.  Restore allocates
 * fresh pages (ids may differ) and copies the bytes back. */
bkv_status bkv_seq_evict(bkv_pool *pool, int32_t seq, int32_t lp0, int32_t n, void *pinned_host,
                         void *stream);
bkv_status bkv_seq_restore(bkv_pool *pool, int32_t seq, int32_t lp0, int32_t n,
                           const void *pinned_host, void *stream);

/* ---- parity / debugging -------------------------------------------------------
 * Dequantised rows of cells [cell0, cell0+n) as f32 [n][n_kv_head][head_dim] in
 * the flat order the reference's CPU attend consumes (qsa/cpu.rs:219-222). */
bkv_status bkv_gather(bkv_pool *pool, int32_t layer, int32_t seq, int64_t cell0, int64_t n,
                      float *k_out_dev, float *v_out_dev, void *stream);

/* How a decode-attention batch would be cut into work-groups on a device of n_cu compute units:
 * the planning step of bkv_decode_attn / bkv_decode_step / bkv_decode_attn_select alone, on the
 * host, nothing launched (no pool or device needed).  pos[n] as for those calls; sel_groups > 0
 * plans every entry for that many groups of four listed blocks (a selection list of
 * 4 * sel_groups ids) instead of its pages.  splits_out[n], pps_out[n]: page ranges per entry and
 * pages per range; *total_out: work-groups of the launch.  BKV_ERR_INVALID when the batch needs
 * more work-groups than the partial-result workspace holds -- the error the attention calls
 * themselves return, before anything is enqueued (qsa/mod.rs:1108-1116). */
bkv_status bkv_attn_plan(int32_t n_cu, int32_t n_kv_head, int32_t n_q_head, int32_t n, const int64_t *pos,
                         int32_t sel_groups, int32_t *splits_out, int32_t *pps_out, int32_t *total_out);

/* ---- per-kernel GPU timing ------------------------------------------------------
 * The analogue of Qsa::stage_timings / Pipe::run_timed (qsa/mod.rs:1733-1970,
 * ops/mod.rs:251-274): while enabled, every hot-path call times each of its kernels
 * with an event pair that rides on the kernel's dispatch (hipExtLaunchKernelGGL): it
 * reads the kernel's own begin and end time stamps, what a profiler's kernel trace
 * reports, free of the queue time that event records around a launch would add.
 * bkv_timing_read waits for the events and returns launches and summed milliseconds of
 * one stage since the last reset.  Debug / benchmark only. */
typedef enum bkv_stage {
    BKV_STAGE_APPEND = 0,
    BKV_STAGE_ATTN_SPLIT = 1, /* split-K online-softmax kernel (the dominant one) */
    BKV_STAGE_ATTN_MERGE = 2,
    BKV_STAGE_PAGE_COPY = 3,
    BKV_STAGE_PREFILL_ATTN = 4, /* chunk attention (bkv_prefill_attn) */
    BKV_STAGE_APPEND_KPREP = 5, /* norm + rotary + append in one kernel */
    BKV_STAGE_IDX_POOL = 6,     /* pooled indexer keys + rolling tail */
    BKV_STAGE_IDX_SCORE = 7,
    BKV_STAGE_TOPK = 8,
    BKV_STAGE_PAGE_STAGE = 9,   /* gather / scatter of whole pages for swap and the prefix tiers */
    BKV_STAGE_COUNT = 10
} bkv_stage;
bkv_status bkv_timing_enable(bkv_pool *pool, int on);
bkv_status bkv_timing_reset(bkv_pool *pool);
bkv_status bkv_timing_read(bkv_pool *pool, int stage, uint64_t *launches, double *total_ms);

#ifdef __cplusplus
}
#endif
#endif /* BRECCIA_KV_H */
