// Host-side page allocator and per-sequence block tables (no HIP here).
//
// The reference has no allocator (docs/plan/PDF-GAP-ANALYSIS.md:56-60); its page
// table is an identity map written once (crates/breccia-kernels/src/qsa/mod.rs:
// 477-481).  The shape below follows the reference's design notes for the planned
// subsystem (docs/reference-engines/02-kv-and-context.md:543-548, :566-581,
// :617-620): fixed 16-token pages, per-page {id, refcount}, a free queue, whole
// pages move between tiers and a page lives in exactly one tier.
#pragma once

#include <cstdint>
#include <deque>
#include <string>
#include <vector>

namespace bkv {

struct PagePair {
    int32_t src;
    int32_t dst;
};

// One (row, column) -> value change of the device block-table arena that has not
// been pushed to the GPU yet.
struct TableUpdate {
    int32_t offset;  // row * max_pages_per_seq + column
    int32_t value;
};

enum class AllocErr { Ok = 0, Invalid, Range, NoPages, State };

class PageAllocator {
public:
    PageAllocator(int32_t n_pages, int32_t page_cells, int32_t max_seqs, int32_t max_pages_per_seq);

    AllocErr seq_create(int32_t* seq_out, std::string& err);
    AllocErr seq_create_identity(int32_t n_pages, int32_t* seq_out, std::string& err);
    AllocErr seq_fork(int32_t parent, int64_t n_tokens, int32_t* child_out, std::string& err);
    AllocErr seq_free(int32_t seq, std::string& err);
    AllocErr seq_reserve(int32_t seq, int64_t new_len, PagePair* cow, int32_t cow_cap,
                         int32_t* n_cow, std::string& err);
    AllocErr seq_truncate(int32_t seq, int64_t new_len, std::string& err);
    // Eviction bookkeeping: pages [lp0, lp0+n) must be complete, resident and
    // exclusively owned.  detach returns their physical ids and frees them.
    AllocErr seq_detach_pages(int32_t seq, int32_t lp0, int32_t n, std::vector<int32_t>& phys_out,
                              std::string& err);
    // Restore bookkeeping: entries [lp0, lp0+n) must be -1; fresh pages are attached.
    AllocErr seq_attach_pages(int32_t seq, int32_t lp0, int32_t n, std::vector<int32_t>& phys_out,
                              std::string& err);
    // A new sequence whose first n logical pages are the given live physical pages (one more
    // reference each) and whose length is n whole pages: how a request adopts a cached prefix.
    AllocErr seq_create_shared(const int32_t* pages, int32_t n, int32_t* seq_out, std::string& err);
    // References held by an owner that is not a sequence (the prefix tree).
    AllocErr retain_page(int32_t page, std::string& err);
    AllocErr release_page(int32_t page, std::string& err);
    // A free page handed to a non-sequence owner (one external reference): where a cached page
    // that comes back from a lower tier lands.
    AllocErr retain_fresh_page(int32_t* page_out, std::string& err);
    int32_t external_refs(int32_t page) const { return external_[(size_t)page]; }
    AllocErr set_free_order(const int32_t* order, int32_t n, std::string& err);
    void reset();

    bool seq_valid(int32_t seq) const {
        return seq >= 0 && seq < max_seqs_ && seqs_[(size_t)seq].live;
    }
    int64_t seq_len(int32_t seq) const { return seqs_[(size_t)seq].len; }
    int32_t seq_n_pages(int32_t seq) const { return seqs_[(size_t)seq].n_pages; }
    int64_t seq_capacity(int32_t seq) const {
        return (int64_t)seqs_[(size_t)seq].n_pages * page_cells_;
    }
    const int32_t* seq_table(int32_t seq) const {
        return table_.data() + (size_t)seq * (size_t)max_pages_per_seq_;
    }
    // True when every page covering cells [0, n_cells) is resident (entry >= 0).
    bool seq_resident(int32_t seq, int64_t n_cells) const;
    int32_t refcount(int32_t page) const { return refcount_[(size_t)page]; }
    int32_t n_pages() const { return n_pages_; }
    int32_t free_pages() const { return (int32_t)free_.size(); }
    int32_t page_cells() const { return page_cells_; }
    int32_t max_seqs() const { return max_seqs_; }
    int32_t max_pages_per_seq() const { return max_pages_per_seq_; }

    // Changes not yet mirrored on the device, in the order they were made.
    std::vector<TableUpdate>& pending() { return pending_; }

    bool check(std::string& err) const;

private:
    struct Seq {
        bool live = false;
        int64_t len = 0;
        int32_t n_pages = 0;
    };

    int32_t take_page();
    void drop_page(int32_t page);
    void set_entry(int32_t seq, int32_t col, int32_t value);

    int32_t n_pages_, page_cells_, max_seqs_, max_pages_per_seq_;
    std::vector<int32_t> refcount_;
    std::vector<int32_t> external_;  // part of refcount_ held by non-sequence owners
    std::deque<int32_t> free_;  // FIFO: the longest-free page is reused first
    std::vector<Seq> seqs_;
    std::vector<int32_t> table_;  // [max_seqs][max_pages_per_seq], -1 = none
    std::vector<TableUpdate> pending_;
};

}  // namespace bkv
