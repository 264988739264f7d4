// Host-side page allocator and block tables.  See allocator.hpp for provenance.
#include "allocator.hpp"

#include <algorithm>
#include <cstdio>

namespace bkv {

namespace {
std::string fmt(const char* f, long long a = 0, long long b = 0, long long c = 0) {
    char buf[256];
    std::snprintf(buf, sizeof buf, f, a, b, c);
    return buf;
}
}  // namespace

PageAllocator::PageAllocator(int32_t n_pages, int32_t page_cells, int32_t max_seqs,
                             int32_t max_pages_per_seq)
    : n_pages_(n_pages),
      page_cells_(page_cells),
      max_seqs_(max_seqs),
      max_pages_per_seq_(max_pages_per_seq),
      refcount_((size_t)n_pages, 0),
      external_((size_t)n_pages, 0),
      seqs_((size_t)max_seqs),
      table_((size_t)max_seqs * (size_t)max_pages_per_seq, -1) {
    for (int32_t p = 0; p < n_pages; ++p) free_.push_back(p);
}

void PageAllocator::reset() {
    std::fill(refcount_.begin(), refcount_.end(), 0);
    std::fill(external_.begin(), external_.end(), 0);
    free_.clear();
    for (int32_t p = 0; p < n_pages_; ++p) free_.push_back(p);
    for (int32_t s = 0; s < max_seqs_; ++s) {
        Seq& q = seqs_[(size_t)s];
        if (q.live)
            for (int32_t c = 0; c < q.n_pages; ++c) set_entry(s, c, -1);
        q = Seq{};
    }
}

AllocErr PageAllocator::set_free_order(const int32_t* order, int32_t n, std::string& err) {
    if (n != (int32_t)free_.size()) {
        err = fmt("free order lists %lld pages but %lld are free", n, (long long)free_.size());
        return AllocErr::Invalid;
    }
    std::vector<char> seen((size_t)n_pages_, 0);
    for (int32_t i = 0; i < n; ++i) {
        const int32_t p = order[i];
        if (p < 0 || p >= n_pages_ || refcount_[(size_t)p] != 0 || seen[(size_t)p]) {
            err = fmt("free order entry %lld (page %lld) is not a distinct free page", i, p);
            return AllocErr::Invalid;
        }
        seen[(size_t)p] = 1;
    }
    free_.assign(order, order + n);
    return AllocErr::Ok;
}

int32_t PageAllocator::take_page() {
    const int32_t p = free_.front();
    free_.pop_front();
    refcount_[(size_t)p] = 1;
    return p;
}

void PageAllocator::drop_page(int32_t page) {
    if (--refcount_[(size_t)page] == 0) free_.push_back(page);
}

void PageAllocator::set_entry(int32_t seq, int32_t col, int32_t value) {
    const size_t off = (size_t)seq * (size_t)max_pages_per_seq_ + (size_t)col;
    if (table_[off] == value) return;
    table_[off] = value;
    pending_.push_back(TableUpdate{(int32_t)off, value});
}

AllocErr PageAllocator::seq_create(int32_t* seq_out, std::string& err) {
    for (int32_t s = 0; s < max_seqs_; ++s) {
        if (!seqs_[(size_t)s].live) {
            seqs_[(size_t)s] = Seq{};
            seqs_[(size_t)s].live = true;
            *seq_out = s;
            return AllocErr::Ok;
        }
    }
    err = fmt("all %lld sequence slots are live", max_seqs_);
    return AllocErr::NoPages;
}

AllocErr PageAllocator::seq_create_identity(int32_t n, int32_t* seq_out, std::string& err) {
    if (n <= 0 || n > n_pages_ || n > max_pages_per_seq_) {
        err = fmt("identity sequence of %lld pages does not fit (pool %lld, table row %lld)", n,
                  n_pages_, max_pages_per_seq_);
        return AllocErr::Invalid;
    }
    for (int32_t p = 0; p < n; ++p) {
        if (refcount_[(size_t)p] != 0) {
            err = fmt("identity sequence needs pages 0..%lld free, page %lld is held", n - 1, p);
            return AllocErr::State;
        }
    }
    int32_t s;
    const AllocErr e = seq_create(&s, err);
    if (e != AllocErr::Ok) return e;
    free_.erase(std::remove_if(free_.begin(), free_.end(), [n](int32_t p) { return p < n; }),
                free_.end());
    for (int32_t p = 0; p < n; ++p) {
        refcount_[(size_t)p] = 1;
        set_entry(s, p, p);
    }
    seqs_[(size_t)s].n_pages = n;
    *seq_out = s;
    return AllocErr::Ok;
}

AllocErr PageAllocator::seq_create_shared(const int32_t* pages, int32_t n, int32_t* seq_out,
                                          std::string& err) {
    if (n < 0 || n > max_pages_per_seq_ || (n > 0 && !pages)) {
        err = fmt("shared sequence of %lld pages does not fit a block-table row of %lld", n,
                  max_pages_per_seq_);
        return AllocErr::Invalid;
    }
    for (int32_t c = 0; c < n; ++c) {
        if (pages[c] < 0 || pages[c] >= n_pages_ || refcount_[(size_t)pages[c]] <= 0) {
            err = fmt("shared sequence: entry %lld (page %lld) is not a live page", c, pages[c]);
            return AllocErr::State;
        }
    }
    int32_t s;
    const AllocErr e = seq_create(&s, err);
    if (e != AllocErr::Ok) return e;
    for (int32_t c = 0; c < n; ++c) {
        ++refcount_[(size_t)pages[c]];
        set_entry(s, c, pages[c]);
    }
    seqs_[(size_t)s].n_pages = n;
    seqs_[(size_t)s].len = (int64_t)n * page_cells_;
    *seq_out = s;
    return AllocErr::Ok;
}

AllocErr PageAllocator::retain_page(int32_t page, std::string& err) {
    if (page < 0 || page >= n_pages_ || refcount_[(size_t)page] <= 0) {
        err = fmt("retain: page %lld is not live", page);
        return AllocErr::State;
    }
    ++refcount_[(size_t)page];
    ++external_[(size_t)page];
    return AllocErr::Ok;
}

AllocErr PageAllocator::release_page(int32_t page, std::string& err) {
    if (page < 0 || page >= n_pages_ || external_[(size_t)page] <= 0) {
        err = fmt("release: page %lld holds no external reference", page);
        return AllocErr::State;
    }
    --external_[(size_t)page];
    drop_page(page);
    return AllocErr::Ok;
}

AllocErr PageAllocator::retain_fresh_page(int32_t* page_out, std::string& err) {
    if (free_.empty()) {
        err = "no free page";
        return AllocErr::NoPages;
    }
    const int32_t p = take_page();
    external_[(size_t)p] = 1;
    *page_out = p;
    return AllocErr::Ok;
}

bool PageAllocator::seq_resident(int32_t seq, int64_t n_cells) const {
    const int64_t pages = (n_cells + page_cells_ - 1) / page_cells_;
    if (pages > seqs_[(size_t)seq].n_pages) return false;
    const int32_t* row = seq_table(seq);
    for (int64_t c = 0; c < pages; ++c)
        if (row[c] < 0) return false;
    return true;
}

AllocErr PageAllocator::seq_fork(int32_t parent, int64_t n_tokens, int32_t* child_out,
                                 std::string& err) {
    if (!seq_valid(parent)) {
        err = fmt("fork: sequence %lld is not live", parent);
        return AllocErr::Range;
    }
    const Seq& p = seqs_[(size_t)parent];
    if (n_tokens < 0 || n_tokens > p.len) {
        err = fmt("fork: %lld tokens requested but the parent holds %lld", n_tokens, p.len);
        return AllocErr::Range;
    }
    if (!seq_resident(parent, n_tokens)) {
        err = "fork: the shared prefix has pages that are swapped out";
        return AllocErr::State;
    }
    int32_t s;
    const AllocErr e = seq_create(&s, err);
    if (e != AllocErr::Ok) return e;
    const int32_t pages = (int32_t)((n_tokens + page_cells_ - 1) / page_cells_);
    const int32_t* prow = seq_table(parent);
    for (int32_t c = 0; c < pages; ++c) {
        ++refcount_[(size_t)prow[c]];
        set_entry(s, c, prow[c]);
    }
    seqs_[(size_t)s].n_pages = pages;
    seqs_[(size_t)s].len = n_tokens;
    *child_out = s;
    return AllocErr::Ok;
}

AllocErr PageAllocator::seq_free(int32_t seq, std::string& err) {
    if (!seq_valid(seq)) {
        err = fmt("free: sequence %lld is not live (double free?)", seq);
        return AllocErr::State;
    }
    Seq& q = seqs_[(size_t)seq];
    const int32_t* row = seq_table(seq);
    for (int32_t c = 0; c < q.n_pages; ++c) {
        const int32_t p = row[c];
        if (p >= 0) {
            if (refcount_[(size_t)p] <= 0) {
                err = fmt("free: page %lld of sequence %lld has refcount %lld (underflow)", p, seq,
                          refcount_[(size_t)p]);
                return AllocErr::State;
            }
            drop_page(p);
        }
        set_entry(seq, c, -1);
    }
    q = Seq{};
    return AllocErr::Ok;
}

AllocErr PageAllocator::seq_reserve(int32_t seq, int64_t new_len, PagePair* cow, int32_t cow_cap,
                                    int32_t* n_cow, std::string& err) {
    if (n_cow) *n_cow = 0;
    if (!seq_valid(seq)) {
        err = fmt("reserve: sequence %lld is not live", seq);
        return AllocErr::Range;
    }
    Seq& q = seqs_[(size_t)seq];
    if (new_len < q.len) {
        err = fmt("reserve: new length %lld is below the current length %lld (use truncate)",
                  new_len, q.len);
        return AllocErr::Range;
    }
    const int64_t need_pages = (new_len + page_cells_ - 1) / page_cells_;
    if (need_pages > max_pages_per_seq_) {
        err = fmt("reserve: %lld cells need %lld pages but a block-table row holds %lld", new_len,
                  need_pages, max_pages_per_seq_);
        return AllocErr::Range;
    }
    if (new_len == q.len) return AllocErr::Ok;

    // Pages that will be written: those covering cells [len, new_len).
    const int32_t first = (int32_t)(q.len / page_cells_);
    const int32_t last = (int32_t)((new_len - 1) / page_cells_);
    const bool first_is_partial = (q.len % page_cells_) != 0;
    const int32_t* row = seq_table(seq);

    int32_t fresh = 0, copies = 0;
    for (int32_t c = first; c <= last; ++c) {
        if (c >= q.n_pages) {
            ++fresh;
        } else if (row[c] < 0) {
            err = fmt("reserve: logical page %lld of sequence %lld is swapped out", c, seq);
            return AllocErr::State;
        } else if (refcount_[(size_t)row[c]] > 1) {
            ++fresh;
            if (c == first && first_is_partial) ++copies;
        }
    }
    if (fresh > (int32_t)free_.size()) {
        err = fmt("reserve: %lld pages needed, %lld free", fresh, (long long)free_.size());
        return AllocErr::NoPages;
    }
    if (copies > 0 && (cow == nullptr || cow_cap < copies)) {
        err = fmt("reserve: %lld copy-on-write pair(s) to report but room for %lld", copies,
                  cow_cap);
        return AllocErr::Invalid;
    }

    int32_t reported = 0;
    for (int32_t c = first; c <= last; ++c) {
        if (c >= q.n_pages) {
            set_entry(seq, c, take_page());
        } else {
            const int32_t old = row[c];
            if (refcount_[(size_t)old] > 1) {
                const int32_t fresh_page = take_page();
                if (c == first && first_is_partial) cow[reported++] = PagePair{old, fresh_page};
                drop_page(old);
                set_entry(seq, c, fresh_page);
            }
        }
    }
    if (last + 1 > q.n_pages) q.n_pages = last + 1;
    q.len = new_len;
    if (n_cow) *n_cow = reported;
    return AllocErr::Ok;
}

AllocErr PageAllocator::seq_truncate(int32_t seq, int64_t new_len, std::string& err) {
    if (!seq_valid(seq)) {
        err = fmt("truncate: sequence %lld is not live", seq);
        return AllocErr::Range;
    }
    Seq& q = seqs_[(size_t)seq];
    if (new_len < 0 || new_len > q.len) {
        err = fmt("truncate: length %lld is outside 0..%lld", new_len, q.len);
        return AllocErr::Range;
    }
    q.len = new_len;
    return AllocErr::Ok;
}

AllocErr PageAllocator::seq_detach_pages(int32_t seq, int32_t lp0, int32_t n,
                                         std::vector<int32_t>& phys_out, std::string& err) {
    phys_out.clear();
    if (!seq_valid(seq)) {
        err = fmt("evict: sequence %lld is not live", seq);
        return AllocErr::Range;
    }
    Seq& q = seqs_[(size_t)seq];
    if (lp0 < 0 || n < 0 || (int64_t)lp0 + n > q.n_pages) {
        err = fmt("evict: pages %lld..%lld are outside the sequence's %lld pages", lp0,
                  (long long)lp0 + n, q.n_pages);
        return AllocErr::Range;
    }
    if ((int64_t)(lp0 + n) * page_cells_ > q.len) {
        err = fmt("evict: only complete pages move; page %lld is partially filled (length %lld)",
                  (long long)lp0 + n - 1, q.len);
        return AllocErr::State;
    }
    const int32_t* row = seq_table(seq);
    for (int32_t c = lp0; c < lp0 + n; ++c) {
        if (row[c] < 0) {
            err = fmt("evict: logical page %lld is already swapped out", c);
            return AllocErr::State;
        }
        if (refcount_[(size_t)row[c]] != 1) {
            err = fmt("evict: page %lld (logical %lld) is shared, refcount %lld", row[c], c,
                      refcount_[(size_t)row[c]]);
            return AllocErr::State;
        }
    }
    for (int32_t c = lp0; c < lp0 + n; ++c) {
        phys_out.push_back(row[c]);
        drop_page(row[c]);
        set_entry(seq, c, -1);
    }
    return AllocErr::Ok;
}

AllocErr PageAllocator::seq_attach_pages(int32_t seq, int32_t lp0, int32_t n,
                                         std::vector<int32_t>& phys_out, std::string& err) {
    phys_out.clear();
    if (!seq_valid(seq)) {
        err = fmt("restore: sequence %lld is not live", seq);
        return AllocErr::Range;
    }
    Seq& q = seqs_[(size_t)seq];
    if (lp0 < 0 || n < 0 || (int64_t)lp0 + n > q.n_pages) {
        err = fmt("restore: pages %lld..%lld are outside the sequence's %lld pages", lp0,
                  (long long)lp0 + n, q.n_pages);
        return AllocErr::Range;
    }
    const int32_t* row = seq_table(seq);
    for (int32_t c = lp0; c < lp0 + n; ++c) {
        if (row[c] >= 0) {
            err = fmt("restore: logical page %lld is resident (page %lld)", c, row[c]);
            return AllocErr::State;
        }
    }
    if (n > (int32_t)free_.size()) {
        err = fmt("restore: %lld pages needed, %lld free", n, (long long)free_.size());
        return AllocErr::NoPages;
    }
    for (int32_t c = lp0; c < lp0 + n; ++c) {
        const int32_t p = take_page();
        phys_out.push_back(p);
        set_entry(seq, c, p);
    }
    return AllocErr::Ok;
}

bool PageAllocator::check(std::string& err) const {
    std::vector<int32_t> seen((size_t)n_pages_, 0);
    for (int32_t s = 0; s < max_seqs_; ++s) {
        const Seq& q = seqs_[(size_t)s];
        const int32_t* row = seq_table(s);
        for (int32_t c = 0; c < max_pages_per_seq_; ++c) {
            const int32_t p = row[c];
            if (!q.live || c >= q.n_pages) {
                if (p != -1) {
                    err = fmt("table entry (%lld,%lld) = %lld outside a live sequence", s, c, p);
                    return false;
                }
                continue;
            }
            if (p < -1 || p >= n_pages_) {
                err = fmt("table entry (%lld,%lld) = %lld is not a page id", s, c, p);
                return false;
            }
            if (p >= 0) ++seen[(size_t)p];
        }
        if (q.live && q.len > (int64_t)q.n_pages * page_cells_) {
            err = fmt("sequence %lld: length %lld exceeds its %lld pages", s, q.len, q.n_pages);
            return false;
        }
    }
    std::vector<char> is_free((size_t)n_pages_, 0);
    for (int32_t p : free_) {
        if (p < 0 || p >= n_pages_ || is_free[(size_t)p]) {
            err = fmt("free queue holds page %lld twice or out of range", p);
            return false;
        }
        is_free[(size_t)p] = 1;
    }
    for (int32_t p = 0; p < n_pages_; ++p) {
        if (seen[(size_t)p] + external_[(size_t)p] != refcount_[(size_t)p]) {
            err = fmt("page %lld: refcount %lld but %lld table entries and external references", p,
                      refcount_[(size_t)p], seen[(size_t)p] + external_[(size_t)p]);
            return false;
        }
        if ((refcount_[(size_t)p] == 0) != (is_free[(size_t)p] != 0)) {
            err = fmt("page %lld: refcount %lld disagrees with the free queue", p,
                      refcount_[(size_t)p]);
            return false;
        }
    }
    return true;
}

}  // namespace bkv
