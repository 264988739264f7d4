// Host-side prefix tree over whole pages: which physical pages already hold the K/V of a
// given token prefix, so that a new request adopts them instead of recomputing (no HIP here).
//
// The reference has no such structure; the shape follows its design notes for the planned
// subsystem (docs/reference-engines/02-kv-and-context.md:543-548 "hash granularity of 16
// tokens so prefix hits are page-aligned", :566-581 tier movement rules, :600-603
// "radix/: TreeNode{refcount, last_access, priority}, eviction as a strategy, read-only
// pinned subtree"): a trie with one node per complete page, keyed by that page's tokens;
// the tree holds one reference on every page it lists; eviction takes least-recently-used
// leaves that nobody else holds; pinned chains (injected read-only context) are never
// evicted.
#pragma once

#include <cstdint>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "allocator.hpp"

namespace bkv {

class PrefixTree {
public:
    PrefixTree(PageAllocator* alloc, int32_t page_cells) : alloc_(alloc), page_cells_(page_cells) {}
    ~PrefixTree() { clear(); }

    // Physical pages of the longest chain of complete pages whose tokens equal the head of
    // tokens[0..n).  `touch` refreshes the chain's last-use stamps.
    void match(const int32_t* tokens, int64_t n, bool touch, std::vector<int32_t>& pages_out);
    // List the complete pages of tokens[0..n), stored in `row` (the block-table row of the
    // sequence that computed them).  Pages of prefixes already listed stay as they are (the
    // first publisher wins); new nodes retain their page.  Returns the number of new nodes,
    // or -1 with `err` set.
    int32_t insert(const int32_t* tokens, int64_t n, const int32_t* row, int32_t row_pages,
                   std::string& err);
    // Drop least-recently-used unpinned leaves whose page only the tree still holds, until
    // `want` pages went back to the free queue or nothing evictable is left.
    int32_t evict(int32_t want);
    // Pin (delta = +1) or unpin (-1) the listed chain of tokens[0..n); returns pages affected.
    int32_t pin(const int32_t* tokens, int64_t n, int delta);
    void clear();

    int32_t nodes() const { return n_nodes_; }
    int32_t pinned_nodes() const;
    int32_t evictable_pages() const;  // pages only the tree holds, in unpinned subtrees' leaves upward

private:
    struct Node {
        std::vector<int32_t> key;  // the page's tokens
        int32_t page = -1;
        Node* parent = nullptr;
        uint64_t last_use = 0;
        int32_t pins = 0;
        std::map<std::vector<int32_t>, std::unique_ptr<Node>> children;
    };
    Node* child_of(Node* n, const int32_t* tokens) const;
    void collect_leaves(Node* n, std::vector<Node*>& out);
    void count(const Node* n, int32_t& pinned, int32_t& evictable) const;
    void release_subtree(Node* n);

    PageAllocator* alloc_;
    int32_t page_cells_;
    Node root_;
    uint64_t clock_ = 0;
    int32_t n_nodes_ = 0;
};

}  // namespace bkv
