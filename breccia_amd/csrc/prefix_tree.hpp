// Host-side prefix tree over whole pages: which physical pages already hold the K/V of a
// given token prefix, so that a new request adopts them instead of recomputing (no HIP here).
//
// The reference has no such structure; the shape follows its design notes for the planned
// subsystem (docs/reference-engines/02-kv-and-context.md:543-548 "hash granularity of 16
// tokens so prefix hits are page-aligned", :566-581 tier movement rules, :600-603
// "radix/: TreeNode{refcount, last_access, priority}, eviction as a strategy, read-only
// pinned subtree", :594-597 "pool/: device.rs T1 VRAM pages, host.rs T2 pinned, hard byte cap,
// disk.rs T3 NVMe"): a trie with one node per complete page, keyed by that page's tokens;
// the tree holds one reference on every device page it lists; eviction takes least-recently-
// used nodes that nobody else holds; pinned chains (injected read-only context) are never
// evicted.
//
// Tiers.  A node's page lives in exactly one place (:568-569): a device page, a slot of the
// pinned-host arena, or a slot of the file on disk.  Without lower tiers an evicted page is
// dropped.  With them it is demoted: device -> host slot; when the arena is full its least
// recently used node goes host -> disk first, and when the file is full its least recently
// used leaf is dropped.  Demotion works upwards from the leaves, so along any chain the tiers
// only ever go down (device ... host ... disk), and a request that matches a chain brings its
// lower part back page by page (promotion) before it adopts it.  The tree only does the
// bookkeeping: every change of place is reported as a TierMove, in the order the bytes must
// move, and the caller that owns the device moves them.
#pragma once

#include <cstdint>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "allocator.hpp"

namespace bkv {

enum class Tier : uint8_t { Device = 0, Host = 1, Disk = 2 };

struct TierMove {
    enum Kind { DeviceToHost, HostToDisk, HostToDevice, DiskToDevice } kind;
    int32_t page;       // device page read or written, -1 when the move has none
    int32_t host_slot;  // -1 when the move has none
    int32_t disk_slot;  // -1 when the move has none
};

// Slot numbers of a fixed-size arena; the lowest free slot is handed out first.
class SlotArena {
public:
    void resize(int32_t n);
    int32_t take();  // -1 when every slot is taken
    void give(int32_t slot);
    int32_t capacity() const { return n_; }
    int32_t used() const { return n_ - (int32_t)free_.size(); }

private:
    int32_t n_ = 0;
    std::vector<int32_t> free_;  // a min-heap
};

struct TierStats {
    int32_t nodes[3] = {0, 0, 0};  // by tier
    uint64_t to_host = 0, to_disk = 0, promoted = 0, dropped = 0;
};

class PrefixTree {
public:
    struct Node;

    PrefixTree(PageAllocator* alloc, int32_t page_cells) : alloc_(alloc), page_cells_(page_cells) {}
    ~PrefixTree() { clear(); }

    // Capacities of the lower tiers in pages; 0 = no such tier.  Nodes that live in a lower tier
    // now are dropped first.
    void set_tiers(int32_t host_slots, int32_t disk_slots);
    bool tiered() const { return host_.capacity() > 0; }

    // The longest chain of complete pages whose tokens equal the head of tokens[0..n), in any
    // tier.  `touch` refreshes the chain's last-use stamps.
    void match_nodes(const int32_t* tokens, int64_t n, bool touch, std::vector<Node*>& chain);
    // The device pages of the leading part of that chain that is on the device.
    void match(const int32_t* tokens, int64_t n, bool touch, std::vector<int32_t>& pages_out);
    static Tier tier_of(const Node* n);
    static int32_t page_of(const Node* n);
    // List the complete pages of tokens[0..n), stored in `row` (the block-table row of the
    // sequence that computed them).  Pages of prefixes already listed stay as they are (the
    // first publisher wins), except that a node in a lower tier takes the sequence's device
    // page and gives its slot back; new nodes retain their page.  Returns the number of new
    // nodes, or -1 with `err` set.
    int32_t insert(const int32_t* tokens, int64_t n, const int32_t* row, int32_t row_pages,
                   std::string& err);
    // Free device pages: least-recently-used unpinned device nodes that only the tree holds and
    // that have no child on the device, until `want` pages went back to the free queue or
    // nothing evictable is left.  With lower tiers and `moves` given the pages are demoted
    // (their moves appended), otherwise dropped.
    int32_t evict(int32_t want, std::vector<TierMove>* moves = nullptr);
    // Bring the first `limit` lower-tier nodes of `chain` (in chain order) back to fresh device
    // pages; stops early when the free queue is empty.  Returns how many came back.
    int32_t promote(const std::vector<Node*>& chain, int32_t limit, std::vector<TierMove>& moves);
    // Pin (delta = +1) or unpin (-1) the listed chain of tokens[0..n); returns pages affected.
    int32_t pin(const int32_t* tokens, int64_t n, int delta);
    void pin_nodes(const std::vector<Node*>& chain, int delta);
    // Forget every node that is not on the device (after an I/O failure, or before the tiers change).
    void drop_lower_tiers();
    void clear();

    int32_t nodes() const { return stats_.nodes[0] + stats_.nodes[1] + stats_.nodes[2]; }
    const TierStats& stats() const { return stats_; }
    int32_t pinned_nodes() const;
    int32_t evictable_pages() const;  // device pages only the tree holds, unpinned
    // Every node's place is consistent with the arenas' and the allocator's books.
    bool check(std::string& err) const;

    struct Node {
        std::vector<int32_t> key;  // the page's tokens
        Tier tier = Tier::Device;
        int32_t page = -1;  // device page (Tier::Device)
        int32_t slot = -1;  // arena or file slot (lower tiers)
        Node* parent = nullptr;
        uint64_t last_use = 0;
        int32_t pins = 0;
        std::map<std::vector<int32_t>, std::unique_ptr<Node>> children;
    };

private:
    Node* child_of(Node* n, const int32_t* tokens) const;
    bool has_child_in(const Node* n, Tier t) const;
    bool device_candidate(const Node* n) const;
    void collect_device_candidates(Node* n, std::vector<Node*>& out);
    template <typename F>
    void walk(Node* from, F f) const;
    struct LowerQueues {
        bool built = false;
        std::vector<Node*> host, disk;  // heaps, least recently used on top
        void build(PrefixTree& t);
        static void push(std::vector<Node*>& heap, Node* n);
        static Node* pop(std::vector<Node*>& heap);
    };
    bool host_candidate(const Node* c) const;
    bool make_host_room(std::vector<TierMove>& moves, LowerQueues& q);
    void drop_subtree(Node* n);  // n and everything below it; n is erased from its parent
    void release_place(Node* n);
    void count(const Node* n, int32_t& pinned, int32_t& evictable) const;
    void release_children(Node* n);

    PageAllocator* alloc_;
    int32_t page_cells_;
    Node root_;
    uint64_t clock_ = 0;
    SlotArena host_, disk_;
    TierStats stats_;
};

}  // namespace bkv
