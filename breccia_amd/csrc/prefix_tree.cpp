// Prefix tree over whole pages, with lower tiers.  See prefix_tree.hpp for provenance.
#include "prefix_tree.hpp"

#include <algorithm>
#include <functional>

namespace bkv {

// ---- slot arena -------------------------------------------------------------------------------
void SlotArena::resize(int32_t n) {
    n_ = n < 0 ? 0 : n;
    free_.resize((size_t)n_);
    for (int32_t i = 0; i < n_; ++i) free_[(size_t)i] = i;
    std::make_heap(free_.begin(), free_.end(), std::greater<int32_t>());
}

int32_t SlotArena::take() {
    if (free_.empty()) return -1;
    std::pop_heap(free_.begin(), free_.end(), std::greater<int32_t>());
    const int32_t s = free_.back();
    free_.pop_back();
    return s;
}

void SlotArena::give(int32_t slot) {
    free_.push_back(slot);
    std::push_heap(free_.begin(), free_.end(), std::greater<int32_t>());
}

// ---- lookups ----------------------------------------------------------------------------------
Tier PrefixTree::tier_of(const Node* n) { return n->tier; }
int32_t PrefixTree::page_of(const Node* n) { return n->page; }

PrefixTree::Node* PrefixTree::child_of(Node* n, const int32_t* tokens) const {
    const std::vector<int32_t> key(tokens, tokens + page_cells_);
    const auto it = n->children.find(key);
    return it == n->children.end() ? nullptr : it->second.get();
}

void PrefixTree::match_nodes(const int32_t* tokens, int64_t n, bool touch, std::vector<Node*>& chain) {
    chain.clear();
    Node* at = &root_;
    if (touch) ++clock_;
    for (int64_t t = 0; t + page_cells_ <= n; t += page_cells_) {
        Node* next = child_of(at, tokens + t);
        if (!next) break;
        if (touch) next->last_use = clock_;
        chain.push_back(next);
        at = next;
    }
}

void PrefixTree::match(const int32_t* tokens, int64_t n, bool touch, std::vector<int32_t>& pages_out) {
    std::vector<Node*> chain;
    match_nodes(tokens, n, touch, chain);
    pages_out.clear();
    for (const Node* x : chain) {
        if (x->tier != Tier::Device) break;
        pages_out.push_back(x->page);
    }
}

// ---- insertion --------------------------------------------------------------------------------
int32_t PrefixTree::insert(const int32_t* tokens, int64_t n, const int32_t* row, int32_t row_pages,
                           std::string& err) {
    Node* at = &root_;
    int32_t added = 0;
    ++clock_;
    for (int64_t t = 0, c = 0; t + page_cells_ <= n; t += page_cells_, ++c) {
        Node* next = child_of(at, tokens + t);
        const bool have_page = c < row_pages && row[c] >= 0;
        // tiers only go down along a chain: nothing new is listed on the device below a node
        // that stays in a lower tier
        const bool below_lower = at != &root_ && at->tier != Tier::Device;
        if (!next) {
            if (below_lower) break;
            if (!have_page) {
                err = "prefix insert: page " + std::to_string(c) + " of the sequence is not resident";
                return -1;
            }
            if (alloc_->retain_page(row[c], err) != AllocErr::Ok) return -1;
            auto node = std::make_unique<Node>();
            node->key.assign(tokens + t, tokens + t + page_cells_);
            node->page = row[c];
            node->parent = at;
            next = node.get();
            at->children.emplace(node->key, std::move(node));
            ++stats_.nodes[0];
            ++added;
        } else if (next->tier != Tier::Device && have_page && !below_lower) {
            // the sequence has recomputed a page the tree only holds in a lower tier: its device
            // copy takes the node's place, which costs no transfer
            if (alloc_->retain_page(row[c], err) != AllocErr::Ok) return -1;
            release_place(next);
            next->tier = Tier::Device;
            next->page = row[c];
            ++stats_.nodes[0];
        }
        next->last_use = clock_;
        at = next;
    }
    return added;
}

// ---- places -----------------------------------------------------------------------------------
// Give back whatever holds the node's page and take the node out of its tier's count.
void PrefixTree::release_place(Node* n) {
    std::string err;
    switch (n->tier) {
        case Tier::Device: alloc_->release_page(n->page, err); break;
        case Tier::Host: host_.give(n->slot); break;
        case Tier::Disk: disk_.give(n->slot); break;
    }
    --stats_.nodes[(int)n->tier];
    n->page = -1;
    n->slot = -1;
}

// Chains are as deep as a sequence is long (one node per page), so nothing here recurses: the
// nodes below n are listed parents first and then released, and destroyed, from the far end.
void PrefixTree::release_children(Node* n) {
    std::vector<Node*> below;
    walk(n, [&](Node* c) {
        below.push_back(c);
        return true;
    });
    for (size_t i = below.size(); i-- > 0;) {
        release_place(below[i]);
        below[i]->children.clear();  // its own children are gone already
    }
    n->children.clear();
}

void PrefixTree::drop_subtree(Node* n) {
    int32_t before = nodes();
    release_children(n);
    release_place(n);
    stats_.dropped += (uint64_t)(before - nodes());
    Node* parent = n->parent;
    parent->children.erase(n->key);  // destroys n
}

bool PrefixTree::has_child_in(const Node* n, Tier t) const {
    for (const auto& kv : n->children)
        if (kv.second->tier == t) return true;
    return false;
}

// ---- eviction ---------------------------------------------------------------------------------
bool PrefixTree::device_candidate(const Node* n) const {
    return n->tier == Tier::Device && n->pins == 0 && alloc_->refcount(n->page) == 1 &&
           !has_child_in(n, Tier::Device);
}

// f(node) for every node below `from`, parents before children; f returns whether to go below
// the node it was given.
template <typename F>
void PrefixTree::walk(Node* from, F f) const {
    std::vector<Node*> stack;
    for (auto& kv : from->children) stack.push_back(kv.second.get());
    while (!stack.empty()) {
        Node* c = stack.back();
        stack.pop_back();
        if (!f(c)) continue;
        for (auto& kv : c->children) stack.push_back(kv.second.get());
    }
}

void PrefixTree::collect_device_candidates(Node* n, std::vector<Node*>& out) {
    walk(n, [&](Node* c) {
        if (c->tier != Tier::Device) return false;  // nothing on the device below a lower tier
        if (device_candidate(c)) out.push_back(c);
        return true;
    });
}

// Least-recently-used first.
static bool newer(const PrefixTree::Node* a, const PrefixTree::Node* b) { return a->last_use > b->last_use; }

bool PrefixTree::host_candidate(const Node* c) const {
    return c->tier == Tier::Host && c->pins == 0 && !has_child_in(c, Tier::Host);
}
static bool disk_leaf(const PrefixTree::Node* c) {
    return c->tier == Tier::Disk && c->pins == 0 && c->children.empty();
}

// The lower tiers' candidates of one evict() call, each list built by one walk when it is first
// needed and kept up to date after that: a node only ever becomes a candidate during the call
// (its last host child left, it arrived without one), and leaves the lists when it is taken.
void PrefixTree::LowerQueues::build(PrefixTree& t) {
    host.clear();
    disk.clear();
    t.walk(&t.root_, [&](Node* c) {
        if (t.host_candidate(c)) host.push_back(c);
        if (disk_leaf(c)) disk.push_back(c);
        return true;
    });
    std::make_heap(host.begin(), host.end(), newer);
    std::make_heap(disk.begin(), disk.end(), newer);
    built = true;
}
void PrefixTree::LowerQueues::push(std::vector<Node*>& heap, Node* n) {
    heap.push_back(n);
    std::push_heap(heap.begin(), heap.end(), newer);
}
PrefixTree::Node* PrefixTree::LowerQueues::pop(std::vector<Node*>& heap) {
    if (heap.empty()) return nullptr;
    std::pop_heap(heap.begin(), heap.end(), newer);
    Node* n = heap.back();
    heap.pop_back();
    return n;
}

// One free slot in the host arena: its least recently used node without a host child goes to
// the file (whose own least recently used leaf is dropped when it is full), or is dropped with
// what hangs below it when there is no file to take it.
bool PrefixTree::make_host_room(std::vector<TierMove>& moves, LowerQueues& q) {
    if (!q.built) q.build(*this);
    Node* h = q.pop(q.host);
    if (!h) return false;
    Node* parent = h->parent;
    bool moved = false;
    if (disk_.capacity() > 0) {
        int32_t d = disk_.take();
        if (d < 0) {
            if (Node* leaf = q.pop(q.disk)) {
                Node* lp = leaf->parent;
                drop_subtree(leaf);
                if (lp != &root_ && disk_leaf(lp)) q.push(q.disk, lp);
                d = disk_.take();
            }
        }
        if (d >= 0) {
            moves.push_back(TierMove{TierMove::HostToDisk, -1, h->slot, d});
            host_.give(h->slot);
            --stats_.nodes[(int)Tier::Host];
            ++stats_.nodes[(int)Tier::Disk];
            ++stats_.to_disk;
            h->tier = Tier::Disk;
            h->slot = d;
            if (disk_leaf(h)) q.push(q.disk, h);
            moved = true;
        }
    }
    if (!moved) {
        // what hangs below h may sit in the lists: they are rebuilt when next needed
        if (!h->children.empty()) q.built = false;
        drop_subtree(h);
    }
    if (q.built && parent != &root_ && host_candidate(parent)) q.push(q.host, parent);
    return true;
}

int32_t PrefixTree::evict(int32_t want, std::vector<TierMove>* moves) {
    int32_t freed = 0;
    const bool demote = moves != nullptr && tiered();
    // least recently used first; a parent becomes a candidate once it has no child on the device
    const auto older = [](const Node* a, const Node* b) { return a->last_use > b->last_use; };
    std::vector<Node*> heap;
    collect_device_candidates(&root_, heap);
    std::make_heap(heap.begin(), heap.end(), older);
    LowerQueues lower;
    while (freed < want && !heap.empty()) {
        std::pop_heap(heap.begin(), heap.end(), older);
        Node* victim = heap.back();
        heap.pop_back();
        Node* parent = victim->parent;
        int32_t slot = -1;
        if (demote) {
            slot = host_.take();
            if (slot < 0 && make_host_room(*moves, lower)) slot = host_.take();
        }
        if (slot >= 0) {
            std::string err;
            moves->push_back(TierMove{TierMove::DeviceToHost, victim->page, slot, -1});
            alloc_->release_page(victim->page, err);
            --stats_.nodes[(int)Tier::Device];
            ++stats_.nodes[(int)Tier::Host];
            ++stats_.to_host;
            victim->tier = Tier::Host;
            victim->page = -1;
            victim->slot = slot;
            if (lower.built && host_candidate(victim)) lower.push(lower.host, victim);
        } else {
            if (!victim->children.empty()) lower.built = false;
            drop_subtree(victim);
        }
        ++freed;
        if (parent != &root_ && device_candidate(parent)) {
            heap.push_back(parent);
            std::push_heap(heap.begin(), heap.end(), older);
        }
    }
    return freed;
}

// ---- promotion --------------------------------------------------------------------------------
int32_t PrefixTree::promote(const std::vector<Node*>& chain, int32_t limit, std::vector<TierMove>& moves) {
    int32_t done = 0;
    std::string err;
    for (Node* x : chain) {
        if (x->tier == Tier::Device) continue;
        if (done == limit) break;
        int32_t page = -1;
        if (alloc_->retain_fresh_page(&page, err) != AllocErr::Ok) break;
        if (x->tier == Tier::Host) {
            moves.push_back(TierMove{TierMove::HostToDevice, page, x->slot, -1});
            host_.give(x->slot);
        } else {
            moves.push_back(TierMove{TierMove::DiskToDevice, page, -1, x->slot});
            disk_.give(x->slot);
        }
        --stats_.nodes[(int)x->tier];
        ++stats_.nodes[(int)Tier::Device];
        ++stats_.promoted;
        x->tier = Tier::Device;
        x->page = page;
        x->slot = -1;
        ++done;
    }
    return done;
}

// ---- pins -------------------------------------------------------------------------------------
int32_t PrefixTree::pin(const int32_t* tokens, int64_t n, int delta) {
    Node* at = &root_;
    int32_t touched = 0;
    for (int64_t t = 0; t + page_cells_ <= n; t += page_cells_) {
        Node* next = child_of(at, tokens + t);
        if (!next) break;
        if (delta > 0 || next->pins > 0) {
            next->pins += delta > 0 ? 1 : -1;
            ++touched;
        }
        at = next;
    }
    return touched;
}

void PrefixTree::pin_nodes(const std::vector<Node*>& chain, int delta) {
    for (Node* x : chain) x->pins += delta;
}

// ---- wholesale --------------------------------------------------------------------------------
void PrefixTree::drop_lower_tiers() {
    // tiers only go down along a chain: a lower-tier node's whole subtree goes with it
    std::vector<Node*> tops;
    walk(&root_, [&](Node* c) {
        if (c->tier == Tier::Device) return true;
        tops.push_back(c);
        return false;
    });
    for (Node* t : tops) drop_subtree(t);
}

void PrefixTree::set_tiers(int32_t host_slots, int32_t disk_slots) {
    drop_lower_tiers();
    host_.resize(host_slots);
    disk_.resize(host_slots > 0 ? disk_slots : 0);
}

void PrefixTree::clear() {
    release_children(&root_);
    stats_.nodes[0] = stats_.nodes[1] = stats_.nodes[2] = 0;
}

// ---- counts and checks ------------------------------------------------------------------------
void PrefixTree::count(const Node* n, int32_t& pinned, int32_t& evictable) const {
    walk(const_cast<Node*>(n), [&](Node* c) {
        if (c->pins > 0) ++pinned;
        if (c->tier == Tier::Device && c->pins == 0 && alloc_->refcount(c->page) == 1) ++evictable;
        return true;
    });
}

int32_t PrefixTree::pinned_nodes() const {
    int32_t p = 0, e = 0;
    count(&root_, p, e);
    return p;
}

int32_t PrefixTree::evictable_pages() const {
    int32_t p = 0, e = 0;
    count(&root_, p, e);
    return e;
}

bool PrefixTree::check(std::string& err) const {
    std::vector<int> host_seen((size_t)host_.capacity(), 0), disk_seen((size_t)disk_.capacity(), 0);
    int32_t by_tier[3] = {0, 0, 0};
    bool ok = true;
    walk(const_cast<Node*>(&root_), [&](Node* c) {
        if (!ok) return false;
        ++by_tier[(int)c->tier];
        if (c->parent != &root_ && (int)c->tier < (int)c->parent->tier) {
            err = "prefix tree: a node sits in a higher tier than its parent";
            ok = false;
        } else if (c->tier == Tier::Device) {
            if (c->page < 0 || c->page >= alloc_->n_pages() || alloc_->external_refs(c->page) < 1) {
                err = "prefix tree: a device node's page holds no reference of the tree";
                ok = false;
            }
        } else {
            std::vector<int>& seen = c->tier == Tier::Host ? host_seen : disk_seen;
            if (c->slot < 0 || c->slot >= (int32_t)seen.size() || seen[(size_t)c->slot]++) {
                err = "prefix tree: a lower-tier slot is out of range or listed twice";
                ok = false;
            }
        }
        return ok;
    });
    if (!ok) return false;
    for (int t = 0; t < 3; ++t)
        if (by_tier[t] != stats_.nodes[t]) {
            err = "prefix tree: the per-tier node counts are off";
            return false;
        }
    if (by_tier[1] != host_.used() || by_tier[2] != disk_.used()) {
        err = "prefix tree: slots in use and nodes in the lower tiers disagree";
        return false;
    }
    return true;
}

}  // namespace bkv
