// Prefix tree over whole pages.  See prefix_tree.hpp for provenance.
#include "prefix_tree.hpp"

#include <algorithm>

namespace bkv {

PrefixTree::Node* PrefixTree::child_of(Node* n, const int32_t* tokens) const {
    const std::vector<int32_t> key(tokens, tokens + page_cells_);
    const auto it = n->children.find(key);
    return it == n->children.end() ? nullptr : it->second.get();
}

void PrefixTree::match(const int32_t* tokens, int64_t n, bool touch, std::vector<int32_t>& pages_out) {
    pages_out.clear();
    Node* at = &root_;
    if (touch) ++clock_;
    for (int64_t t = 0; t + page_cells_ <= n; t += page_cells_) {
        Node* next = child_of(at, tokens + t);
        if (!next) break;
        if (touch) next->last_use = clock_;
        pages_out.push_back(next->page);
        at = next;
    }
}

int32_t PrefixTree::insert(const int32_t* tokens, int64_t n, const int32_t* row, int32_t row_pages,
                           std::string& err) {
    Node* at = &root_;
    int32_t added = 0;
    ++clock_;
    for (int64_t t = 0, c = 0; t + page_cells_ <= n; t += page_cells_, ++c) {
        Node* next = child_of(at, tokens + t);
        if (!next) {
            if (c >= row_pages || row[c] < 0) {
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
            ++n_nodes_;
            ++added;
        }
        next->last_use = clock_;
        at = next;
    }
    return added;
}

void PrefixTree::collect_leaves(Node* n, std::vector<Node*>& out) {
    for (auto& kv : n->children) {
        Node* c = kv.second.get();
        if (c->children.empty())
            out.push_back(c);
        else
            collect_leaves(c, out);
    }
}

int32_t PrefixTree::evict(int32_t want) {
    int32_t freed = 0;
    std::string err;
    // least recently used first; a parent becomes a candidate once its last child is gone
    const auto older = [](const Node* a, const Node* b) { return a->last_use > b->last_use; };
    std::vector<Node*> heap;
    collect_leaves(&root_, heap);
    heap.erase(std::remove_if(heap.begin(), heap.end(),
                              [this](Node* x) { return x->pins > 0 || alloc_->refcount(x->page) != 1; }),
               heap.end());
    std::make_heap(heap.begin(), heap.end(), older);
    while (freed < want && !heap.empty()) {
        std::pop_heap(heap.begin(), heap.end(), older);
        Node* victim = heap.back();
        heap.pop_back();
        Node* parent = victim->parent;
        alloc_->release_page(victim->page, err);
        ++freed;
        --n_nodes_;
        parent->children.erase(victim->key);
        if (parent != &root_ && parent->children.empty() && parent->pins == 0 &&
            alloc_->refcount(parent->page) == 1) {
            heap.push_back(parent);
            std::push_heap(heap.begin(), heap.end(), older);
        }
    }
    return freed;
}

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

void PrefixTree::release_subtree(Node* n) {
    std::string err;
    for (auto& kv : n->children) {
        release_subtree(kv.second.get());
        alloc_->release_page(kv.second->page, err);
    }
    n->children.clear();
}

void PrefixTree::clear() {
    release_subtree(&root_);
    n_nodes_ = 0;
}

void PrefixTree::count(const Node* n, int32_t& pinned, int32_t& evictable) const {
    for (const auto& kv : n->children) {
        const Node* c = kv.second.get();
        if (c->pins > 0) ++pinned;
        if (c->pins == 0 && alloc_->refcount(c->page) == 1) ++evictable;
        count(c, pinned, evictable);
    }
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

}  // namespace bkv
