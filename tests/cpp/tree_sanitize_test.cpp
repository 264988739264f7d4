// Randomised exercise of the host-side page allocator and the tiered prefix tree, meant to be
// built with -fsanitize=address,undefined: the tree juggles raw node pointers in per-call heaps
// while it drops subtrees, which is exactly what a sanitizer is for.  After every operation the
// allocator's and the tree's own invariant checks must hold.  Prints "ok" and exits 0.
#include <cstdio>
#include <cstdlib>
#include <random>
#include <string>
#include <vector>

#include "../../breccia_amd/csrc/allocator.hpp"
#include "../../breccia_amd/csrc/prefix_tree.hpp"

using namespace bkv;

static void must(bool ok, const char* what, const std::string& err = "") {
    if (!ok) {
        std::fprintf(stderr, "FAILED: %s %s\n", what, err.c_str());
        std::exit(1);
    }
}

int main(int argc, char** argv) {
    const unsigned seed = argc > 1 ? (unsigned)std::atoi(argv[1]) : 1u;
    const int steps = argc > 2 ? std::atoi(argv[2]) : 4000;
    std::mt19937 rng(seed);
    const auto pick = [&](int lo, int hi) { return lo + (int)(rng() % (unsigned)(hi - lo + 1)); };

    const int kPages = 64, kCells = 16, kSeqs = 8, kPerSeq = 24;
    PageAllocator alloc(kPages, kCells, kSeqs, kPerSeq);
    PrefixTree tree(&alloc, kCells);
    tree.set_tiers(10, 14);

    // prompts that share heads, so that chains branch
    std::vector<std::vector<int32_t>> prompts;
    for (int i = 0; i < 7; ++i) {
        std::vector<int32_t> p;
        const int head = i % 3;
        for (int t = 0; t < 16 * 5; ++t) p.push_back(1000 * head + t);
        const int tail = 16 * pick(1, 12) + pick(0, 15);
        for (int t = 0; t < tail; ++t) p.push_back(100000 * (i + 1) + t);
        prompts.push_back(p);
    }
    struct Live {
        int32_t seq;
        int prompt;
    };
    std::vector<Live> live;
    std::string err;
    uint64_t moves_seen = 0;
    for (int step = 0; step < steps; ++step) {
        const int op = pick(0, 7);
        std::vector<TierMove> moves;
        if (op <= 1 && live.size() < 5) {
            // a request: match, promote what lives below, adopt, reserve the rest, publish
            const int pi = pick(0, (int)prompts.size() - 1);
            const std::vector<int32_t>& pr = prompts[(size_t)pi];
            std::vector<PrefixTree::Node*> chain;
            tree.match_nodes(pr.data(), (int64_t)pr.size(), true, chain);
            if ((int)chain.size() > kPerSeq) chain.resize(kPerSeq);
            int lower = 0;
            for (const PrefixTree::Node* x : chain) lower += PrefixTree::tier_of(x) != Tier::Device;
            if (lower > 0) {
                tree.pin_nodes(chain, +1);
                const int missing = lower - alloc.free_pages();
                if (missing > 0) tree.evict(missing, &moves);
                tree.promote(chain, lower, moves);
                tree.pin_nodes(chain, -1);
            }
            std::vector<int32_t> pages;
            for (const PrefixTree::Node* x : chain) {
                if (PrefixTree::tier_of(x) != Tier::Device) break;
                pages.push_back(PrefixTree::page_of(x));
            }
            int32_t s = -1;
            if (alloc.seq_create_shared(pages.data(), (int32_t)pages.size(), &s, err) == AllocErr::Ok) {
                PagePair cow[4];
                int32_t n_cow = 0;
                AllocErr e = alloc.seq_reserve(s, (int64_t)pr.size(), cow, 4, &n_cow, err);
                if (e == AllocErr::NoPages) {
                    const int64_t grow = ((int64_t)pr.size() - alloc.seq_len(s) + kCells - 1) / kCells + 1;
                    if (tree.evict((int32_t)(grow - alloc.free_pages()), &moves) > 0)
                        e = alloc.seq_reserve(s, (int64_t)pr.size(), cow, 4, &n_cow, err);
                }
                if (e == AllocErr::Ok) {
                    if (pick(0, 3) != 0)
                        must(tree.insert(pr.data(), (int64_t)pr.size(), alloc.seq_table(s), alloc.seq_n_pages(s), err) >= 0,
                             "insert", err);
                    live.push_back(Live{s, pi});
                } else {
                    alloc.seq_free(s, err);
                }
            }
        } else if (op == 2 && !live.empty()) {
            const size_t i = (size_t)pick(0, (int)live.size() - 1);
            must(alloc.seq_free(live[i].seq, err) == AllocErr::Ok, "seq_free", err);
            live.erase(live.begin() + (long)i);
        } else if (op == 3) {
            tree.evict(pick(0, 9), &moves);
        } else if (op == 4) {
            tree.evict(pick(0, 5), nullptr);  // plain drop, tiers or not
        } else if (op == 5) {
            const std::vector<int32_t>& pr = prompts[(size_t)pick(0, (int)prompts.size() - 1)];
            tree.pin(pr.data(), 16 * pick(1, 6), pick(0, 1) ? +1 : -1);
        } else if (op == 6 && step % 211 == 0) {
            tree.set_tiers(pick(0, 12), pick(0, 16));
        } else if (op == 7 && step % 503 == 0) {
            tree.drop_lower_tiers();
        }
        // every reported move names places inside the arenas
        for (const TierMove& m : moves) {
            must(m.page >= -1 && m.page < kPages && m.host_slot >= -1 && m.disk_slot >= -1, "move fields");
            ++moves_seen;
        }
        must(alloc.check(err), "allocator check", err);
        must(tree.check(err), "tree check", err);
    }
    for (const Live& l : live) alloc.seq_free(l.seq, err);
    tree.clear();
    must(alloc.free_pages() == kPages, "every page is free at the end");
    const TierStats& st = tree.stats();
    must(st.to_host > 0 && st.to_disk > 0 && st.promoted > 0 && st.dropped > 0 && moves_seen > 0, "every path was taken");
    std::printf("ok %llu moves, %llu to host, %llu to disk, %llu promoted, %llu dropped\n", (unsigned long long)moves_seen,
                (unsigned long long)st.to_host, (unsigned long long)st.to_disk, (unsigned long long)st.promoted,
                (unsigned long long)st.dropped);
    return 0;
}
