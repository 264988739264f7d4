"""Host-side checks that need no GPU: the library loads and exports every entry point the
header declares, every range/size violation is an error return (never a launch), and the
page allocator keeps its invariants.  Pools here are created host-only."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from breccia_amd import kv, lib as L
from breccia_amd.kv import BkvError, Pool

HEADER = os.path.join(os.path.dirname(__file__), "..", "include", "breccia_kv.h")
BENCH_HEADER = os.path.join(os.path.dirname(__file__), "..", "include", "breccia_kv_bench.h")


def declared_functions(header=HEADER):
    text = open(header).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(bkv_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = declared_functions()
    assert len(names) >= 45
    for name in names:
        assert hasattr(L._product, name), "libbreccia_kv.so does not export " + name
    # and the Python binding covers each of them
    assert sorted(L._SIGNATURES) == names


def test_the_product_library_carries_no_probe_or_plumbing_entry_point():
    # device allocation, copies, streams, events, graphs and the bandwidth probes live in
    # libbreccia_kv_bench.so (include/breccia_kv_bench.h): what an integration links has the path only
    bench = declared_functions(BENCH_HEADER)
    assert "bkv_copy_probe" in bench and "bkv_dev_alloc" in bench and "bkv_graph_launch" in bench
    assert sorted(L._BENCH_SIGNATURES) == bench
    for name in bench:
        assert hasattr(L._bench, name), "libbreccia_kv_bench.so does not export " + name
        assert not hasattr(L._product, name), "libbreccia_kv.so still exports " + name
    assert not set(bench) & set(declared_functions())


def test_wait_options_round_trip_and_reject_a_zero_deadline():
    # crates/breccia-vk/src/ctx.rs:1545-1553: the reference's waits have a 10 s deadline; so have these
    assert kv.wait_options() == (10000, 4000)
    assert kv.wait_options(timeout_ms=250, poll_us=0) == (250, 0)
    assert kv.wait_options(timeout_ms=-1) == (-1, 0)
    expect(L.ERR_INVALID, kv.wait_options, 0, 100)
    expect(L.ERR_INVALID, kv.wait_options, 100, -5)
    assert kv.wait_options(10000, 4000) == (10000, 4000)


def test_rust_binding_text_lists_every_declaration_with_its_argument_count():
    """The Rust `extern "C"` block a maintainer would add (kept with the drop-in notes at the repository
    root; source only, no Rust toolchain here) names every function of the header with as many arguments
    as the header gives it."""
    doc = open(os.path.join(os.path.dirname(__file__), "..", "INTEGRATION.md")).read()
    rust = dict((m.group(1), m.group(2)) for m in re.finditer(r"pub fn (bkv_[a-z0-9_]+)\(([^;]*?)\)(?: -> [^;]+)?;", doc, re.S))
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    header = dict((m.group(1), m.group(2)) for m in re.finditer(r"\b(bkv_[a-z0-9_]+)\s*\(([^;{}]*?)\);", text, re.S))
    assert sorted(header) == declared_functions()
    assert sorted(rust) == sorted(header)
    for name, args in header.items():
        n_c = 0 if args.strip() in ("", "void") else args.count(",") + 1
        n_rust = 0 if not rust[name].strip() else rust[name].count(":")
        assert n_c == n_rust, (name, n_c, n_rust)


def test_header_structs_match_the_binding():
    text = open(HEADER).read()
    body = re.search(r"typedef struct bkv_pool_desc \{(.*?)\} bkv_pool_desc;", text, re.S).group(1)
    fields = re.findall(r"(?:int32_t|uint32_t)\s+(\w+);", body)
    assert fields == [f[0] for f in L.PoolDesc._fields_]
    assert C.sizeof(L.PagePair) == 8
    assert int(re.search(r"#define BKV_MAX_BATCH (\d+)", text).group(1)) == L.MAX_BATCH


def host_pool(**kw):
    kw.setdefault("host_only", True)
    return Pool(**kw)


def expect(status, fn, *a, **k):
    with pytest.raises(BkvError) as ei:
        fn(*a, **k)
    assert ei.value.status == status, ei.value
    assert ei.value.message, "an error must carry a message"
    return ei.value.message


def test_invalid_geometry_is_refused():
    # crates/breccia-kernels/src/qsa/mod.rs:405-409: a state needs capacity > 0
    expect(L.ERR_INVALID, host_pool, n_pages=0)
    expect(L.ERR_INVALID, host_pool, n_layers=0)
    expect(L.ERR_INVALID, host_pool, head_dim=100)
    expect(L.ERR_INVALID, host_pool, head_dim=512)
    expect(L.ERR_INVALID, host_pool, page_cells=4)
    expect(L.ERR_INVALID, host_pool, layout=7)
    expect(L.ERR_INVALID, host_pool, max_seqs=0)


def test_sizes_follow_the_reference_layouts():
    # crates/breccia-kernels/src/qsa/mod.rs:237-240, :316-370
    with host_pool(n_layers=12, n_pages=8) as p:
        assert p.page_bytes(0) == 16384 and p.page_bytes(1) == 16384
        assert p.swap_page_bytes() == 12 * 32768
    with host_pool(n_pages=2048, layout=L.LAYOUT_Q8V) as p:
        assert p.page_bytes(0) == 16384 and p.page_bytes(1) == 32 * 288
        assert p.page_bytes(1) / p.page_bytes(0) == 0.5625
    with host_pool(layout=L.LAYOUT_I8H) as p:
        assert p.page_bytes(0) == p.page_bytes(1) == 32 * 272


def test_device_calls_on_a_host_only_pool_fail_cleanly():
    with host_pool() as p:
        s = p.seq_create()
        p.seq_reserve(s, 20)
        z = C.c_void_p(0x1000)
        expect(L.ERR_NO_DEVICE, p.append, 0, [s], [0], [1], z, z)
        expect(L.ERR_NO_DEVICE, p.decode_attn, 0, [s], [5], 16, z, z, 0.0625)
        expect(L.ERR_NO_DEVICE, p.page_copy, [(0, 1)])
        expect(L.ERR_NO_DEVICE, p.fill, 0xFF)


def test_append_and_attention_range_checks_come_before_any_launch():
    # crates/breccia-kernels/src/qsa/mod.rs:1108-1116 (append past capacity is an Err)
    with host_pool(n_pages=8, max_seqs=4) as p:
        s = p.seq_create()
        p.seq_reserve(s, 40)  # 3 pages = 48 addressable cells
        z = C.c_void_p(0x1000)
        msg = expect(L.ERR_RANGE, p.append, 0, [s], [47], [2], z, z)
        assert "47..49" in msg and "48" in msg
        expect(L.ERR_RANGE, p.append, 0, [s], [-1], [1], z, z)
        expect(L.ERR_RANGE, p.append, 0, [s], [0], [-1], z, z)
        expect(L.ERR_RANGE, p.append, 1, [s], [0], [1], z, z)        # layer
        expect(L.ERR_RANGE, p.append, 0, [3], [0], [1], z, z)        # dead sequence
        expect(L.ERR_RANGE, p.decode_attn, 0, [s], [48], 16, z, z, 0.0625)
        expect(L.ERR_RANGE, p.decode_attn, 0, [s], [-1], 16, z, z, 0.0625)
        expect(L.ERR_INVALID, p.decode_attn, 0, [s], [5], 15, z, z, 0.0625)   # 15 q heads / 2 kv
        expect(L.ERR_INVALID, p.decode_attn, 0, [s] * 65, [5] * 65, 16, z, z, 0.0625)
        expect(L.ERR_RANGE, p.page_copy, [(0, 8)])
        expect(L.ERR_INVALID, p.page_copy, [(0, 1), (2, 1)])
        expect(L.ERR_RANGE, lambda: kv.check(L.lib.bkv_gather(p.handle, 0, s, 40, 9, z, z, None)))


def test_allocator_basic_growth_and_free():
    with host_pool(n_pages=10, max_seqs=3, max_pages_per_seq=6) as p:
        a = p.seq_create()
        assert p.seq_reserve(a, 1) == [] and p.seq_n_pages(a) == 1 and p.seq_len(a) == 1
        assert p.seq_reserve(a, 16) == [] and p.seq_n_pages(a) == 1
        assert p.seq_reserve(a, 17) == [] and p.seq_n_pages(a) == 2
        assert p.free_pages() == 8 and p.seq_capacity(a) == 32
        p.check()
        expect(L.ERR_RANGE, p.seq_reserve, a, 16 * 6 + 1)      # longer than a table row
        expect(L.ERR_RANGE, p.seq_reserve, a, 5)               # shrinking is truncate's job
        b = p.seq_create()
        p.seq_reserve(b, 16 * 6)
        c = p.seq_create()
        msg = expect(L.ERR_NO_PAGES, p.seq_reserve, c, 16 * 3)  # only 2 pages left
        assert "2 free" in msg
        assert p.seq_len(c) == 0 and p.seq_n_pages(c) == 0 and p.free_pages() == 2  # unchanged
        expect(L.ERR_NO_PAGES, p.seq_create)                    # all 3 slots live
        p.seq_free(b)
        assert p.free_pages() == 8
        expect(L.ERR_STATE, p.seq_free, b)                      # double free
        p.check()
        tab = p.block_table(a)
        assert len(set(tab.tolist())) == 2 and all(p.page_refcount(int(x)) == 1 for x in tab)


def test_fork_shares_pages_and_cow_fires_only_on_a_shared_partial_page():
    with host_pool(n_pages=64, max_seqs=8, max_pages_per_seq=16) as p:
        root = p.seq_create()
        p.seq_reserve(root, 40)                 # 2 full pages + 8 cells of a third
        kids = [p.seq_fork(root, 40) for _ in range(3)]
        tab = p.block_table(root)
        assert all(p.page_refcount(int(x)) == 4 for x in tab)
        for k in kids:
            assert np.array_equal(p.block_table(k), tab) and p.seq_len(k) == 40
        p.check()
        # first writer: copies the shared partial page, leaves the full pages shared
        pairs = p.seq_reserve(kids[0], 41)
        assert pairs == [(int(tab[2]), int(p.block_table(kids[0])[2]))]
        assert pairs[0][1] != pairs[0][0] and p.page_refcount(int(tab[2])) == 3
        assert np.array_equal(p.block_table(kids[0])[:2], tab[:2])
        # others likewise; the last holder writes in place (refcount is back to 1)
        assert len(p.seq_reserve(kids[1], 50)) == 1
        assert len(p.seq_reserve(kids[2], 41)) == 1
        assert p.page_refcount(int(tab[2])) == 1
        assert p.seq_reserve(root, 41) == []
        assert p.block_table(root)[2] == tab[2]
        p.check()
        # a fork at a page boundary never copies: appends start on a fresh page
        edge = p.seq_fork(root, 32)
        assert p.seq_reserve(edge, 33) == []
        assert p.block_table(edge)[2] not in (tab[2],)
        # the report buffer being too small is an error and changes nothing
        k4 = p.seq_fork(kids[1], 50)
        free_before = p.free_pages()
        expect(L.ERR_INVALID, p.seq_reserve, k4, 51, 0)
        assert p.free_pages() == free_before and p.seq_len(k4) == 50
        for s in kids + [root, edge, k4]:
            p.seq_free(s)
        assert p.free_pages() == 64
        p.check()


def test_truncate_then_regrow_does_not_write_into_shared_pages():
    with host_pool(n_pages=32, max_seqs=4, max_pages_per_seq=8) as p:
        a = p.seq_create()
        p.seq_reserve(a, 64)
        b = p.seq_fork(a, 64)
        p.seq_truncate(b, 20)                       # speculative rollback keeps the pages
        assert p.seq_n_pages(b) == 4 and p.seq_len(b) == 20
        pairs = p.seq_reserve(b, 50)                # rewrites cells 20..49: pages 1, 2, 3
        tb, ta = p.block_table(b), p.block_table(a)
        assert tb[0] == ta[0]                       # untouched page stays shared
        assert pairs == [(int(ta[1]), int(tb[1]))]  # partial page is copied
        assert tb[2] != ta[2] and tb[3] != ta[3]    # fully rewritten pages are fresh, no copy
        expect(L.ERR_RANGE, p.seq_truncate, b, 51)
        p.check()


def test_identity_sequence_is_the_reference_page_table():
    # crates/breccia-kernels/src/qsa/mod.rs:477-481
    with host_pool(n_pages=8, max_seqs=2) as p:
        s = p.seq_create_identity(3)
        assert p.block_table(s).tolist() == [0, 1, 2] and p.seq_capacity(s) == 48
        assert p.free_pages() == 5
        expect(L.ERR_STATE, p.seq_create_identity, 2)
        p.check()


def test_evict_restore_bookkeeping():
    with host_pool(n_pages=16, max_seqs=4, max_pages_per_seq=8) as p:
        a = p.seq_create()
        p.seq_reserve(a, 70)                        # 4 full pages + 6 cells
        host = C.c_void_p(0x1000)                   # never dereferenced by a host-only pool
        expect(L.ERR_STATE, lambda: kv.check(L.lib.bkv_seq_evict(p.handle, a, 3, 2, host, None)))
        b = p.seq_fork(a, 16)
        expect(L.ERR_STATE, lambda: kv.check(L.lib.bkv_seq_evict(p.handle, a, 0, 1, host, None)))
        p.seq_free(b)
        kv.check(L.lib.bkv_seq_evict(p.handle, a, 1, 2, host, None))
        assert p.block_table(a).tolist()[1:3] == [-1, -1] and p.free_pages() == 13
        z = C.c_void_p(0x1000)
        expect(L.ERR_STATE, p.decode_attn, 0, [a], [69], 16, z, z, 0.0625)
        expect(L.ERR_STATE, p.append, 0, [a], [20], [1], z, z)
        expect(L.ERR_STATE, lambda: kv.check(L.lib.bkv_seq_restore(p.handle, a, 0, 1, host, None)))
        kv.check(L.lib.bkv_seq_restore(p.handle, a, 1, 2, host, None))
        assert all(x >= 0 for x in p.block_table(a)) and p.free_pages() == 11
        p.check()


def test_randomised_allocator_keeps_its_invariants():
    rng = np.random.Generator(np.random.PCG64(2))
    with host_pool(n_pages=48, max_seqs=12, max_pages_per_seq=12) as p:
        live = {}
        for step in range(600):
            op = rng.integers(0, 5)
            try:
                if op == 0 or not live:
                    s = p.seq_create()
                    live[s] = 0
                elif op == 1:
                    s = int(rng.choice(list(live)))
                    new_len = live[s] + int(rng.integers(1, 40))
                    p.seq_reserve(s, new_len, cow_capacity=4)
                    live[s] = new_len
                elif op == 2:
                    s = int(rng.choice(list(live)))
                    n = int(rng.integers(0, live[s] + 1))
                    c = p.seq_fork(s, n)
                    live[c] = n
                elif op == 3:
                    s = int(rng.choice(list(live)))
                    p.seq_free(s)
                    del live[s]
                else:
                    s = int(rng.choice(list(live)))
                    n = int(rng.integers(0, live[s] + 1))
                    p.seq_truncate(s, n)
                    live[s] = n
            except BkvError as e:
                assert e.status in (L.ERR_NO_PAGES, L.ERR_RANGE), e
            p.check()
            for s, n in live.items():
                assert p.seq_len(s) == n
        total_refs = sum(p.page_refcount(i) for i in range(48))
        entries = sum(int((p.block_table(s) >= 0).sum()) for s in live)
        assert total_refs == entries
        for s in list(live):
            p.seq_free(s)
        assert p.free_pages() == 48


def test_rope_table_is_the_reference_formula():
    # crates/breccia-kernels/src/ops/mod.rs:2504-2522 (bit for bit against the formula) and
    # the errors of RopeTable::build (odd n_rot, empty table)
    import oracle
    from breccia_amd.kv import rope_table

    for base, n_rot, max_pos in [(1e7, 64, 8), (1e7, 64, 300), (1e4, 128, 17), (5e5, 2, 3)]:
        got = rope_table(base, n_rot, max_pos)
        assert np.array_equal(got.view(np.uint32), oracle.rope_table(base, n_rot, max_pos).view(np.uint32))
    for bad in [(1e7, 63, 8), (1e7, 64, 0), (1e7, 0, 8)]:
        with pytest.raises(BkvError) as ei:
            rope_table(*bad)
        assert ei.value.status == L.ERR_INVALID


def test_attention_planning_terminates_and_fits_for_every_batch_shape():
    """The cut of a batch into work-groups must come back for every shape the calls accept (a batch
    whose one-range-per-entry cut already exceeds what is resident at once used to spin on the
    host), cover every page, and fit the partial-result workspace -- or be refused as a size
    error before anything is enqueued (crates/breccia-kernels/src/qsa/mod.rs:1108-1116)."""
    rng = np.random.Generator(np.random.PCG64(77))
    checked = 0
    for n_cu in (256, 64, 8):
        for n_kv in range(1, L.MAX_KV_HEAD + 1):
            for group in range(1, 17):
                # a work-group writes `group` head rows of a workspace that holds 4096 x 8
                cap = 4096 * 8 // group if group > 8 else 4096
                for n in (1, 2, 7, 33, 64):
                    for sel_groups in (0, 129):
                        pos = rng.integers(0, 40000, size=n)
                        if n >= 33:
                            pos[: n // 2] = rng.integers(0, 64, size=n // 2)   # many one-page entries
                        assert n * n_kv <= cap    # 64 entries x 16 kv heads always fit
                        splits, pps, total = kv.attn_plan(n_cu, n_kv, n_kv * group, pos, sel_groups)
                        pages = np.full(n, sel_groups) if sel_groups else pos // 16 + 1
                        assert total == int(splits.sum()) * n_kv <= cap
                        assert np.all(pps % 4 == 0) and np.all(splits >= 1)
                        assert np.all(splits * pps >= pages) and np.all((splits - 1) * pps < pages)
                        # one generation (two work-groups per compute unit) whenever one is possible at all
                        assert total <= max(2 * n_cu, n * n_kv)
                        checked += 1
    assert checked > 5000


def test_attention_batches_larger_than_one_generation_are_planned_not_spun_on():
    with host_pool(n_pages=64, n_kv_head=16, max_seqs=64, max_pages_per_seq=2) as p:
        seqs = [p.seq_create() for _ in range(64)]
        for s in seqs:
            p.seq_reserve(s, 4)
        z = C.c_void_p(0)
        # 64 entries x 16 kv heads of 13 q heads each = 1024 work-groups: accepted as a plan (and then
        # refused for lack of a device); one more kv head cannot exist
        expect(L.ERR_NO_DEVICE, p.decode_attn, 0, seqs, [3] * 64, 16 * 13, z, z, 0.0625)
    expect(L.ERR_INVALID, host_pool, n_kv_head=L.MAX_KV_HEAD + 1)
    expect(L.ERR_INVALID, kv.attn_plan, 256, L.MAX_KV_HEAD + 1, 17, [5], 0)
    # the largest accepted shapes are planned as one range per entry, in more than one generation
    splits, pps, total = kv.attn_plan(256, 16, 16 * 16, [5] * 64, 0)
    assert total == 1024 and np.all(splits == 1)
    splits, pps, total = kv.attn_plan(256, 9, 9, [70000] * 64, 0)      # 576 > 512 resident: used to spin
    assert total == 576 and np.all(splits == 1) and np.all(pps >= 70000 // 16 + 1)


def test_writes_need_reserved_cells_on_pages_the_sequence_holds_alone():
    """bkv_append / bkv_append_kprep / bkv_decode_step write only cells that bkv_seq_reserve has
    made the sequence's own: past the reserved length is a range error, a page another holder
    still shares is a state error (the copy-on-write pair was never asked for), and nothing
    changes -- tables, lengths and refcounts stay as they were."""
    with host_pool(n_pages=32, max_seqs=4, max_pages_per_seq=8) as p:
        z = C.c_void_p(0)
        parent = p.seq_create()
        p.seq_reserve(parent, 40)                      # pages 0, 1 full, page 2 half full
        child = p.seq_fork(parent, 40)
        before = (p.block_table(parent).tolist(), p.block_table(child).tolist(), p.free_pages())
        shared = int(p.block_table(child)[2])
        assert p.page_refcount(shared) == 2
        # the child appends at its length without a reserve: capacity (48) would allow it
        msg = expect(L.ERR_RANGE, p.append, 0, [child], [40], [1], z, z)
        assert "reserve" in msg
        expect(L.ERR_RANGE, p.decode_step, 0, [child], [40], z, z, 16, z, z, 0.0625)
        # rewriting cells it does hold, on a page the parent still shares
        msg = expect(L.ERR_STATE, p.append, 0, [child], [33], [2], z, z)
        assert "holders" in msg
        expect(L.ERR_STATE, p.append, 0, [parent], [0], [40], z, z)
        expect(L.ERR_STATE, p.decode_step, 0, [parent], [39], z, z, 16, z, z, 0.0625)
        assert (p.block_table(parent).tolist(), p.block_table(child).tolist(), p.free_pages()) == before
        assert p.seq_len(child) == 40 and p.seq_len(parent) == 40 and p.page_refcount(shared) == 2
        p.check()
        # with the reserve the child gets its own copy of the half page; both may then write
        pairs = p.seq_reserve(child, 41)
        assert pairs == [(shared, int(p.block_table(child)[2]))] and p.page_refcount(shared) == 1
        expect(L.ERR_NO_DEVICE, p.append, 0, [child], [40], [1], z, z)       # passes every host check
        p.seq_reserve(parent, 41)                                            # sole holder again: in place
        expect(L.ERR_NO_DEVICE, p.append, 0, [parent], [40], [1], z, z)
        expect(L.ERR_NO_DEVICE, p.decode_step, 0, [parent], [40], z, z, 16, z, z, 0.0625)
        # a page a cached prefix lists is shared too
        p.prefix_insert(parent, np.arange(32))
        expect(L.ERR_STATE, p.append, 0, [parent], [16], [4], z, z)
        p.check()


def test_step_plan_checks_come_before_any_device_work():
    """bkv_step_plan_create validates like bkv_decode_step, for every cell of the horizon, on the host:
    a host-only pool gets as far as the device check and no further."""
    import ctypes as C
    from breccia_amd.kv import StepPlan

    with host_pool(n_pages=16, max_seqs=4) as pool:
        s = pool.seq_create()
        pool.seq_reserve(s, 30)
        for kw, status in ((dict(seqs=[s], pos=[25], horizon=6), L.ERR_RANGE),      # cell 30 is not reserved
                           (dict(seqs=[s, s], pos=[1, 2], horizon=2), L.ERR_INVALID),
                           (dict(seqs=[7], pos=[0], horizon=1), L.ERR_RANGE),
                           (dict(seqs=[s], pos=[0], horizon=0), L.ERR_INVALID),
                           (dict(seqs=[s], pos=[0], horizon=4, n_q=17), L.ERR_INVALID),
                           (dict(seqs=[s], pos=[20], horizon=10), L.ERR_NO_DEVICE)):  # valid: stops at the device
            with pytest.raises(BkvError) as ei:
                StepPlan(pool, kw["seqs"], kw["pos"], kw["horizon"], kw.get("n_q", 16))
            assert ei.value.status == status, (kw, ei.value)
        child = pool.seq_fork(s, 20)
        with pytest.raises(BkvError) as ei:       # the page of cells 16..31 is shared now
            StepPlan(pool, [s], [20], 5, 16)
        assert ei.value.status == L.ERR_STATE
        pool.seq_free(child)
        for fn in ("bkv_step_plan_destroy",):
            assert getattr(L.lib, fn)(None) == L.ERR_INVALID
        assert L.lib.bkv_step_plan_decode(None, 0, None, None, None, None, 0, 0, C.c_float(1.0), None, None) == L.ERR_INVALID
        assert L.lib.bkv_step_plan_advance(None, None) == L.ERR_INVALID
        assert L.lib.bkv_graph_begin_capture(None) == L.ERR_INVALID
