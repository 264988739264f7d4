"""Pins the oracle's pool addressing, append and gather (CPU only).

Independent statement of the layout: a pool is the C-ordered array
[page][kv head][cell in page][head dim] -- numpy's own stride arithmetic, not the
oracle's index formula -- and the stored half is numpy's float16 cast (inputs here
are far from the two ranges where the cache rule deviates from IEEE)."""
import json
import os

import numpy as np

import oracle
from helpers import np_cache_f16

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_kats.json")))
G = oracle.Geom(2, 256, 16)


def test_size_identities_of_the_reference():
    # crates/breccia-kernels/src/qsa/mod.rs:2028-2048, :2127-2134
    s = GOLD["sizes"]
    assert oracle.row_bytes(G, oracle.LAYOUT_F16, "k") == s["f16_row_words"] * 4
    assert oracle.row_bytes(G, oracle.LAYOUT_Q8V, "v") == s["q8v_row_words"] * 4
    assert oracle.row_bytes(G, oracle.LAYOUT_Q8V, "k") == s["f16_row_words"] * 4
    for pages in (1, 8, 128, 2048):
        assert G.rows(pages) == pages * s["pool_rows_per_page"]
    img = oracle.PoolImage(G, 1)
    assert img.page_bytes("k") + img.page_bytes("v") == s["page_bytes_k_plus_v"]
    assert oracle.row_bytes(G, oracle.LAYOUT_I8H, "k") == 272  # 34 B per 32 values


def test_reference_layout_recipe_33_cells():
    # crates/breccia-kernels/tests/attn_conformance.rs:1172-1275
    r = GOLD["layout_recipe"]
    pages = (r["capacity_cells"] + 15) // 16
    img = oracle.PoolImage(G, pages)
    table = np.arange(pages, dtype=np.int32)  # the reference's identity page table
    dim = 512
    i = np.arange(dim)
    expect_k = np.zeros((pages * 16, dim), dtype=np.float32)
    expect_v = np.zeros((pages * 16, dim), dtype=np.float32)
    for t in range(r["n_tokens"]):
        cell = r["start_cell"] + t
        k = (np.sin((cell * 97 + i * 13).astype(np.float32) * np.float32(0.017)) * np.float32(3.0)).astype(np.float32)
        v = (np.cos((cell * 61 + i * 7).astype(np.float32) * np.float32(0.031)) * np.float32(2.0)).astype(np.float32)
        expect_k[cell], expect_v[cell] = k, v
        assert img.append(table, cell, k, v, capacity_cells=pages * 16) == 0
    kp = img.k.view(np.uint16).reshape(pages, 2, 16, 256)
    vp = img.v.view(np.uint16).reshape(pages, 2, 16, 256)
    checked = 0
    for cell in range(r["start_cell"], r["start_cell"] + r["n_tokens"]):
        for kvh in range(2):
            want_k = expect_k[cell, kvh * 256:(kvh + 1) * 256].astype(np.float16).view(np.uint16)
            want_v = expect_v[cell, kvh * 256:(kvh + 1) * 256].astype(np.float16).view(np.uint16)
            assert np.array_equal(kp[cell // 16, kvh, cell % 16], want_k)
            assert np.array_equal(vp[cell // 16, kvh, cell % 16], want_v)
            checked += 256  # one per (cell, kv head, d): K and V are checked together
    assert checked == r["elements_checked"]
    # cells outside 5..37 were never written
    touched = np.zeros((pages, 2, 16), dtype=bool)
    for cell in range(r["start_cell"], r["start_cell"] + r["n_tokens"]):
        touched[cell // 16, :, cell % 16] = True
    assert not kp[~touched].any() and not vp[~touched].any()
    # word packing: even element in the low half (attn_conformance.rs:1221-1227)
    words = img.k.view(np.uint32)
    e = oracle.elem_index(G, 0, 1, 7, 10)
    assert words[e // 2] & 0xFFFF == kp[0, 1, 7, 10] and words[e // 2] >> 16 == kp[0, 1, 7, 11]


def test_append_past_capacity_is_refused():
    # crates/breccia-kernels/src/qsa/mod.rs:1108-1116
    img = oracle.PoolImage(G, 3)
    z = np.zeros((2, 512), dtype=np.float32)
    assert img.append(np.arange(3), 47, z, z, capacity_cells=48) == -1
    assert img.append(np.arange(3), 46, z, z, capacity_cells=48) == 0


def _random_case(layout, seed, n_pages=24, T=150, pos0=7):
    rng = np.random.Generator(np.random.PCG64(seed))
    img = oracle.PoolImage(G, n_pages, layout)
    table = rng.permutation(n_pages).astype(np.int32)[: (pos0 + T + 15) // 16]
    k = rng.standard_normal((T, 2, 256)).astype(np.float32)
    v = rng.standard_normal((T, 2, 256)).astype(np.float32)
    return rng, img, table, k, v, pos0, T


def test_permuted_append_then_gather_round_trip_f16():
    rng, img, table, k, v, pos0, T = _random_case(oracle.LAYOUT_F16, 21)
    before_k = img.k.copy()
    assert img.append(table, pos0, k, v) == 0
    gk, gv = img.gather(table, pos0, T)
    assert np.array_equal(gk, np_cache_f16(k))
    assert np.array_equal(gv, np_cache_f16(v))
    # bytes of rows that were not appended are unchanged (still zero)
    rows = np.zeros((img.n_pages, 2, 16), dtype=bool)
    for c in range(pos0, pos0 + T):
        rows[table[c // 16], :, c % 16] = True
    k4 = img.k.view(np.uint16).reshape(img.n_pages, 2, 16, 256)
    assert not k4[~rows].any() and before_k.sum() == 0
    # append(T) == T x append(1), byte for byte
    img2 = oracle.PoolImage(G, img.n_pages)
    for t in range(T):
        assert img2.append(table, pos0 + t, k[t], v[t]) == 0
    assert np.array_equal(img.k, img2.k) and np.array_equal(img.v, img2.v)


def test_q8v_layout_words_and_round_trip():
    rng, img, table, k, v, pos0, T = _random_case(oracle.LAYOUT_Q8V, 22, T=40)
    assert img.append(table, pos0, k, v) == 0
    gk, gv = img.gather(table, pos0, T)
    assert np.array_equal(gk, np_cache_f16(k))
    deq, q, sc = oracle.to_q8_0(v.reshape(-1))
    assert np.array_equal(gv.reshape(-1), deq)
    # word layout of one block, stated from the shader comment
    # (crates/breccia-kernels/shaders/qsa_kv_append.comp:38-44): [f32 scale][8 x 4 packed i8]
    cell, kvh, blk = pos0 + 3, 1, 5
    row = (int(table[cell // 16]) * 2 + kvh) * 16 + cell % 16
    w = img.v.view(np.uint32)[(row * 8 + blk) * 9:(row * 8 + blk) * 9 + 9]
    src = v[3, kvh, blk * 32:(blk + 1) * 32]
    _, qb, sb = oracle.to_q8_0(src)
    assert w[0] == sb.view(np.uint32)[0]
    packed = w[1:].view(np.int8)  # little-endian: element j in byte j%4 of word 1+j/4
    assert np.array_equal(packed, qb)


def test_i8h_layout_and_round_trip():
    rng, img, table, k, v, pos0, T = _random_case(oracle.LAYOUT_I8H, 23, T=40)
    assert img.append(table, pos0, k, v) == 0
    gk, gv = img.gather(table, pos0, T)
    dk, qk, sk = oracle.to_i8h(k.reshape(-1))
    dv, qv, sv = oracle.to_i8h(v.reshape(-1))
    assert np.array_equal(gk.reshape(-1), dk) and np.array_equal(gv.reshape(-1), dv)
    cell, kvh = pos0 + 9, 0
    row = (int(table[cell // 16]) * 2 + kvh) * 16 + cell % 16
    rowb = img.k[row * 272:(row + 1) * 272]
    assert np.array_equal(rowb[:256].view(np.int8), qk.reshape(T, 2, 256)[9, kvh])
    assert np.array_equal(rowb[256:].view(np.uint16), sk.reshape(T, 2, 8)[9, kvh])


def test_page_copy_and_swap_are_byte_moves():
    rng, img, table, k, v, pos0, T = _random_case(oracle.LAYOUT_F16, 24)
    img.append(table, pos0, k, v)
    before = img.k.copy()
    free = [p for p in range(img.n_pages) if p not in set(table.tolist())]
    pairs = [(int(table[0]), free[0]), (int(table[3]), free[1])]
    img.page_copy(pairs)
    pb = img.page_bytes("k")
    for s, d in pairs:
        assert np.array_equal(img.k[d * pb:(d + 1) * pb], before[s * pb:(s + 1) * pb])
        assert np.array_equal(img.k[s * pb:(s + 1) * pb], before[s * pb:(s + 1) * pb])
    untouched = np.ones(img.n_pages, dtype=bool)
    untouched[[d for _, d in pairs]] = False
    assert np.array_equal(img.k.reshape(img.n_pages, pb)[untouched], before.reshape(img.n_pages, pb)[untouched])
