"""Pins the oracle's block selection (indexer score, top-k with ties and the own block)
against the reference's known answers, its LCG score recipes and independent numpy
statements.  CPU only."""
import numpy as np
import pytest

import oracle

DEAD = np.float32(-1.0e29)        # crates/breccia-kernels/tests/qsa_topk.rs:25


def lcg_scores(n):
    # crates/breccia-kernels/tests/qsa_topk.rs:90-95
    seed = 0x9E3779B9
    out = np.empty(n, dtype=np.float32)
    for i in range(n):
        seed = (seed * 1664525 + 1013904223) & 0xFFFFFFFF
        out[i] = np.float32(((seed >> 8) & 0xFFFF) / 65536.0)
    return out


def numpy_topk(scores, k, own):
    s = np.asarray(scores, dtype=np.float64)
    idx = np.arange(s.size)
    live = np.isfinite(s)
    order = idx[live][np.lexsort((idx[live], -s[live]))][:k]
    out = list(order)
    if own is not None and own not in out:
        out.append(own)
    return np.asarray(out, dtype=np.uint32)


def test_reference_known_answers():
    # crates/breccia-kernels/src/qsa/cpu.rs:517-536
    s = [1.0, 3.0, 3.0, 2.0]
    assert list(oracle.topk_blocks(s, 2, None)) == [1, 2]
    assert list(oracle.topk_blocks(s, 4, 9)) == [1, 2, 3, 0, 9]
    assert list(oracle.topk_blocks(s, 3, 3)) == [1, 2, 3]
    assert list(oracle.topk_blocks([-np.inf, -np.inf, 1.0], 3, None)) == [2]


@pytest.mark.parametrize("cells", [65536, 65521])
def test_reference_lcg_recipes_against_numpy_lexsort(cells):
    # crates/breccia-kernels/tests/qsa_topk.rs:87-122: distinct, a boundary made of ties, dead
    # blocks interspersed, all equal, own block appended; 512 blocks kept
    n, k = cells // 4, 512
    distinct = lcg_scores(n)
    tied = np.zeros(n, dtype=np.float32)
    tied[:100] = 1.0
    dead = distinct.copy()
    dead[::3] = DEAD
    cases = [("distinct", distinct, 0), ("ties", tied, 0), ("dead", dead, 0),
             ("all-equal", np.full(n, 0.5, dtype=np.float32), 0), ("own", distinct, 4 * (n - 3))]
    for what, sc, pos0 in cases:
        own = pos0 // 4
        got = oracle.topk_blocks(sc, k, own)
        assert np.array_equal(got, numpy_topk(sc, k, own)), what
        assert len(set(got.tolist())) == got.size, what
    # closed forms the recipes were built for
    assert list(oracle.topk_blocks(tied, k, 0)) == list(range(512))          # 100 ones, then zeros by index
    assert list(oracle.topk_blocks(np.full(n, 0.5), k, 0)) == list(range(512))
    got = oracle.topk_blocks(dead, k, 0)
    assert np.all(got[:512] % 3 != 0) and got[-1] == 0                       # dead never chosen; own block 0 appended
    got = oracle.topk_blocks(distinct, k, n - 3)
    assert got.size in (512, 513) and (n - 3) in got


def test_topk_fewer_live_blocks_than_k():
    s = np.array([0.25, -np.inf, 0.75, -np.inf, 0.5])
    assert list(oracle.topk_blocks(s, 512, None)) == [2, 4, 0]
    assert list(oracle.topk_blocks(s, 512, 1)) == [2, 4, 0, 1]
    assert list(oracle.topk_blocks(np.array([]), 512, 0)) == [0]
    assert list(oracle.topk_blocks(np.array([-np.inf]), 4, None)) == []


def test_indexer_score_against_numpy_float64():
    # generator and shapes of crates/breccia-kernels/tests/attn_conformance.rs:908-916
    n_blocks = 515
    q = oracle.normalish(0xE1, 4 * 128).reshape(4, 128)
    pooled = oracle.normalish(0xE2, (n_blocks + 1) * 128).reshape(n_blocks + 1, 128)
    pos = 2061
    got = oracle.indexer_score(q, pooled, n_blocks, pos)
    dots = pooled[:n_blocks].astype(np.float64) @ q.astype(np.float64).T
    want = np.maximum(dots, 0.0).sum(axis=1) / np.sqrt(128.0)
    assert np.max(np.abs(got - want)) < 1e-12
    assert np.all(got >= 0.0)
    # blocks that start after the query are dead (qsa/cpu.rs:107-109): with pos 21 blocks 0..5 live
    early = oracle.indexer_score(q, pooled, n_blocks, 21)
    assert np.all(np.isfinite(early[:6])) and np.all(np.isneginf(early[6:]))
    assert np.array_equal(early[:6], got[:6])
    # relu per head: flipping one head's query removes exactly its positive share
    q2 = q.copy()
    q2[1] = -q2[1]
    got2 = oracle.indexer_score(q2, pooled, n_blocks, pos)
    share = np.maximum(dots[:, 1], 0.0) - np.maximum(-dots[:, 1], 0.0)
    assert np.max(np.abs((got - got2) - share / np.sqrt(128.0))) < 1e-12
    # positive scaling of q scales the scores
    assert np.max(np.abs(oracle.indexer_score(q * 4, pooled, n_blocks, pos) - 4 * got)) < 1e-12


def test_score_then_topk_is_the_reference_selection_at_2062_cells():
    # crates/breccia-kernels/tests/attn_conformance.rs:897-1004: 515 whole blocks, query at 2061,
    # 512 blocks kept, own block 515 (the unpooled tail) appended last
    q = oracle.normalish(0xE1, 4 * 128)
    pooled = oracle.normalish(0xE2, 516 * 128)
    scores = oracle.indexer_score(q, pooled, 515, 2061)
    ids = oracle.topk_blocks(scores, 512, 2061 // 4)
    assert ids.size == 513 and ids[-1] == 515
    assert np.array_equal(ids, numpy_topk(scores, 512, 515))
    assert np.all(np.diff(scores[ids[:512]]) <= 0)
    dropped = np.setdiff1d(np.arange(515), ids[:512])
    assert dropped.size == 3 and scores[dropped].max() <= scores[ids[:512]].min()
