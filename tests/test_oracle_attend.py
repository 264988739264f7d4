"""Pins the oracle's attention (crates/breccia-kernels/src/qsa/cpu.rs:197-246) against a
library routine (torch float64 scaled_dot_product_attention on the CPU), an independent
numpy softmax, and closed forms chosen so that a dropped scale, a wrong head->kv-head
map, a transposed operand or a missing causal test each fail at least one of them."""
import numpy as np

import oracle
from helpers import max_abs


def _case(seed, n_cells, n_head, n_kv, hd=256):
    rng = np.random.Generator(np.random.PCG64(seed))
    q = rng.standard_normal((n_head, hd)).astype(np.float32)
    k = oracle.to_f16(rng.standard_normal((n_cells, n_kv, hd)).astype(np.float32))
    v = oracle.to_f16(rng.standard_normal((n_cells, n_kv, hd)).astype(np.float32))
    gate = rng.standard_normal((n_head, hd)).astype(np.float32)
    return q, k, v, gate


def _numpy_attend(q, k, v, pos, n_head, n_kv, gate=None):
    q64, k64, v64 = q.astype(np.float64), k.astype(np.float64), v.astype(np.float64)
    hd = q.shape[1]
    out = np.zeros((n_head, hd))
    for h in range(n_head):
        kvh = h // (n_head // n_kv)
        logits = k64[: pos + 1, kvh] @ q64[h] / np.sqrt(hd)
        w = np.exp(logits - logits.max())
        w /= w.sum()
        out[h] = w @ v64[: pos + 1, kvh]
    if gate is not None:
        out = out / (1.0 + np.exp(-gate.astype(np.float64)))
    return out


def test_dense_attend_matches_torch_sdpa_float64():
    import torch  # CPU only; imported here so GPU test processes never load torch's HIP runtime

    for n_head, n_kv, n_cells, pos in ((16, 2, 300, 299), (24, 2, 130, 100), (4, 4, 33, 32)):
        q, k, v, gate = _case(100 + n_head, n_cells, n_head, n_kv)
        got = oracle.attend(q, k, v, oracle.dense_cells(pos), pos, n_head, n_kv, 256)
        group = n_head // n_kv
        tq = torch.from_numpy(q.astype(np.float64))[None, :, None, :]           # [1, H, 1, D]
        tk = torch.from_numpy(k[: pos + 1].astype(np.float64)).permute(1, 0, 2)  # [KV, C, D]
        tv = torch.from_numpy(v[: pos + 1].astype(np.float64)).permute(1, 0, 2)
        tk = tk.repeat_interleave(group, dim=0)[None]
        tv = tv.repeat_interleave(group, dim=0)[None]
        want = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv)[0, :, 0, :].numpy()
        assert max_abs(got, want) < 3e-7  # f32 rounding of the output only


def test_dense_attend_matches_numpy_with_gate():
    q, k, v, gate = _case(7, 513, 16, 2)
    pos = 500
    got = oracle.attend(q, k, v, oracle.dense_cells(pos), pos, 16, 2, 256, gate=gate)
    want = _numpy_attend(q, k, v, pos, 16, 2, gate)
    assert max_abs(got, want) < 3e-7
    # threads > 1 is the same arithmetic per head
    got_mt = oracle.attend(q, k, v, oracle.dense_cells(pos), pos, 16, 2, 256, gate=gate, threads=4)
    assert np.array_equal(got, got_mt)


def test_dense_selection_is_cells_0_to_pos():
    # crates/breccia-kernels/shaders/qsa_topk.comp:78-95 with the causal test of attend
    for pos in (0, 1, 3, 4, 6, 37, 2061):
        cells = oracle.dense_cells(pos)
        live = cells[cells <= pos]
        assert np.array_equal(live, np.arange(pos + 1, dtype=np.uint32))
        assert cells.max() < pos + 4
    assert list(oracle.dense_ids(9, 10)) == [0, 1, 2]       # blocks 0,1 complete + own tail block 2
    assert list(oracle.dense_ids(7, 8)) == [0, 1]
    assert list(oracle.cells_of([0, 5, 9, 15])) == [0, 1, 2, 3, 20, 21, 22, 23, 36, 37, 38, 39, 60, 61, 62, 63]


def test_closed_forms():
    n_head, n_kv, hd = 16, 2, 256
    q, k, v, gate = _case(3, 64, n_head, n_kv)
    sig = 1.0 / (1.0 + np.exp(-gate.astype(np.float64)))
    # one live cell: out = v * sigmoid(gate), whatever q and k are
    out = oracle.attend(q, k, v, [0, 1, 2, 3], 0, n_head, n_kv, hd, gate=gate)
    want = np.repeat(v[0].astype(np.float64), n_head // n_kv, axis=0) * sig
    assert max_abs(out, want) < 3e-7  # the f32 rounding of the output
    # identical K rows: uniform weights -> mean of V (catches a wrong softmax normaliser)
    k_same = np.broadcast_to(k[:1], k.shape).copy()
    out = oracle.attend(q, k_same, v, np.arange(64), 63, n_head, n_kv, hd)
    want = np.repeat(v.astype(np.float64).mean(axis=0), n_head // n_kv, axis=0)
    assert max_abs(out, want) < 3e-7  # the f32 rounding of the output
    # gate = 0 halves the ungated result exactly
    ungated = oracle.attend(q, k, v, np.arange(64), 63, n_head, n_kv, hd)
    halved = oracle.attend(q, k, v, np.arange(64), 63, n_head, n_kv, hd, gate=np.zeros_like(gate))
    assert np.array_equal(halved, (ungated.astype(np.float64) * 0.5).astype(np.float32))
    # cells past pos contribute exactly nothing
    a = oracle.attend(q, k, v, np.arange(64), 40, n_head, n_kv, hd)
    b = oracle.attend(q, k[:41], v[:41], np.arange(41), 40, n_head, n_kv, hd)
    assert np.array_equal(a, b)
    # a cell listed twice counts twice; list order does not matter beyond rounding
    dup = oracle.attend(q, k, v, [5, 9, 9], 63, n_head, n_kv, hd)
    k2, v2 = np.stack([k[5], k[9], k[9]]), np.stack([v[5], v[9], v[9]])
    assert max_abs(dup, oracle.attend(q, k2, v2, [0, 1, 2], 2, n_head, n_kv, hd)) < 3e-7  # the f32 rounding of the output
    perm = np.random.Generator(np.random.PCG64(1)).permutation(64)
    assert max_abs(oracle.attend(q, k, v, perm, 63, n_head, n_kv, hd), ungated) < 1e-6
    # no live cell: zeros
    assert not oracle.attend(q, k, v, [50, 51], 10, n_head, n_kv, hd).any()
    # scale is 1/sqrt(hd): scaling q by 2 must equal halving hd's effect -- check one logit pair
    p = oracle.attend_probs(q, k, np.arange(2), 1, 3, n_head, n_kv, hd)
    kvh = 3 * n_kv // n_head
    l0 = float(q[3].astype(np.float64) @ k[0, kvh].astype(np.float64)) / 16.0
    l1 = float(q[3].astype(np.float64) @ k[1, kvh].astype(np.float64)) / 16.0
    assert abs(p[0] / p[1] - np.exp(l0 - l1)) < 1e-9 * max(1.0, p[0] / p[1])


def test_head_to_kv_head_map_is_contiguous_groups():
    # kvh = h * n_kv / n_head (crates/breccia-kernels/src/qsa/cpu.rs:211): make kv head 1's V
    # distinguishable and check which q heads see it
    n_head, n_kv, hd = 24, 2, 256
    q, k, v, _ = _case(5, 8, n_head, n_kv)
    v[:, 0, :] = 1.0
    v[:, 1, :] = -1.0
    out = oracle.attend(q, k, v, np.arange(8), 7, n_head, n_kv, hd)
    assert np.allclose(out[:12], 1.0) and np.allclose(out[12:], -1.0)


def test_normalish_generator_of_the_reference_tests():
    # crates/breccia-kernels/tests/attn_conformance.rs:110-124, restated with Python integers
    seed, n = 0xF3, 64
    got = oracle.normalish(seed, n)
    s = seed | 1
    for i in range(n):
        acc = np.float32(0.0)
        for _ in range(4):
            s = (s * 6364136223846793005 + 1442695040888963407) % (1 << 64)
            acc = np.float32(acc + np.float32(np.float32(s >> 33) / np.float32(2147483647)))
        want = np.float32(np.float32(acc - np.float32(1.0)) * np.float32(1.732))
        assert got[i] == want
    big = oracle.normalish(0xE3, 1 << 16)
    assert abs(float(big.mean()) - 1.732) < 0.05 and abs(float(big.std()) - 1.0) < 0.05
