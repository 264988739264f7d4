"""Pins the oracle's K preparation (RMSNorm with gamma, rotary table, partial NEOX rotary)
against the reference's own known answers, independent numpy float64 statements and the
invariants of a rotation.  CPU only."""
import numpy as np
import pytest

import oracle

ULP32 = float(np.finfo(np.float32).eps)


# ---- known answers held by the reference's unit tests -----------------------------------
def test_rmsnorm_of_a_constant_row_is_one():
    # crates/breccia-kernels/src/ops/cpu.rs:373-381
    y = oracle.rmsnorm(np.full(4, 3.0, dtype=np.float32), 4, gamma=None, eps=0.0)
    assert np.all(np.abs(y - 1.0) < 1e-7)


def test_rope_is_the_identity_at_position_zero():
    # crates/breccia-kernels/src/ops/cpu.rs:383-398
    table = oracle.rope_table(1e7, 64, 4)
    x = (np.arange(256) * np.float32(0.01)).astype(np.float32)
    y = oracle.rope_apply(x, 256, 64, table, [0])
    assert np.all(np.abs(x - y) < 1e-6)
    assert np.array_equal(x[64:], y[64:])


def test_rope_is_the_neox_pairing_not_the_adjacent_one():
    # crates/breccia-kernels/src/ops/cpu.rs:400-421: a one-hot at dim 1 rotates into dim 33
    table = oracle.rope_table(1e7, 64, 2)
    x = np.zeros(64, dtype=np.float32)
    x[1] = 1.0
    y = oracle.rope_apply(x, 64, 64, table, [1])
    assert abs(y[1] - table[1, 1, 0]) < 1e-6
    assert abs(y[33] - table[1, 1, 1]) < 1e-6
    assert abs(y[2]) < 1e-9


def test_rope_table_formula_of_the_reference():
    # crates/breccia-kernels/src/ops/mod.rs:2504-2522 states the formula cell by cell; here it
    # is evaluated by numpy's own pow/cos/sin in float64 and by angle identities
    t = oracle.rope_table(1e7, 64, 8)
    assert t.shape == (8, 32, 2)
    p = np.arange(8, dtype=np.float64)[:, None]
    i = np.arange(32, dtype=np.float64)[None, :]
    ang = p * np.power(1e7, -2.0 * i / 64.0)
    assert np.max(np.abs(t[..., 0] - np.cos(ang))) <= ULP32 / 2
    assert np.max(np.abs(t[..., 1] - np.sin(ang))) <= ULP32 / 2
    assert np.mean(t[..., 0] == np.cos(ang).astype(np.float32)) > 0.99
    assert np.array_equal(t[0, :, 0], np.ones(32, dtype=np.float32))
    assert np.array_equal(t[0, :, 1], np.zeros(32, dtype=np.float32))
    # pair 0 turns by exactly p radians; the last pair by p * 1e7^(-31/32)
    assert abs(float(t[3, 0, 0]) - np.cos(3.0)) < 1e-7 and abs(float(t[3, 0, 1]) - np.sin(3.0)) < 1e-7
    assert abs(float(t[5, 31, 1]) - np.sin(5.0 * 1e7 ** (-31.0 / 32.0))) < 1e-9
    # double-angle identity links row 2p to row p
    c, s = t[:4, :, 0].astype(np.float64), t[:4, :, 1].astype(np.float64)
    assert np.max(np.abs(t[0:8:2, :, 0] - (c * c - s * s))) < 3e-7
    assert np.max(np.abs(t[0:8:2, :, 1] - 2 * c * s)) < 3e-7
    assert np.max(np.abs(c * c + s * s - 1.0)) < 2e-7


# ---- independent statements ------------------------------------------------------------
@pytest.mark.parametrize("cols,rows,wgroups", [(256, 48, 1), (128, 8, 1), (2560, 8, 4), (256, 5, 0)])
def test_rmsnorm_against_numpy_float64(cols, rows, wgroups):
    # shapes and generator of crates/breccia-kernels/tests/ops_conformance.rs:140-180
    x = oracle.normalish(0x12345678 ^ cols, rows * cols).reshape(rows, cols)
    g = oracle.normalish(0xFEED, max(wgroups, 1) * cols).reshape(max(wgroups, 1), cols) if wgroups else None
    got = oracle.rmsnorm(x, cols, g, wgroups=wgroups if wgroups else None, eps=1e-6)
    x64 = x.astype(np.float64)
    inv = 1.0 / np.sqrt(np.mean(x64 * x64, axis=1, keepdims=True) + np.float64(np.float32(1e-6)))
    want = x64 * inv
    if wgroups:
        want = want * g.astype(np.float64)[np.arange(rows) % wgroups]
    err = np.abs(got.reshape(rows, cols) - want)
    assert np.all(err <= np.abs(want) * ULP32 * 0.5000001 + 1e-45)   # one f32 rounding of the f64 value
    if not wgroups:
        rms = np.sqrt(np.mean(got.astype(np.float64).reshape(rows, cols) ** 2, axis=1))
        assert np.max(np.abs(rms - 1.0)) < 1e-5


def test_rmsnorm_invariants():
    rng = np.random.Generator(np.random.PCG64(5))
    x = rng.standard_normal((6, 256)).astype(np.float32)
    g = rng.standard_normal(256).astype(np.float32)
    y = oracle.rmsnorm(x, 256, g, eps=0.0)
    # positive rescaling of a row by a power of two leaves the result bit-identical
    assert np.array_equal(y, oracle.rmsnorm(x * np.float32(8.0), 256, g, eps=0.0))
    # a sign flip of the row flips the result; gamma enters as a plain factor
    assert np.array_equal(-y, oracle.rmsnorm(-x, 256, g, eps=0.0))
    y1 = oracle.rmsnorm(x, 256, np.ones(256, dtype=np.float32), eps=0.0)
    assert np.max(np.abs(y - y1.astype(np.float64) * g)) < 1e-6
    # eps matters exactly where the row is tiny: a zero row stays zero, no NaN
    z = oracle.rmsnorm(np.zeros((1, 256), dtype=np.float32), 256, g, eps=1e-6)
    assert np.array_equal(z, np.zeros((1, 256), dtype=np.float32))
    # row r takes gamma slice r % wgroups
    g3 = rng.standard_normal((3, 256)).astype(np.float32)
    y3 = oracle.rmsnorm(x, 256, g3, wgroups=3, eps=1e-6)
    for r in range(6):
        assert np.array_equal(y3[r], oracle.rmsnorm(x[r], 256, g3[r % 3], eps=1e-6).reshape(-1))


@pytest.mark.parametrize("head_dim,n_rot,heads,tokens", [(256, 64, 24, 1), (256, 64, 2, 1), (256, 64, 24, 3),
                                                         (128, 64, 4, 2), (128, 64, 1, 5), (64, 64, 4, 2)])
def test_rope_against_complex_multiplication(head_dim, n_rot, heads, tokens):
    # cases, generator and positions of crates/breccia-kernels/tests/ops_conformance.rs:186-206
    table = oracle.rope_table(1e7, 64, 1024)
    rows = heads * tokens
    x = oracle.normalish(0xBEEF ^ head_dim, rows * head_dim).reshape(rows, head_dim)
    positions = np.array([7 + r // heads for r in range(rows)], dtype=np.int32)
    got = oracle.rope_apply(x, head_dim, n_rot, table, positions).reshape(rows, head_dim)
    half = n_rot // 2
    z = x[:, :half].astype(np.float64) + 1j * x[:, half:n_rot].astype(np.float64)
    w = table[positions, :, 0].astype(np.float64) + 1j * table[positions, :, 1].astype(np.float64)
    zz = z * w
    assert np.max(np.abs(got[:, :half] - zz.real)) < 3e-7 * max(1.0, np.max(np.abs(x)))
    assert np.max(np.abs(got[:, half:n_rot] - zz.imag)) < 3e-7 * max(1.0, np.max(np.abs(x)))
    assert np.array_equal(got[:, n_rot:], x[:, n_rot:])           # tail copied, bit for bit
    # a rotation keeps the length of every pair
    n0 = np.hypot(x[:, :half].astype(np.float64), x[:, half:n_rot].astype(np.float64))
    n1 = np.hypot(got[:, :half].astype(np.float64), got[:, half:n_rot].astype(np.float64))
    assert np.max(np.abs(n0 - n1)) < 1e-6


def test_rope_angles_add_and_positions_clamp():
    table = oracle.rope_table(1e7, 64, 64)
    rng = np.random.Generator(np.random.PCG64(8))
    x = rng.standard_normal((4, 256)).astype(np.float32)
    a = oracle.rope_apply(x, 256, 64, table, [5, 5, 5, 5])
    ab = oracle.rope_apply(a, 256, 64, table, [9, 9, 9, 9])
    direct = oracle.rope_apply(x, 256, 64, table, [14, 14, 14, 14])
    assert np.max(np.abs(ab - direct)) < 2e-6
    # and rotating back by the conjugate table undoes it
    conj = table.copy()
    conj[..., 1] = -conj[..., 1]
    back = oracle.rope_apply(a, 256, 64, conj, [5, 5, 5, 5])
    assert np.max(np.abs(back - x)) < 1e-6
    # out-of-range positions read the first / last table row (ops/cpu.rs:141)
    lo = oracle.rope_apply(x, 256, 64, table, [-3, -1, 0, 0])
    assert np.array_equal(lo, oracle.rope_apply(x, 256, 64, table, [0, 0, 0, 0]))
    hi = oracle.rope_apply(x, 256, 64, table, [63, 64, 1000, 2**31 - 1])
    assert np.array_equal(hi, oracle.rope_apply(x, 256, 64, table, [63, 63, 63, 63]))


def test_k_prep_composes_norm_then_rotary_per_kv_head():
    # crates/breccia-kernels/src/qsa/cpu.rs:383-397
    rng = np.random.Generator(np.random.PCG64(21))
    T, n_kv, hd = 5, 2, 256
    k = rng.standard_normal((T, n_kv, hd)).astype(np.float32) * 3
    g = rng.standard_normal(hd).astype(np.float32)
    table = oracle.rope_table(1e7, 64, 128)
    pos = np.array([100, 101, 102, 103, 104])
    got = oracle.k_prep(k, n_kv, hd, g, 1e-6, table, 64, pos)
    for t in range(T):
        for h in range(n_kv):
            n = oracle.rmsnorm(k[t, h], hd, g, eps=1e-6)
            r = oracle.rope_apply(n, hd, 64, table, [pos[t]])
            assert np.array_equal(got[t, h], r.reshape(-1))


def test_pool_keys_mean_then_norm_then_rotary_at_the_first_cell():
    # crates/breccia-kernels/src/qsa/cpu.rs:154-185
    rng = np.random.Generator(np.random.PCG64(33))
    raw = rng.standard_normal((23, 128)).astype(np.float32)          # 5 whole blocks + 3 cells
    gamma = rng.standard_normal(128).astype(np.float32)
    table = oracle.rope_table(1e7, 64, 64)
    got = oracle.pool_keys(raw, gamma, table)
    assert got.shape == (5, 128)
    for b in range(5):
        mean = np.zeros(128, dtype=np.float32)
        for k in range(4):
            mean = (mean + raw[4 * b + k] / np.float32(4)).astype(np.float32)    # f32, cell order
        want = oracle.rope_apply(oracle.rmsnorm(mean, 128, gamma, eps=1e-6), 128, 64, table, [4 * b])
        assert np.array_equal(got[b], want.reshape(-1))
    # closed forms: four equal rows pool to that row's normalised rotation; block 0 is not rotated
    same = np.tile(raw[:1], (4, 1))
    one = oracle.pool_keys(same, gamma, table)[0]
    assert np.array_equal(one, oracle.rmsnorm(raw[0], 128, gamma, eps=1e-6).reshape(-1))
    # a block with one non-zero row equals that row / 4 before the norm, and the norm undoes the 4
    lone = np.zeros((8, 128), dtype=np.float32)
    lone[5] = raw[5]
    got2 = oracle.pool_keys(lone, np.ones(128, dtype=np.float32), table, eps=0.0)
    ref2 = oracle.rope_apply(oracle.rmsnorm(raw[5], 128, None, eps=0.0), 128, 64, table, [4])
    assert np.max(np.abs(got2[1] - ref2.reshape(-1))) < 1e-6
    # (block 0 is all zeros: with eps = 0 its norm is 0/0, as the formula says)
    assert np.all(oracle.pool_keys(lone, np.ones(128, dtype=np.float32), table, eps=1e-6)[0] == 0.0)
