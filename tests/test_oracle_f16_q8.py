"""Pins the oracle's storage encodings (f16 rule, q8_0, int8+f16-scale) against the
reference's own known answers and against independent converters.  CPU only."""
import json
import os

import numpy as np
import pytest

import oracle

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_kats.json")))


def bits_of(x):
    return np.asarray(x, dtype=np.float32).view(np.uint32)


def test_f16_known_answers_of_the_reference():
    # crates/breccia-kernels/src/qsa/cpu.rs:501-515
    for case in GOLD["f16_round_trip"]["cases"]:
        got = float(oracle.to_f16(np.array([case["in"]], dtype=np.float32))[0])
        if case["out"] == "inf":
            assert np.isinf(got) and got > 0
        else:
            assert got == np.float32(case["out"]), case
        if "half_bits" in case:
            assert int(oracle.f32_to_f16_bits(np.array([case["in"]], dtype=np.float32))[0]) == int(case["half_bits"], 16)


def test_f16_driver_known_answer():
    # crates/breccia-kernels/shaders/f16_storage.glsl:5-6: RNE gives 0x3AFF, truncation 0x3AFE
    kat = GOLD["f16_driver_kat"]
    x = np.array([int(kat["f32_bits"], 16)], dtype=np.uint32).view(np.float32)
    assert int(oracle.f32_to_f16_bits(x)[0]) == int(kat["half_bits"], 16)


def _numpy_expected(bits: np.ndarray) -> np.ndarray:
    """numpy's IEEE RNE cast with the cache rule's two documented deviations applied."""
    with np.errstate(over="ignore", invalid="ignore"):
        h = bits.view(np.float32).astype(np.float16).view(np.uint16)
    mag = bits & np.uint32(0x7FFFFFFF)
    sign = ((bits >> np.uint32(16)) & np.uint32(0x8000)).astype(np.uint16)
    h = np.where(mag < np.uint32(0x38800000), sign, h)
    h = np.where(mag > np.uint32(0x7F800000), sign | np.uint16(0x7C00), h)
    return h.astype(np.uint16)


def test_f16_encode_matches_numpy_on_a_structured_sample():
    rng = np.random.Generator(np.random.PCG64(11))
    parts = [rng.integers(0, 2**32, size=1 << 21, dtype=np.uint64).astype(np.uint32)]
    # every exponent with mantissas at and around the rounding boundaries
    exps = np.arange(256, dtype=np.uint32) << np.uint32(23)
    man = np.array([0, 1, 0xFFF, 0x1000, 0x1001, 0x1FFF, 0x2000, 0x2FFF, 0x3000, 0x3001,
                    0x7FE000, 0x7FEFFF, 0x7FF000, 0x7FF001, 0x7FFFFF], dtype=np.uint32)
    grid = (exps[:, None] | man[None, :]).reshape(-1)
    parts += [grid, grid | np.uint32(0x80000000)]
    # dense neighbourhoods of 2^-14, 65504/65520 and the f32 subnormal range
    for centre in (0x38800000, 0x477FE000, 0x477FF000, 0x00800000, 0x7F800000):
        parts.append(np.arange(centre - 4096, centre + 4096, dtype=np.uint32))
    bits = np.concatenate(parts)
    got = oracle.f32_to_f16_bits(bits.view(np.float32))
    want = _numpy_expected(bits)
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, (hex(int(bits[bad[0]])), hex(int(got[bad[0]])), hex(int(want[bad[0]])))


def test_f16_encode_exhaustive_against_the_f16c_instruction():
    """All 2^32 inputs: the oracle equals the x86 F16C convert except |x| < 2^-14 -> 0 and NaN -> inf."""
    convert = oracle.f16c_reference()
    if convert is None:
        pytest.skip("this CPU has no F16C")
    chunk = 1 << 26
    total_bad = 0
    for first in range(0, 1 << 32, chunk):
        want = convert(first, chunk)
        total_bad += oracle.f16_sweep_mismatches(first, want, documented_deviations=True)
    assert total_bad == 0
    # and the deviations are real: without them the subnormal/NaN ranges disagree
    first = 0x38000000  # just below 2^-14: IEEE gives subnormal halves, the cache rule zero
    assert oracle.f16_sweep_mismatches(first, convert(first, 1 << 16), False) > 0


def test_f16_decode_matches_numpy_on_every_code():
    codes = np.arange(1 << 16, dtype=np.uint16)
    got = oracle.f16_bits_to_f32(codes)
    want = codes.view(np.float16).astype(np.float32)
    e = (codes >> 10) & 0x1F
    sub = e == 0  # documented deviation: subnormal codes read as signed zero
    want = np.where(sub, np.where(codes & 0x8000, np.float32(-0.0), np.float32(0.0)), want)
    assert np.array_equal(got.view(np.uint32), want.astype(np.float32).view(np.uint32))


def test_f16_round_trip_is_idempotent_and_monotone():
    rng = np.random.Generator(np.random.PCG64(5))
    x = np.sort(rng.standard_normal(1 << 16).astype(np.float32) * 50)
    y = oracle.to_f16(x)
    assert np.array_equal(oracle.to_f16(y).view(np.uint32), y.view(np.uint32))
    assert np.all(np.diff(y) >= 0)


# ---------------------------------------------------------------------------- q8_0
def test_q8_0_reference_bound_fixture():
    # crates/breccia-kernels/src/qsa/mod.rs:2072-2106
    zeros = np.zeros(64, dtype=np.float32)
    deq, q, sc = oracle.to_q8_0(zeros)
    assert np.array_equal(deq.view(np.uint32), zeros.view(np.uint32))
    assert np.all(sc == 1.0) and np.all(q == 0)
    x = oracle.q8_fixture(256)
    # the fixture is a pure integer LCG: check its first values against the recipe done in Python
    s = 12345
    for i in range(4):
        s = (s * 6364136223846793005 + 1) % (1 << 64)
        assert x[i] == np.float32((np.float32(s >> 40) / np.float32(1 << 24) - np.float32(0.5)) * np.float32(8.0))
    deq, q, sc = oracle.to_q8_0(x)
    for b in range(256 // 32):
        blk = slice(b * 32, b * 32 + 32)
        amax = np.abs(x[blk]).max()
        half_lsb = np.float32(amax) / np.float32(127.0) / np.float32(2.0)
        assert np.all(np.abs(deq[blk] - x[blk]) <= half_lsb * 1.001)
        assert abs(np.abs(deq[blk]).max() - amax) <= half_lsb * 1.001
        assert sc[b] == np.float32(amax) / np.float32(127.0)
    assert np.all(np.abs(q.astype(np.int32)) <= 127)


def test_q8_0_against_an_independent_numpy_statement():
    rng = np.random.Generator(np.random.PCG64(3))
    x = (rng.standard_normal(32 * 512) * rng.uniform(1e-3, 30, size=32 * 512)).astype(np.float32)
    x[64:96] = 0.0
    deq, q, sc = oracle.to_q8_0(x)
    xb = x.reshape(-1, 32)
    amax = np.abs(xb).max(axis=1)
    scale = np.where(amax > 0, amax / np.float32(127.0), np.float32(1.0)).astype(np.float32)
    t = np.clip(xb / scale[:, None], -127.0, 127.0).astype(np.float32)
    # round half away from zero, stated without calling any rounding routine
    r = np.sign(t) * np.floor(np.abs(t) + np.float32(0.5))
    assert np.array_equal(q.reshape(-1, 32), r.astype(np.int8))
    assert np.array_equal(sc, scale)
    assert np.array_equal(deq.reshape(-1, 32), (r.astype(np.float32) * scale[:, None]).astype(np.float32))


def test_q8_0_rounds_half_away_from_zero():
    # amax = 127 -> scale exactly 1: values at .5 must move away from zero
    x = np.zeros(32, dtype=np.float32)
    x[0], x[1], x[2], x[3], x[4] = 127.0, 0.5, -0.5, 2.5, -3.5
    _, q, sc = oracle.to_q8_0(x)
    assert sc[0] == 1.0
    assert list(q[:5]) == [127, 1, -1, 3, -4]


# ---------------------------------------------------------- int8 with an f16 scale
def test_i8h_bounds_and_scale_rule():
    """Not in the reference: pinned by closed-form properties only."""
    rng = np.random.Generator(np.random.PCG64(9))
    x = (rng.standard_normal(32 * 256)).astype(np.float32)
    x[:32] = 0.0
    x[32:64] *= 1e-4   # amax/127 below 2^-14: the scale must be raised to the smallest normal
    deq, q, sb = oracle.to_i8h(x)
    scale = oracle.f16_bits_to_f32(sb)
    assert sb[0] == 0x3C00 and np.all(deq[:32] == 0)
    assert sb[1] == 0x0400
    xb, db = x.reshape(-1, 32), deq.reshape(-1, 32)
    amax = np.abs(xb).max(axis=1)
    want_scale = oracle.to_f16((amax / np.float32(127.0)).astype(np.float32))
    ok = (amax > 0) & (want_scale >= 2.0 ** -14)
    assert np.array_equal(scale[ok], want_scale[ok])
    assert np.all(np.abs(q.astype(np.int32)) <= 127)
    # error bound: half a step, plus the clamp loss when the f16 scale rounded down
    step = scale[:, None]
    clamp_loss = np.maximum(np.abs(xb) - 127.0 * step, 0.0)
    assert np.all(np.abs(db - xb) <= 0.5 * step * 1.0001 + clamp_loss)
    assert np.array_equal(db, q.reshape(-1, 32).astype(np.float32) * step)
