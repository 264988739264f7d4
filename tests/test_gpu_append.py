"""GPU parity of paged K/V append, gather and the pool lifecycle against the CPU oracle.
Bit-exact: every byte of every pool is compared."""
import json
import os

import numpy as np
import pytest

import oracle
from breccia_amd import lib as L
from breccia_amd.kv import BkvError, DeviceBuffer, Stream, device_sync
from gpu_common import Twin

pytestmark = pytest.mark.gpu
GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_kats.json")))


def test_reference_layout_recipe_on_the_gpu():
    # crates/breccia-kernels/tests/attn_conformance.rs:1172-1275: identity table, capacity 40,
    # 33 single-token appends from cell 5; every stored half must be the cache encoding.
    r = GOLD["layout_recipe"]
    with Twin(n_pages=3, max_seqs=2) as tw:
        s = tw.pool.seq_create_identity(3)
        tw.pool.seq_reserve(s, 48)      # capacity 40 rounded up to whole pages
        i = np.arange(512)
        for t in range(r["n_tokens"]):
            cell = r["start_cell"] + t
            k = (np.sin((cell * 97 + i * 13).astype(np.float32) * np.float32(0.017)) * np.float32(3.0)).astype(np.float32)
            v = (np.cos((cell * 61 + i * 7).astype(np.float32) * np.float32(0.031)) * np.float32(2.0)).astype(np.float32)
            tw.append(0, [s], [cell], [k], [v])
        tw.assert_pools_equal()
        kp = tw.pool.read_layer(0, 0).view(np.uint16).reshape(3, 2, 16, 256)
        assert kp[0, :, :5].sum() == 0 and kp[2, :, 6:].sum() == 0   # unwritten cells still zero
        # the reference's capacity error (qsa/mod.rs:1108-1116)
        z = DeviceBuffer(4096)
        with pytest.raises(BkvError) as ei:
            tw.pool.append(0, [s], [47], [2], z, z)
        assert ei.value.status == L.ERR_RANGE
        z.free()


def test_batched_ragged_append_through_permuted_tables():
    rng = np.random.Generator(np.random.PCG64(31))
    with Twin(n_pages=256, max_seqs=8) as tw:
        perm = rng.permutation(256)
        seqs = [tw.pool.seq_create() for _ in range(5)]
        lens = [37, 0, 512, 1000, 16]
        # scramble physical pages: reserve in interleaved steps so tables are not contiguous
        for step in range(0, 1100, 48):
            for s, n in zip(seqs, lens):
                tgt = min(n, step + 48)
                if tgt > tw.pool.seq_len(s):
                    tw.pool.seq_reserve(s, tgt)
        ks = [rng.standard_normal((n, 2, 256)).astype(np.float32) for n in lens]
        vs = [rng.standard_normal((n, 2, 256)).astype(np.float32) for n in lens]
        tw.append(0, seqs, [0] * 5, ks, vs)          # one ragged call, one empty sequence
        tw.assert_pools_equal()
        # decode-style step: one token each where there is room, crossing page boundaries
        for s in seqs:
            tw.pool.seq_reserve(s, tw.pool.seq_len(s) + 1)
        k1 = [rng.standard_normal((1, 2, 256)).astype(np.float32) for _ in seqs]
        v1 = [rng.standard_normal((1, 2, 256)).astype(np.float32) for _ in seqs]
        tw.append(0, seqs, lens, k1, v1)
        tw.assert_pools_equal()
        # gather == the f16 round trip of what went in
        gk, gv = tw.pool.gather(0, seqs[3], 990, 11)
        want_k = oracle.to_f16(np.concatenate([ks[3][990:], k1[3]]))
        assert np.array_equal(gk, want_k)
        ok, ov = tw.images[0].gather(tw.pool.block_table(seqs[3]), 990, 11)
        assert np.array_equal(gk, ok) and np.array_equal(gv, ov)
        tw.pool.check()


def test_special_values_follow_the_cache_f16_rule():
    # crates/breccia-kernels/shaders/f16_storage.glsl:26-55: below 2^-14 -> +-0, NaN -> +-inf,
    # >= 65520 -> inf, ties to even
    bits = []
    for centre in (0x38800000, 0x477FE000, 0x477FF000, 0x00800000, 0x7F800000, 0x33000000):
        bits.append(np.arange(centre - 512, centre + 512, dtype=np.uint32))
    exps = np.arange(256, dtype=np.uint32) << np.uint32(23)
    man = np.array([0, 1, 0xFFF, 0x1000, 0x1001, 0x2FFF, 0x3000, 0x3001, 0x7FEFFF, 0x7FF000, 0x7FFFFF],
                   dtype=np.uint32)
    bits.append((exps[:, None] | man[None, :]).reshape(-1))
    b = np.concatenate(bits)
    b = np.concatenate([b, b | np.uint32(0x80000000)])
    rng = np.random.Generator(np.random.PCG64(8))
    pad = (-b.size) % 512
    b = np.concatenate([b, rng.integers(0, 2**32, size=pad, dtype=np.uint64).astype(np.uint32)])
    x = b.view(np.float32).reshape(-1, 2, 256)
    T = x.shape[0]
    with Twin(n_pages=(T + 15) // 16 + 1, max_seqs=2) as tw:
        s = tw.pool.seq_create()
        tw.pool.seq_reserve(s, T)
        tw.append(0, [s], [0], [x], [x[::-1].copy()])
        tw.assert_pools_equal()


def test_random_bit_patterns_two_million():
    rng = np.random.Generator(np.random.PCG64(77))
    T = 4096
    x = rng.integers(0, 2**32, size=(T, 2, 256), dtype=np.uint64).astype(np.uint32).view(np.float32)
    y = rng.integers(0, 2**32, size=(T, 2, 256), dtype=np.uint64).astype(np.uint32).view(np.float32)
    with Twin(n_pages=T // 16, max_seqs=2) as tw:
        s = tw.pool.seq_create()
        tw.pool.seq_reserve(s, T)
        tw.append(0, [s], [0], [x], [y])
        tw.assert_pools_equal()


def test_prefill_chunks_equal_token_by_token_appends():
    rng = np.random.Generator(np.random.PCG64(4))
    k = rng.standard_normal((300, 2, 256)).astype(np.float32)
    v = rng.standard_normal((300, 2, 256)).astype(np.float32)
    with Twin(n_pages=64, max_seqs=4) as tw:
        a, b = tw.pool.seq_create(), tw.pool.seq_create()
        tw.pool.seq_reserve(a, 303)
        tw.pool.seq_reserve(b, 303)
        tw.append(0, [a], [3], [k], [v])
        kd, vd = DeviceBuffer.from_numpy(k), DeviceBuffer.from_numpy(v)
        for t in range(300):  # T x append(1) straight through the C ABI, no sync in between
            tw.pool.append(0, [b], [3 + t], [1], kd.at(t * 2048), vd.at(t * 2048))
        device_sync()
        ka, va = tw.pool.gather(0, a, 0, 303)
        kb, vb = tw.pool.gather(0, b, 0, 303)
        assert np.array_equal(ka, kb) and np.array_equal(va, vb)
        kd.free()
        vd.free()


@pytest.mark.parametrize("layout", [L.LAYOUT_Q8V, L.LAYOUT_I8H])
def test_quantised_append_is_bit_exact(layout):
    # q8_0 V: crates/breccia-kernels/shaders/qsa_kv_append.comp:87-132, qsa/cpu.rs:65-82
    rng = np.random.Generator(np.random.PCG64(12 + layout))
    with Twin(n_pages=96, layout=layout, max_seqs=4) as tw:
        perm_owner = tw.pool.seq_create()
        tw.pool.seq_reserve(perm_owner, 16 * 7)     # shift the next sequence's pages
        s = tw.pool.seq_create()
        lens = 517
        tw.pool.seq_reserve(s, lens)
        k = (rng.standard_normal((lens, 2, 256)) * rng.uniform(0.01, 20, size=(lens, 2, 1))).astype(np.float32)
        v = (rng.standard_normal((lens, 2, 256)) * rng.uniform(0.01, 20, size=(lens, 2, 1))).astype(np.float32)
        v[5, 0, 32:64] = 0.0                        # an all-zero block keeps scale 1
        k[9, 1, :32] *= 1e-5                        # a scale the f16 rule would flush
        tw.append(0, [s], [0], [k[:500]], [v[:500]])
        tw.append(0, [s], [500], [k[500:]], [v[500:]])
        tw.assert_pools_equal()
        gk, gv = tw.pool.gather(0, s, 0, lens)
        ok, ov = tw.images[0].gather(tw.pool.block_table(s), 0, lens)
        assert np.array_equal(gk, ok) and np.array_equal(gv, ov)


@pytest.mark.parametrize("f16_rows", [False, True])
@pytest.mark.parametrize("layout", [L.LAYOUT_Q8V, L.LAYOUT_I8H])
def test_quantised_bulk_append_with_ties_is_bit_exact(layout, f16_rows):
    # The bulk kernels take the codes from a reciprocal of the scale where that provably gives the
    # rule's round-half-away(clamp(x / scale)) (qsa/cpu.rs:65-82) and from the division itself
    # elsewhere: 3000 tokens (most waves on the short cut, some not), blocks of exact ties
    # (scale 1 and 1/4: values k + 1/2 and (k + 1/2) / 4, both signs), values one ulp either side
    # of a tie, blocks below 2^-6 (f16 rows are flushed there), an all-zero block, a lone large value.
    rng = np.random.Generator(np.random.PCG64(300 + 2 * layout + int(f16_rows)))
    T = 3000
    k = (rng.standard_normal((T, 2, 256)) * rng.uniform(0.05, 30, size=(T, 2, 1))).astype(np.float32)
    v = (rng.standard_normal((T, 2, 256)) * rng.uniform(0.05, 30, size=(T, 2, 1))).astype(np.float32)
    halves = (np.arange(32, dtype=np.float32) * 7.0) % 126.0 + 0.5
    halves[::2] *= -1.0
    for x in (k, v):
        x[10, 0, 0:32] = halves
        x[10, 0, 0] = 127.0                         # amax 127: scale exactly 1
        x[11, 1, 64:96] = halves / 4.0
        x[11, 1, 64] = -127.0 / 4.0                 # scale exactly 1/4
        x[12, 0, 32:64] = np.nextafter(halves, np.float32(1000.0))
        x[12, 0, 32] = 127.0
        x[13, 1, 32:64] = np.nextafter(halves, np.float32(-1000.0))
        x[13, 1, 32] = 127.0
        x[14, 0, 96:128] = rng.standard_normal(32).astype(np.float32) * 1e-3     # amax below 2^-6
        x[15, 1, 0:32] = rng.standard_normal(32).astype(np.float32) * 3e-5       # around 2^-14 and below
        x[16, 0, 128:160] = 0.0
        x[17, 1, 160:192] = 1e-4
        x[17, 1, 161] = 5e4
    if f16_rows:
        with np.errstate(over="ignore"):
            k, v = k.astype(np.float16).view(np.uint16), v.astype(np.float16).view(np.uint16)
    with Twin(n_pages=T // 16 + 8, layout=layout, max_seqs=4) as tw:
        s = tw.pool.seq_create()
        tw.pool.seq_reserve(s, T + 5)
        tw.append(0, [s], [5], [k], [v], f16_rows=f16_rows)
        tw.assert_pools_equal()


@pytest.mark.parametrize("layout", [L.LAYOUT_F16, L.LAYOUT_Q8V, L.LAYOUT_I8H])
def test_f16_rows_append_like_their_widened_f32_rows(layout):
    # bkv_append_f16: raw binary16 rows, read under the cache's load rule
    # (crates/breccia-kernels/shaders/f16_storage.glsl:58-69), then the path of bkv_append.
    rng = np.random.Generator(np.random.PCG64(90 + layout))
    T = 259
    k = rng.standard_normal((T, 2, 256)).astype(np.float16).view(np.uint16)
    v = rng.standard_normal((T, 2, 256)).astype(np.float16).view(np.uint16)
    # every one of the 65536 codes appears at least once: subnormals, infinities, NaN payloads
    codes = np.arange(65536, dtype=np.uint16).reshape(128, 2, 256)
    k = np.concatenate([k, codes[:64], v[:5]])
    v = np.concatenate([v, codes[64:], k[:5]])
    n = k.shape[0]
    with Twin(n_pages=64, layout=layout, max_seqs=4) as tw:
        other = tw.pool.seq_create()
        tw.pool.seq_reserve(other, 40)
        s = tw.pool.seq_create()
        tw.pool.seq_reserve(s, n + 3)
        tw.append(0, [s], [3], [k], [v], f16_rows=True)
        tw.assert_pools_equal()
        if layout == L.LAYOUT_F16:
            # finite normal codes are stored verbatim; subnormal codes as signed zeros; NaN as inf
            got = tw.pool.gather(0, s, 3, n)[0].reshape(-1)
            src = k.reshape(-1)
            normal = ((src >> 10) & 0x1F != 0) & ((src >> 10) & 0x1F != 31)
            assert np.array_equal(oracle.f32_to_f16_bits(got[normal]), src[normal])
        # the f32 append of the widened rows lands on the same bytes
        t2 = tw.pool.seq_create()
        tw.pool.seq_reserve(t2, n + 3)
        wk = oracle.f16_bits_to_f32(k.reshape(-1)).reshape(k.shape)
        wv = oracle.f16_bits_to_f32(v.reshape(-1)).reshape(v.shape)
        tw.append(0, [t2], [3], [wk], [wv])
        a = tw.pool.gather(0, s, 3, n)
        b = tw.pool.gather(0, t2, 3, n)
        assert np.array_equal(a[0].view(np.uint32), b[0].view(np.uint32))
        assert np.array_equal(a[1].view(np.uint32), b[1].view(np.uint32))
        # errors are the same as bkv_append's
        z = DeviceBuffer(4096)
        with pytest.raises(BkvError) as ei:
            tw.pool.append(0, [s], [tw.pool.seq_capacity(s)], [1], z, z, f16_rows=True)
        assert ei.value.status == L.ERR_RANGE
        z.free()


def test_enqueue_on_a_stream_equals_sync_after_every_call():
    # the reference's batching contract (crates/breccia-kernels/tests/batching.rs:27-88):
    # six dependent operations recorded back to back == the same six run one at a time
    rng = np.random.Generator(np.random.PCG64(6))
    k = [rng.standard_normal((t, 2, 256)).astype(np.float32) for t in (40, 1, 1, 25, 1, 1)]
    v = [rng.standard_normal((t, 2, 256)).astype(np.float32) for t in (40, 1, 1, 25, 1, 1)]
    images = []
    for sync_each in (False, True):
        with Twin(n_pages=16, max_seqs=2) as tw:
            st = Stream()
            s = tw.pool.seq_create()
            bufs, pos = [], 0
            for ki, vi in zip(k, v):
                tw.pool.seq_reserve(s, pos + ki.shape[0])
                kd, vd = DeviceBuffer.from_numpy(ki), DeviceBuffer.from_numpy(vi)
                bufs += [kd, vd]
                tw.pool.append(0, [s], [pos], [ki.shape[0]], kd, vd, st)
                if sync_each:
                    st.sync()
                pos += ki.shape[0]
            st.sync()
            images.append((tw.pool.read_layer(0, 0), tw.pool.read_layer(0, 1)))
            for b in bufs:
                b.free()
            st.close()
    assert np.array_equal(images[0][0], images[1][0]) and np.array_equal(images[0][1], images[1][1])


def test_reset_zeroes_the_pools_and_frees_every_sequence():
    # crates/breccia-kernels/src/qsa/mod.rs:551-570
    rng = np.random.Generator(np.random.PCG64(1))
    with Twin(n_pages=8, max_seqs=2) as tw:
        s = tw.pool.seq_create()
        tw.pool.seq_reserve(s, 100)
        x = rng.standard_normal((100, 2, 256)).astype(np.float32)
        tw.append(0, [s], [0], [x], [x])
        assert tw.pool.read_layer(0, 0).any()
        tw.pool.reset()
        device_sync()
        assert not tw.pool.read_layer(0, 0).any() and not tw.pool.read_layer(0, 1).any()
        assert tw.pool.free_pages() == 8 and tw.pool.seq_len(s) == -1
        tw.pool.fill(0xFF)
        device_sync()
        assert (tw.pool.read_layer(0, 1) == 0xFF).all()


@pytest.mark.parametrize("layout", [L.LAYOUT_F16, L.LAYOUT_Q8V, L.LAYOUT_I8H])
@pytest.mark.parametrize("n_kv,hd", [(3, 96), (1, 32), (8, 128), (5, 256)])
def test_other_geometries_append_bit_exact(layout, n_kv, hd):
    # the append kernels (plain and with the K preparation fused in) take any head count and any
    # head dim that is a multiple of 32 (the int8 layout: head dim 256 only): every pool byte
    # against the oracle, chunked and one token at a time, through a permuted table
    from breccia_amd.kv import rope_table
    if layout == L.LAYOUT_I8H and hd != 256:
        with pytest.raises(BkvError) as ei:
            Twin(n_pages=8, n_kv=n_kv, hd=hd, layout=layout, max_seqs=2)
        assert ei.value.status == L.ERR_INVALID
        return
    rng = np.random.Generator(np.random.PCG64(40 + layout + 7 * n_kv + hd))
    n_rot = min(64, hd)
    gamma = (1.0 + 0.3 * rng.standard_normal(hd)).astype(np.float32)
    table = rope_table(1e7, n_rot, 512)
    gd, td = DeviceBuffer.from_numpy(gamma), DeviceBuffer.from_numpy(table)
    with Twin(n_pages=64, n_kv=n_kv, hd=hd, layout=layout, max_seqs=4) as tw:
        tw.pool.set_free_order(rng.permutation(64).astype(np.int32))
        a, b = tw.pool.seq_create(), tw.pool.seq_create()
        n = 203
        for s in (a, b):
            tw.pool.seq_reserve(s, n)
        k = (rng.standard_normal((n, n_kv, hd)) * rng.uniform(0.01, 20, size=(n, n_kv, 1))).astype(np.float32)
        v = (rng.standard_normal((n, n_kv, hd)) * rng.uniform(0.01, 20, size=(n, n_kv, 1))).astype(np.float32)
        # plain append: a chunk, then token by token
        tw.append(0, [a], [0], [k[:190]], [v[:190]])
        for t in range(190, n):
            tw.append(0, [a], [t], [k[t:t + 1]], [v[t:t + 1]])
        tw.assert_pools_equal()
        # fused K preparation on the second sequence: two chunks
        for lo, hi in ((0, 150), (150, n)):
            kd = DeviceBuffer.from_numpy(np.concatenate([k[lo:hi].reshape(-1), np.zeros(4, np.float32)]))
            vd = DeviceBuffer.from_numpy(np.concatenate([v[lo:hi].reshape(-1), np.zeros(4, np.float32)]))
            tw.pool.append_kprep(0, [b], [lo], [hi - lo], kd, vd, gd, 1e-6, td, n_rot, 512, None)
            device_sync()
            kd.free()
            vd.free()
            want_k = oracle.k_prep(k[lo:hi], n_kv, hd, gamma, 1e-6, table, n_rot, np.arange(lo, hi))
            assert tw.images[0].append(tw.pool.block_table(b), lo, want_k, v[lo:hi],
                                       capacity_cells=tw.pool.seq_capacity(b)) == 0
        tw.assert_pools_equal()
        tw.pool.check()
        if hd != 256:
            # the attention kernels are built for head dim 256: refused, not launched
            z = DeviceBuffer(1 << 16)
            for call in (lambda: tw.pool.decode_attn(0, [a], [n - 1], 2 * n_kv, z, z, 0.0625),
                         lambda: tw.pool.prefill_attn(0, [a], [0], [n], 2 * n_kv, z, z, 0.0625)):
                with pytest.raises(BkvError) as ei:
                    call()
                assert ei.value.status == L.ERR_INVALID
            z.free()
    gd.free()
    td.free()
