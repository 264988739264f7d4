"""BASELINE.json's batched configurations at full size on the GPU.

configs[2] (batch 8, contexts 1k..32k, f16): parity against the oracle on every (sequence, head).
configs[4] (batch 16, contexts 8k..128k, int8 K/V with f16 scales): the oracle attends over the
rows read back through bkv_gather for a seeded subset of sequences (shortest, median, longest --
all 16 heads each; the full f64 oracle over all 16 sequences is ~10^10 MACs), plus
size-independent properties on all of them: the batched call equals the per-sequence call to
1e-6, and every output is a convex combination of V rows (bounded by the largest |v|).
configs[3] shape (4 sequences, 2048-token prefix + 1024-token chunk) through the chunk kernel on
all three layouts: sampled tokens against the oracle, the chunk's tail against the decode kernel."""
import numpy as np
import pytest

import oracle
from breccia_amd import lib as L
from breccia_amd.kv import DeviceBuffer, Pool, device_sync
from gpu_common import REF_BAR_MAX_REL, check_attn
from helpers import max_abs

pytestmark = pytest.mark.gpu
N_Q, N_KV, HD = 16, 2, 256


def build(rng, n_seqs, lo, hi, layout, occupancy=0.6):
    ctx = []
    for _ in range(n_seqs):
        c = int(rng.integers(lo, hi + 1))
        if c % 16 == 0:
            c -= 3
        ctx.append(c)
    live = sum((c + 15) // 16 for c in ctx)
    n_pages = int(np.ceil(live / occupancy))
    pool = Pool(n_layers=1, n_pages=n_pages, n_kv_head=N_KV, head_dim=HD, layout=layout,
                max_seqs=n_seqs + 1, max_pages_per_seq=max(ctx) // 16 + 2)
    pool.set_free_order(rng.permutation(n_pages).astype(np.int32))
    seqs = [pool.seq_create() for _ in ctx]
    grown = [0] * n_seqs
    while any(g < c for g, c in zip(grown, ctx)):   # deal pages round-robin: interleaved tables
        for i, s in enumerate(seqs):
            if grown[i] < ctx[i]:
                grown[i] = min(ctx[i], grown[i] + 16 * 8)
                pool.seq_reserve(s, grown[i])
    return pool, seqs, ctx


def fill_tiled(pool, seqs, ctx, rng, tile=8192):
    """Append N(0,1) rows; one random tile of `tile` tokens per sequence offset keeps the host
    side small while every sequence still holds distinct data (a different window per chunk)."""
    src_k = rng.standard_normal((3 * tile, N_KV, HD), dtype=np.float32)
    src_v = rng.standard_normal((3 * tile, N_KV, HD), dtype=np.float32)
    kd, vd = DeviceBuffer.from_numpy(src_k), DeviceBuffer.from_numpy(src_v)
    row = N_KV * HD * 4
    for i, (s, c) in enumerate(zip(seqs, ctx)):
        at = 0
        while at < c:
            n = min(tile, c - at)
            off = int(rng.integers(0, 2 * tile)) * row
            pool.append(0, [s], [at], [n], kd.at(off), vd.at(off))
            at += n
    device_sync()
    kd.free()
    vd.free()


def run_attn(pool, seqs, pos, q):
    qd = DeviceBuffer.from_numpy(q)
    od = DeviceBuffer(q.nbytes)
    pool.decode_attn(0, seqs, pos, N_Q, qd, od, 1.0 / 16.0)
    device_sync()
    out = od.download(np.float32).reshape(len(seqs), N_Q, HD)
    qd.free()
    od.free()
    return out


def oracle_for(pool, seq, pos, q):
    k, v = pool.gather(0, seq, 0, pos + 1)
    return oracle.attend(q, k, v, oracle.dense_cells(pos), pos, N_Q, N_KV, HD, threads=8), v


def test_config3_batch8_mixed_1k_32k_all_heads():
    rng = np.random.Generator(np.random.PCG64(20250003))
    pool, seqs, ctx = build(rng, 8, 1024, 32768, L.LAYOUT_F16)
    try:
        fill_tiled(pool, seqs, ctx, rng)
        # the step: one more token per sequence, then attention at the new position
        for s, c in zip(seqs, ctx):
            pool.seq_reserve(s, c + 1)
        new = rng.standard_normal((8, N_KV, HD), dtype=np.float32)
        nd = DeviceBuffer.from_numpy(new)
        pool.append(0, seqs, ctx, [1] * 8, nd, nd)
        q = rng.standard_normal((8, N_Q, HD), dtype=np.float32)
        out = run_attn(pool, seqs, ctx, q)
        worst = 0.0
        for i, s in enumerate(seqs):
            want, _ = oracle_for(pool, s, ctx[i], q[i])
            _, rel = check_attn(out[i], want, "config3 seq %d (ctx %d)" % (i, ctx[i]))
            worst = max(worst, rel)
        assert worst <= REF_BAR_MAX_REL, worst
        nd.free()
    finally:
        pool.destroy()


def test_config5_batch16_int8_8k_128k():
    rng = np.random.Generator(np.random.PCG64(20250005))
    pool, seqs, ctx = build(rng, 16, 8192, 131072, L.LAYOUT_I8H)
    try:
        fill_tiled(pool, seqs, ctx, rng)
        q = rng.standard_normal((16, N_Q, HD), dtype=np.float32)
        pos = [c - 1 for c in ctx]
        out = run_attn(pool, seqs, pos, q)
        assert np.all(np.isfinite(out))
        order = np.argsort(ctx)
        for i in (int(order[0]), int(order[8]), int(order[-1])):
            want, v = oracle_for(pool, seqs[i], pos[i], q[i])
            _, rel = check_attn(out[i], want, "config5 seq %d (ctx %d)" % (i, ctx[i]))
            assert rel <= REF_BAR_MAX_REL, rel
            assert np.abs(out[i]).max() <= np.abs(v).max()
        # batched == one at a time (different split plans), all 16 sequences
        for i in range(16):
            alone = run_attn(pool, [seqs[i]], [pos[i]], q[i:i + 1])
            assert max_abs(alone[0], out[i]) < 1e-6, i
    finally:
        pool.destroy()


@pytest.mark.parametrize("layout", [L.LAYOUT_F16, L.LAYOUT_Q8V, L.LAYOUT_I8H])
def test_config4_shape_prefill_of_1024_token_chunks_on_2048_token_prefixes(layout):
    # BASELINE configs[3] at full size through the chunk kernel: 4 sequences, a 2048-token prefix in
    # the cache, a 1024-token chunk each, one call.  Sampled tokens of every sequence against the
    # oracle (over the rows read back through bkv_gather) at the reference's bar; the chunk's last 64
    # positions of one sequence against the decode kernel; every output bounded by the largest |v|.
    rng = np.random.Generator(np.random.PCG64(20250004 + layout))
    before, t = 2048, 1024
    ctx = [before + t] * 4
    live = sum((c + 15) // 16 for c in ctx)
    pool = Pool(n_layers=1, n_pages=int(np.ceil(live / 0.6)), n_kv_head=N_KV, head_dim=HD, layout=layout,
                max_seqs=5, max_pages_per_seq=ctx[0] // 16 + 2)
    pool.set_free_order(rng.permutation(pool.desc.n_pages).astype(np.int32))
    try:
        seqs = [pool.seq_create() for _ in ctx]
        for s in seqs:
            pool.seq_reserve(s, ctx[0])
        fill_tiled(pool, seqs, ctx, rng, tile=1024)
        q = rng.standard_normal((4 * t, N_Q, HD), dtype=np.float32)
        qd, od = DeviceBuffer.from_numpy(q), DeviceBuffer(q.nbytes)
        pool.prefill_attn(0, seqs, [before] * 4, [t] * 4, N_Q, qd, od, 1.0 / 16.0)
        device_sync()
        out = od.download(np.float32).reshape(4, t, N_Q, HD)
        assert np.all(np.isfinite(out))
        worst = 0.0
        for i, s in enumerate(seqs):
            k, v = pool.gather(0, s, 0, ctx[i])
            assert np.abs(out[i]).max() <= np.abs(v).max()
            for tok in sorted({0, t - 1, t // 2, int(rng.integers(0, t)), int(rng.integers(0, t))}):
                pos = before + tok
                want = oracle.attend(q[i * t + tok], k[:pos + 1], v[:pos + 1], oracle.dense_cells(pos), pos, N_Q,
                                     N_KV, HD, threads=8)
                _, rel = check_attn(out[i, tok], want, "config4 seq %d token %d" % (i, tok))
                worst = max(worst, rel)
        assert worst <= REF_BAR_MAX_REL, worst
        tail = list(range(ctx[2] - 64, ctx[2]))
        dec = run_attn(pool, [seqs[2]] * 64, tail, q[2 * t + t - 64:3 * t])
        assert max_abs(dec, out[2, -64:]) < 5e-6
        qd.free()
        od.free()
    finally:
        pool.destroy()
