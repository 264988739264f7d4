"""The per-kernel timers (bkv_timing_*): launches are attributed to their stages, the durations are
those of the kernels (positive, and together no longer than the stream time around them), results
do not depend on whether the timers are on, and a reset starts from zero."""
import numpy as np
import pytest

from breccia_amd import lib as L
from breccia_amd.kv import Event, Stream
from gpu_common import Twin, check_attn
from test_gpu_attn import fill

pytestmark = pytest.mark.gpu

STAGES = (L.STAGE_APPEND, L.STAGE_ATTN_SPLIT, L.STAGE_ATTN_MERGE, L.STAGE_PAGE_COPY)


def read_all(pool):
    return {s: pool.timing_read(s) for s in STAGES}


def test_timers_count_each_stage_and_leave_results_alone():
    rng = np.random.Generator(np.random.PCG64(4711))
    with Twin(n_pages=256, max_seqs=4) as tw:
        st = Stream()
        a, b = tw.pool.seq_create(), tw.pool.seq_create()
        fill(tw, a, 1500, rng)
        fill(tw, b, 333, rng)
        q = rng.standard_normal((2, 16, 256)).astype(np.float32)
        pos = [1499, 332]
        plain = tw.decode_attn(0, [a, b], pos, q, 16, stream=st)
        # off: nothing is counted
        assert all(n == 0 and ms == 0.0 for n, ms in read_all(tw.pool).values())

        tw.pool.timing_enable(True)
        e0, e1 = Event(), Event()
        e0.record(st)
        timed = tw.decode_attn(0, [a, b], pos, q, 16, stream=st)
        k = rng.standard_normal((7, 2, 256)).astype(np.float32)
        tw.pool.seq_reserve(a, 1507)
        tw.append(0, [a], [1500], [k], [k], stream=st)
        free = [p for p in range(256) if tw.pool.page_refcount(p) == 0][:3]
        pairs = [(int(tw.pool.block_table(a)[i]), free[i]) for i in range(3)]
        tw.pool.page_copy(pairs, st)
        for img in tw.images:
            img.page_copy(pairs)
        e1.record(st)
        st.sync()
        wall = e0.elapsed_ms(e1)
        tw.pool.timing_enable(False)
        got = read_all(tw.pool)
        assert got[L.STAGE_ATTN_SPLIT][0] == 1 and got[L.STAGE_ATTN_MERGE][0] == 1
        assert got[L.STAGE_APPEND][0] == 1 and got[L.STAGE_PAGE_COPY][0] == 1
        total = sum(ms for _, ms in got.values())
        assert all(ms > 0.0 for _, ms in got.values())
        assert total < wall, "kernels %.4f ms, stream time around them %.4f ms" % (total, wall)
        # the same bytes with the timers on or off, and both are the oracle's answer
        assert np.array_equal(plain.view(np.uint32), timed.view(np.uint32))
        for i, s in enumerate([a, b]):
            check_attn(timed[i], tw.oracle_attend(0, s, pos[i], q[i], 16), "seq %d" % s)
        tw.assert_pools_equal()

        # off again: later launches are not counted; a reset starts from zero
        tw.decode_attn(0, [a, b], pos, q, 16, stream=st)
        assert read_all(tw.pool) == got
        tw.pool.timing_reset()
        assert all(n == 0 and ms == 0.0 for n, ms in read_all(tw.pool).values())

        # many launches in one session, read while still enabled
        tw.pool.timing_enable(True)
        for _ in range(50):
            tw.decode_attn(0, [a, b], pos, q, 16, stream=st)
        n, ms = tw.pool.timing_read(L.STAGE_ATTN_SPLIT)
        assert n == 50 and 0.0 < ms / n < 1.0
        tw.pool.timing_enable(False)
        e0.close()
        e1.close()
        st.close()


def test_every_kernel_of_the_path_has_a_stage_timer():
    """Chunk attention, the fused K preparation, the selection kernels and the page staging of a swap
    report under stages of their own (the reference stamps every stage of a layer,
    crates/breccia-kernels/src/qsa/mod.rs:1733-1970)."""
    from breccia_amd.kv import DeviceBuffer, device_sync, rope_table

    rng = np.random.Generator(np.random.PCG64(4712))
    with Twin(n_pages=64, max_seqs=4) as tw:
        pool = tw.pool
        s = pool.seq_create()
        fill(tw, s, 300, rng)
        pool.timing_enable(True)
        q = DeviceBuffer.from_numpy(rng.standard_normal((40, 16, 256)).astype(np.float32))
        out = DeviceBuffer(40 * 16 * 256 * 4)
        pool.prefill_attn(0, [s], [260], [40], 16, q, out, 1.0 / 16.0)
        pool.seq_reserve(s, 305)
        kv = DeviceBuffer.from_numpy(rng.standard_normal((5, 2, 256)).astype(np.float32))
        gamma = DeviceBuffer.from_numpy(np.ones(256, dtype=np.float32))
        table = DeviceBuffer.from_numpy(rope_table(1e7, 64, 512))
        pool.append_kprep(0, [s], [300], [5], kv, kv, gamma, 1e-6, table, 64, 512)
        pooled = DeviceBuffer.from_numpy(rng.standard_normal((75, 128)).astype(np.float32))
        iq = DeviceBuffer.from_numpy(rng.standard_normal((1, 4, 128)).astype(np.float32))
        ids, counts = DeviceBuffer(64 * 4), DeviceBuffer(16)
        pool.select_blocks([299], iq, [pooled], [75], 4, 128, 16, ids, 64, counts, 64)
        tail = DeviceBuffer(3 * 128 * 4)
        raw = DeviceBuffer.from_numpy(rng.standard_normal((9, 128)).astype(np.float32))
        g128 = DeviceBuffer.from_numpy(np.ones(128, dtype=np.float32))
        pool.idx_pool(pooled, 75, tail, raw, 0, 9, g128, 1e-6, table, 64, 512, 128)
        host = pool.host_alloc(2 * pool.swap_page_bytes())
        pool.swap_out(pool.block_table(s)[:2], host)
        pool.swap_wait()
        device_sync()
        pool.timing_enable(False)
        want = {L.STAGE_PREFILL_ATTN: 1, L.STAGE_APPEND_KPREP: 1, L.STAGE_IDX_SCORE: 1, L.STAGE_TOPK: 1,
                L.STAGE_IDX_POOL: 2, L.STAGE_PAGE_STAGE: 1, L.STAGE_APPEND: 0, L.STAGE_ATTN_SPLIT: 0}
        for stage, n_want in want.items():
            n, ms = pool.timing_read(stage)
            assert n == n_want, (stage, n)
            assert (ms > 0.0) == (n_want > 0) and ms < 5.0, (stage, ms)
        host.free()
        for b in (q, out, kv, gamma, table, pooled, iq, ids, counts, tail, raw, g128):
            b.free()


def test_read_probe_accepts_whole_power_of_two_chunk_counts_only():
    import ctypes as C

    from breccia_amd.kv import BkvError, DeviceBuffer, check, device_sync, lib

    buf, sink = DeviceBuffer(1 << 20), DeviceBuffer(16)
    for scattered in (0, 1, 2):
        check(lib.bkv_read_probe(buf.ptr, 1 << 20, scattered, sink.ptr, None))
    check(lib.bkv_read_probe(buf.ptr, 8192, 2, sink.ptr, None))
    for bad_order in (-1, 3):
        with pytest.raises(BkvError) as ei:
            check(lib.bkv_read_probe(buf.ptr, 1 << 20, bad_order, sink.ptr, None))
        assert ei.value.status == L.ERR_INVALID
    check(lib.bkv_read_probe(buf.ptr, 8192, 1, sink.ptr, None))
    device_sync()
    for bad in (0, 8191, 3 * 8192, (1 << 20) + 16):
        with pytest.raises(BkvError) as ei:
            check(lib.bkv_read_probe(buf.ptr, bad, 0, sink.ptr, None))
        assert ei.value.status == L.ERR_INVALID
    with pytest.raises(BkvError):
        check(lib.bkv_read_probe(None, 8192, 0, sink.ptr, None))
    buf.free()
    sink.free()
