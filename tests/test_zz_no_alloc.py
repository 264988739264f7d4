"""bkv_decode_attn_static: decode attention whose split-K partials live in the library's static
device array instead of a workspace the pool allocated.  Checked through the C ABI against
bkv_decode_attn (same kernels and cut, so bit for bit) and against the oracle, on two calls in a
row, the second with a smaller batch, so that what the first call left in the array is there when
the second one runs."""
import numpy as np
import pytest

from breccia_amd import lib as L
from breccia_amd.kv import BkvError, DeviceBuffer, Graph, Stream, device_mem_free, device_sync
from gpu_common import REF_BAR_MAX_REL, Twin, check_attn

pytestmark = pytest.mark.gpu


def _both(tw, seqs, pos, q, n_q, gate=None):
    """(bkv_decode_attn, bkv_decode_attn_static) outputs for one batch."""
    n = len(seqs)
    qd = DeviceBuffer.from_numpy(q)
    gd = DeviceBuffer.from_numpy(gate) if gate is not None else None
    o_ref, o_static = DeviceBuffer(q.nbytes), DeviceBuffer(q.nbytes)
    ss, hs = (n_q * 256, 256) if gate is not None else (0, 0)
    try:
        tw.pool.decode_attn(0, seqs, pos, n_q, qd, o_ref, 1.0 / 16.0, gate_dev=gd, gate_seq_stride=ss,
                            gate_head_stride=hs)
        tw.pool.decode_attn_static(0, seqs, pos, n_q, qd, o_static, 1.0 / 16.0, gate_dev=gd, gate_seq_stride=ss,
                                   gate_head_stride=hs)
        device_sync()
        return (o_ref.download(np.float32).reshape(n, n_q, 256), o_static.download(np.float32).reshape(n, n_q, 256))
    finally:
        for b in (qd, gd, o_ref, o_static):
            if b is not None:
                b.free()


@pytest.mark.parametrize("layout", [L.LAYOUT_F16, L.LAYOUT_Q8V, L.LAYOUT_I8H])
def test_static_scratch_call_equals_the_allocating_call_twice_in_a_row(layout):
    rng = np.random.Generator(np.random.PCG64(7100 + layout))
    n_kv, n_q = 2, 16
    lens = [1500, 37, 700, 2048, 16, 333]
    with Twin(n_pages=400, n_kv=n_kv, layout=layout, max_seqs=8) as tw:
        tw.pool.set_free_order(rng.permutation(400).astype(np.int32))
        seqs = [tw.pool.seq_create() for _ in lens]
        for s, n in zip(seqs, lens):
            tw.pool.seq_reserve(s, n)
        ks = [rng.standard_normal((n, n_kv, 256)).astype(np.float32) for n in lens]
        vs = [rng.standard_normal((n, n_kv, 256)).astype(np.float32) for n in lens]
        tw.append(0, seqs, [0] * len(lens), ks, vs)

        # first call: the whole batch, with a gate
        pos = [n - 1 for n in lens]
        q = rng.standard_normal((len(lens), n_q, 256)).astype(np.float32)
        gate = rng.standard_normal((len(lens), n_q, 256)).astype(np.float32)
        ref, got = _both(tw, seqs, pos, q, n_q, gate)
        assert np.array_equal(ref.view(np.uint32), got.view(np.uint32))
        for i in range(len(lens)):
            _, rel = check_attn(got[i], tw.oracle_attend(0, seqs[i], pos[i], q[i], n_q, gate=gate[i]), "first call, entry %d" % i)
            assert rel <= REF_BAR_MAX_REL, (i, rel)

        # second call, smaller: two of the sequences at earlier positions, fewer work-groups, so most
        # of what the first call wrote is still in the array
        seqs2, pos2 = [seqs[2], seqs[0]], [100, 799]
        q2 = rng.standard_normal((2, n_q, 256)).astype(np.float32)
        ref2, got2 = _both(tw, seqs2, pos2, q2, n_q)
        assert np.array_equal(ref2.view(np.uint32), got2.view(np.uint32))
        for i in range(2):
            _, rel = check_attn(got2[i], tw.oracle_attend(0, seqs2[i], pos2[i], q2[i], n_q), "second call, entry %d" % i)
            assert rel <= REF_BAR_MAX_REL, (i, rel)


def test_static_scratch_call_rejects_batches_beyond_the_array():
    # 9 kv heads x 16 q heads each: a work-group writes 16 head rows, so the array serves
    # 1024 * 8 / 16 = 512 work-groups; 64 entries need at least 64 * 9 = 576.
    n_kv, n_q = 9, 144
    with Twin(n_pages=64, n_kv=n_kv, max_seqs=64, max_pages_per_seq=2) as tw:
        seqs = [tw.pool.seq_create() for _ in range(64)]
        for s in seqs:
            tw.pool.seq_reserve(s, 5)
        qd = DeviceBuffer(64 * n_q * 256 * 4)
        od = DeviceBuffer(64 * n_q * 256 * 4)
        with pytest.raises(BkvError) as ei:
            tw.pool.decode_attn_static(0, seqs, [4] * 64, n_q, qd, od, 1.0 / 16.0)
        assert ei.value.status == L.ERR_INVALID and "static scratch" in ei.value.message
        # 56 entries fit (504 work-groups)
        tw.pool.decode_attn_static(0, seqs[:56], [4] * 56, n_q, qd, od, 1.0 / 16.0)
        device_sync()
        qd.free()
        od.free()


def test_static_scratch_call_allocates_nothing_and_replays_from_a_graph():
    # What the entry point is for: callers that cannot allocate.  Free device memory is the same
    # before and after a run of calls (the allocating entry point's workspace was made at pool
    # creation, so it serves as the control), and the call can be recorded into a graph: three
    # replays, with eager work on the same pool and a synchronisation between them, each return the
    # bits of the eager call on that replay's inputs.  Block-table changes pending at capture time
    # are refused, as for step plans.
    rng = np.random.Generator(np.random.PCG64(7200))
    n_q, lens = 16, [900, 41, 2047]
    st = Stream()
    with Twin(n_pages=300, max_seqs=8) as tw:
        tw.pool.set_free_order(rng.permutation(300).astype(np.int32))
        seqs = [tw.pool.seq_create() for _ in lens]
        for s, n in zip(seqs, lens):
            tw.pool.seq_reserve(s, n)
        tw.append(0, seqs, [0] * 3, [rng.standard_normal((n, 2, 256)).astype(np.float32) for n in lens],
                  [rng.standard_normal((n, 2, 256)).astype(np.float32) for n in lens])
        pos = [n - 1 for n in lens]
        qd = DeviceBuffer(3 * n_q * 256 * 4)
        o_static, o_ref = DeviceBuffer(3 * n_q * 256 * 4), DeviceBuffer(3 * n_q * 256 * 4)
        qd.upload(rng.standard_normal((3, n_q, 256)).astype(np.float32))
        tw.pool.decode_attn_static(0, seqs, pos, n_q, qd, o_static, 1.0 / 16.0, stream=st)
        st.sync()
        free0 = device_mem_free()
        for _ in range(50):
            tw.pool.decode_attn_static(0, seqs, pos, n_q, qd, o_static, 1.0 / 16.0, stream=st)
        st.sync()
        assert device_mem_free() == free0
        # pending table changes at capture time: refused, and the capture can go on after an eager flush
        extra = tw.pool.seq_create()
        tw.pool.seq_reserve(extra, 20)
        g = Graph(st)
        with pytest.raises(BkvError) as ei:
            tw.pool.decode_attn_static(0, seqs, pos, n_q, qd, o_static, 1.0 / 16.0, stream=st)
        assert ei.value.status == L.ERR_STATE and "captured" in ei.value.message
        g.end()
        g.destroy()
        tw.pool.decode_attn(0, seqs, pos, n_q, qd, o_ref, 1.0 / 16.0, stream=st)    # eager: flushes the tables
        st.sync()
        g = Graph(st)
        tw.pool.decode_attn_static(0, seqs, pos, n_q, qd, o_static, 1.0 / 16.0, stream=st)
        g.end()
        free1 = None
        for rep in range(3):
            q = rng.standard_normal((3, n_q, 256)).astype(np.float32)
            qd.upload(q, st)
            tw.pool.decode_attn(0, seqs, pos, n_q, qd, o_ref, 1.0 / 16.0, stream=st)      # eager work in between
            st.sync()
            g.launch(st)
            st.sync()
            got = o_static.download(np.float32, stream=st)
            want = o_ref.download(np.float32, stream=st)
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), rep
            if free1 is None:
                # instantiating a graph and launching it for the first time take device memory of the
                # runtime's own; from then on nothing moves
                free1 = device_mem_free()
        assert device_mem_free() == free1
        g.destroy()
        for b in (qd, o_static, o_ref):
            b.free()
