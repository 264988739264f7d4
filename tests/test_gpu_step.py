"""The fused decode step (append one token per sequence + attention in one launch) against the
two-call sequence bkv_append -> bkv_decode_attn: identical pool bytes, bit-identical outputs,
and the usual tolerance against the oracle."""
import numpy as np
import pytest

from breccia_amd import lib as L
from breccia_amd.kv import BkvError, DeviceBuffer, device_sync
from gpu_common import REF_BAR_MAX_REL, Twin, check_attn
from test_gpu_attn import fill

pytestmark = pytest.mark.gpu


def step(tw, layer, seqs, pos, k_new, v_new, q, n_head, gate=None):
    n = len(seqs)
    kd, vd = DeviceBuffer.from_numpy(k_new), DeviceBuffer.from_numpy(v_new)
    qd, od = DeviceBuffer.from_numpy(q), DeviceBuffer(q.nbytes)
    gd = None if gate is None else DeviceBuffer.from_numpy(gate)
    try:
        tw.pool.decode_step(layer, seqs, pos, kd, vd, n_head, qd, od, 1.0 / 16.0, gate_dev=gd,
                            gate_seq_stride=n_head * 256 if gd else 0, gate_head_stride=256 if gd else 0)
        return od.download(np.float32, q.size).reshape(n, n_head, 256)
    finally:
        for b in (kd, vd, qd, od, gd):
            if b is not None:
                b.free()


@pytest.mark.parametrize("layout", [L.LAYOUT_F16, L.LAYOUT_Q8V, L.LAYOUT_I8H])
@pytest.mark.parametrize("n_q", [16, 24])
def test_fused_step_equals_append_then_attend(n_q, layout):
    rng = np.random.Generator(np.random.PCG64(800 + n_q + 7 * layout))
    lens = [37, 512, 1000, 2048, 15, 16, 1, 0, 4099]      # page edges, an empty sequence, long
    with Twin(n_pages=700, max_seqs=24, layout=layout) as tw:
        tw.pool.set_free_order(rng.permutation(700).astype(np.int32))
        fused = [tw.pool.seq_create() for _ in lens]
        for s, n in zip(fused, lens):
            if n:
                fill(tw, s, n, rng, chunk=1024)
        twocall = [tw.pool.seq_fork(s, n) for s, n in zip(fused, lens)]   # same contents, shared pages
        for t in range(3):                                   # three consecutive decode steps
            pos = [n + t for n in lens]
            k_new = rng.standard_normal((len(lens), 2, 256)).astype(np.float32)
            v_new = rng.standard_normal((len(lens), 2, 256)).astype(np.float32)
            k_new[0, 0, :4] = [1e-6, -1e-9, np.nan, 7e4]     # the store rule's special cases
            v_new[1, 1, 32:64] = 0.0                           # an all-zero block (scale 1 by rule)
            v_new[2, 0, 64:96] *= 1e-7                         # a block whose f16 scale would flush
            q = rng.standard_normal((len(lens), n_q, 256)).astype(np.float32)
            gate = rng.standard_normal((len(lens), n_q, 256)).astype(np.float32)
            # two calls on the forks (copy-on-write where a shared partial page is written)
            for s, p in zip(twocall, pos):
                pairs = tw.pool.seq_reserve(s, p + 1)
                if pairs:
                    tw.pool.page_copy(pairs)
                    for img in tw.images:
                        img.page_copy(pairs)
            tw.append(0, twocall, pos, list(k_new[:, None]), list(v_new[:, None]))
            want = tw.decode_attn(0, twocall, pos, q, n_q, scale=1.0 / 16.0, gate=gate)
            # one call on the originals
            for s, p in zip(fused, pos):
                pairs = tw.pool.seq_reserve(s, p + 1)
                if pairs:
                    tw.pool.page_copy(pairs)
                    for img in tw.images:
                        img.page_copy(pairs)
            got = step(tw, 0, fused, pos, k_new, v_new, q, n_q, gate=gate)
            device_sync()
            for s, p, k1, v1 in zip(fused, pos, k_new, v_new):   # the oracle image follows the pool
                tw.images[0].append(tw.pool.block_table(s), p, k1, v1, capacity_cells=tw.pool.seq_capacity(s))
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), "step %d" % t
            tw.assert_pools_equal()
            if t == 0:
                finite = [i for i in range(len(lens)) if i != 0]   # entry 0 holds a NaN-derived inf
                for i in finite[:4]:
                    w = tw.oracle_attend(0, fused[i], pos[i], q[i], n_q, gate=gate[i])
                    _, rel = check_attn(got[i], w, "entry %d" % i)
                    assert rel <= REF_BAR_MAX_REL
        tw.pool.check()


def test_step_errors_come_before_any_launch():
    with Twin(n_pages=16, max_seqs=4) as tw:
        s = tw.pool.seq_create()
        tw.pool.seq_reserve(s, 20)
        z = DeviceBuffer(1 << 16)
        before = tw.pool.read_layer(0, 0).copy()
        for kw, status in [(dict(seqs=[s, s], pos=[19, 19]), L.ERR_INVALID), (dict(k_new_dev=None), L.ERR_INVALID),
                           (dict(pos=[32]), L.ERR_RANGE), (dict(n_q_head=15), L.ERR_INVALID)]:
            a = dict(layer=0, seqs=[s], pos=[19], k_new_dev=z, v_new_dev=z, n_q_head=16, q_dev=z, out_dev=z,
                     scale=0.0625)
            a.update(kw)
            with pytest.raises(BkvError) as ei:
                tw.pool.decode_step(**a)
            assert ei.value.status == status, kw
        device_sync()
        assert np.array_equal(before, tw.pool.read_layer(0, 0))
        z.free()
    with Twin(n_pages=16, max_seqs=4, layout=L.LAYOUT_I8H) as tw:
        # 24 q heads per kv head are beyond what the kernels take
        s = tw.pool.seq_create()
        tw.pool.seq_reserve(s, 20)
        z = DeviceBuffer(1 << 18)
        with pytest.raises(BkvError) as ei:
            tw.pool.decode_step(0, [s], [19], z, z, 48, z, z, 0.0625)
        assert ei.value.status == L.ERR_INVALID
        z.free()
