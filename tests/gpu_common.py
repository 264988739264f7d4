"""Plumbing shared by the GPU parity tests: a device pool and the oracle's host image of
the same pool, driven with identical inputs."""
import numpy as np

import oracle
from breccia_amd import lib as L
from breccia_amd.kv import DeviceBuffer, Pool

ORACLE_LAYOUT = {L.LAYOUT_F16: oracle.LAYOUT_F16, L.LAYOUT_Q8V: oracle.LAYOUT_Q8V,
                 L.LAYOUT_I8H: oracle.LAYOUT_I8H}

# north_star tolerance for f16-input / f32-accumulate attention, checked against the f64 oracle
ATTN_MAX_ABS = 2e-3
ATTN_MAX_REL = 1e-3
# the reference's own bar (crates/breccia-kernels/tests/attn_conformance.rs:1148-1151)
REF_BAR_MAX_REL = 1e-5


class Twin:
    """A device pool plus one oracle PoolImage per layer, kept in step."""

    def __init__(self, n_layers=1, n_pages=512, n_kv=2, hd=256, layout=L.LAYOUT_F16, max_seqs=16,
                 max_pages_per_seq=None):
        self.pool = Pool(n_layers=n_layers, n_pages=n_pages, n_kv_head=n_kv, head_dim=hd,
                         layout=layout, max_seqs=max_seqs, max_pages_per_seq=max_pages_per_seq)
        self.g = oracle.Geom(n_kv, hd, 16)
        self.layout = layout
        self.images = [oracle.PoolImage(self.g, n_pages, ORACLE_LAYOUT[layout]) for _ in range(n_layers)]

    def close(self):
        self.pool.destroy()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def append(self, layer, seqs, pos0, k_list, v_list, stream=None, f16_rows=False):
        """k_list[i], v_list[i]: float32 [T_i, n_kv, hd] -- or raw binary16 codes (uint16) of the
        same shape when f16_rows is set, which go through bkv_append_f16 on the device and,
        widened under the cache's load rule, through the same oracle append.  Appends on the
        device (one call) and in the oracle image."""
        dt = np.uint16 if f16_rows else np.float32
        n_tok = [int(np.asarray(k).reshape(-1, self.g.n_kv, self.g.head_dim).shape[0]) for k in k_list]
        if sum(n_tok):
            kcat = np.concatenate([np.asarray(k, dtype=dt).reshape(-1) for k in k_list])
            vcat = np.concatenate([np.asarray(v, dtype=dt).reshape(-1) for v in v_list])
        else:
            kcat = vcat = np.zeros(8, dtype=dt)
        kd, vd = DeviceBuffer.from_numpy(kcat), DeviceBuffer.from_numpy(vcat)
        try:
            self.pool.append(layer, seqs, pos0, n_tok, kd, vd, stream, f16_rows=f16_rows)
            if stream is not None:
                stream.sync()
            else:
                from breccia_amd.kv import device_sync
                device_sync()
        finally:
            kd.free()
            vd.free()
        for s, p0, k, v, t in zip(seqs, pos0, k_list, v_list, n_tok):
            if t:
                if f16_rows:
                    k = oracle.f16_bits_to_f32(np.asarray(k, dtype=np.uint16).reshape(-1))
                    v = oracle.f16_bits_to_f32(np.asarray(v, dtype=np.uint16).reshape(-1))
                rc = self.images[layer].append(self.pool.block_table(s), p0, k, v,
                                               capacity_cells=self.pool.seq_capacity(s))
                assert rc == 0

    def assert_pools_equal(self, layer=0):
        gk = self.pool.read_layer(layer, 0)
        gv = self.pool.read_layer(layer, 1)
        img = self.images[layer]
        bad_k = np.nonzero(gk != img.k)[0]
        bad_v = np.nonzero(gv != img.v)[0]
        assert bad_k.size == 0, "K pool differs at %d bytes, first at byte %d" % (bad_k.size, bad_k[0])
        assert bad_v.size == 0, "V pool differs at %d bytes, first at byte %d" % (bad_v.size, bad_v[0])

    def oracle_attend(self, layer, seq, pos, q, n_head, gate=None, threads=4):
        table = self.pool.block_table(seq)
        k, v = self.images[layer].gather(table, 0, pos + 1)
        return oracle.attend(q, k, v, oracle.dense_cells(pos), pos, n_head, self.g.n_kv,
                             self.g.head_dim, gate=gate, threads=threads)

    def decode_attn(self, layer, seqs, pos, q, n_head, scale=None, gate=None, gate_strides=None,
                    stream=None):
        """q: float32 [n, n_head, hd] -> out float32 [n, n_head, hd]."""
        q = np.ascontiguousarray(q, dtype=np.float32)
        n = len(seqs)
        qd = DeviceBuffer.from_numpy(q)
        od = DeviceBuffer(max(q.nbytes, 16))
        gd = None
        try:
            ss = hs = 0
            if gate is not None:
                gate = np.ascontiguousarray(gate, dtype=np.float32)
                gd = DeviceBuffer.from_numpy(gate)
                ss, hs = gate_strides if gate_strides else (n_head * self.g.head_dim, self.g.head_dim)
            if scale is None:
                scale = 1.0 / np.sqrt(self.g.head_dim)
            self.pool.decode_attn(layer, seqs, pos, n_head, qd, od, float(scale), gate_dev=gd,
                                  gate_seq_stride=ss, gate_head_stride=hs, stream=stream)
            out = od.download(np.float32, q.size, stream).reshape(n, n_head, self.g.head_dim)
        finally:
            qd.free()
            od.free()
            if gd is not None:
                gd.free()
        return out


def check_attn(got, want, what=""):
    """north_star tolerance; returns (max_abs, max_rel) so callers can also report the stricter
    reference bar."""
    from helpers import max_abs, max_rel
    a, r = max_abs(got, want), max_rel(got, want)
    assert np.all(np.isfinite(got)), what + ": non-finite output"
    assert a <= ATTN_MAX_ABS, "%s: max abs error %.3e > %.1e" % (what, a, ATTN_MAX_ABS)
    assert r <= ATTN_MAX_REL, "%s: max rel error %.3e > %.1e" % (what, r, ATTN_MAX_REL)
    return a, r
