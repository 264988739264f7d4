"""Thin Python host layer over the C ABI: device buffers, streams, events and the pool.

Everything numerical happens in libbreccia_kv.so; this module only marshals numpy
arrays and integers into the C calls and turns status codes into exceptions.
"""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

from . import lib as L
from .lib import BkvError, PagePair, PoolDesc, check, lib  # noqa: F401


def _i32(a):
    a = np.ascontiguousarray(a, dtype=np.int32)
    return a, a.ctypes.data_as(C.POINTER(C.c_int32))


def _i64(a):
    a = np.ascontiguousarray(a, dtype=np.int64)
    return a, a.ctypes.data_as(C.POINTER(C.c_int64))


class Stream:
    def __init__(self):
        h = C.c_void_p()
        check(lib.bkv_stream_create(C.byref(h)))
        self.handle = h

    def sync(self) -> None:
        check(lib.bkv_stream_sync(self.handle))

    def wait(self, timeout_ms: int) -> None:
        """The library's bounded wait (bkv_stream_wait): BkvError with ERR_TIMEOUT past the deadline."""
        check(lib.bkv_stream_wait(self.handle, timeout_ms))

    def close(self) -> None:
        if self.handle:
            check(lib.bkv_stream_destroy(self.handle))
            self.handle = None


class Event:
    def __init__(self):
        h = C.c_void_p()
        check(lib.bkv_event_create(C.byref(h)))
        self.handle = h

    def record(self, stream=None) -> None:
        check(lib.bkv_event_record(self.handle, _sh(stream)))

    def sync(self) -> None:
        check(lib.bkv_event_sync(self.handle))

    def elapsed_ms(self, stop: "Event") -> float:
        ms = C.c_float()
        check(lib.bkv_event_elapsed_ms(self.handle, stop.handle, C.byref(ms)))
        return float(ms.value)

    def close(self) -> None:
        if self.handle:
            check(lib.bkv_event_destroy(self.handle))
            self.handle = None


def _sh(stream):
    return stream.handle if isinstance(stream, Stream) else stream


def rope_table(freq_base: float, n_rot: int, max_pos: int) -> np.ndarray:
    """float32 [max_pos, n_rot/2, 2] of (cos, sin), built by the library on the host."""
    out = np.empty((max_pos, max(n_rot // 2, 1), 2), dtype=np.float32)
    check(lib.bkv_rope_table(freq_base, n_rot, max_pos, out.ctypes.data))
    return out


def attn_plan(n_cu: int, n_kv_head: int, n_q_head: int, pos, sel_groups: int = 0):
    """How the library would cut a decode-attention batch into work-groups on a device of n_cu
    compute units -> (splits per entry, pages per split, total work-groups).  Host only."""
    pos, pp = _i64(pos)
    splits = np.zeros(max(pos.size, 1), dtype=np.int32)
    pps = np.zeros(max(pos.size, 1), dtype=np.int32)
    total = C.c_int32()
    check(lib.bkv_attn_plan(n_cu, n_kv_head, n_q_head, pos.size, pp, sel_groups,
                            splits.ctypes.data_as(C.POINTER(C.c_int32)), pps.ctypes.data_as(C.POINTER(C.c_int32)),
                            C.byref(total)))
    return splits[:pos.size], pps[:pos.size], int(total.value)


def wait_options(timeout_ms: int | None = None, poll_us: int | None = None):
    """Set (where given) and return the process-wide (deadline in ms, spin window in us) of the library's waits."""
    t, p = C.c_int64(), C.c_int64()
    check(lib.bkv_wait_options_get(C.byref(t), C.byref(p)))
    if timeout_ms is not None or poll_us is not None:
        check(lib.bkv_wait_options(t.value if timeout_ms is None else timeout_ms,
                                   p.value if poll_us is None else poll_us))
        check(lib.bkv_wait_options_get(C.byref(t), C.byref(p)))
    return int(t.value), int(p.value)


def device_sync() -> None:
    check(lib.bkv_device_sync())


def device_info():
    name = C.create_string_buffer(256)
    cu = C.c_int32()
    mem = C.c_uint64()
    check(lib.bkv_device_info(name, 256, C.byref(cu), C.byref(mem)))
    return name.value.decode(), int(cu.value), int(mem.value)


def device_mem_free() -> int:
    f = C.c_uint64()
    check(lib.bkv_device_mem_info(C.byref(f), None))
    return int(f.value)


class DeviceBuffer:
    """A hipMalloc'd region with numpy upload/download."""

    def __init__(self, nbytes: int):
        self.nbytes = int(nbytes)
        p = C.c_void_p()
        check(lib.bkv_dev_alloc(self.nbytes, C.byref(p)))
        self.ptr = p

    @classmethod
    def from_numpy(cls, a: np.ndarray, stream=None) -> "DeviceBuffer":
        a = np.ascontiguousarray(a)
        buf = cls(max(a.nbytes, 16))
        buf.upload(a, stream)
        return buf

    def upload(self, a: np.ndarray, stream=None, offset: int = 0) -> None:
        a = np.ascontiguousarray(a)
        assert offset + a.nbytes <= self.nbytes
        if a.nbytes == 0:
            return
        check(lib.bkv_memcpy_h2d(C.c_void_p(self.ptr.value + offset), a.ctypes.data, a.nbytes,
                                 _sh(stream)))
        check(lib.bkv_stream_sync(_sh(stream)))

    def download(self, dtype, count: int | None = None, stream=None, offset: int = 0) -> np.ndarray:
        dt = np.dtype(dtype)
        if count is None:
            count = (self.nbytes - offset) // dt.itemsize
        out = np.empty(count, dtype=dt)
        if out.nbytes:
            assert offset + out.nbytes <= self.nbytes
            check(lib.bkv_memcpy_d2h(out.ctypes.data, C.c_void_p(self.ptr.value + offset),
                                     out.nbytes, _sh(stream)))
            check(lib.bkv_stream_sync(_sh(stream)))
        return out

    def at(self, offset: int) -> C.c_void_p:
        return C.c_void_p(self.ptr.value + offset)

    def free(self) -> None:
        if self.ptr:
            check(lib.bkv_dev_free(self.ptr))
            self.ptr = None


class Pool:
    """bkv_pool handle.  Method names follow the C entry points."""

    def __init__(self, n_layers=1, n_pages=512, n_kv_head=2, head_dim=256, page_cells=16,
                 layout=L.LAYOUT_F16, max_seqs=16, max_pages_per_seq=None, host_only=False):
        if max_pages_per_seq is None:
            max_pages_per_seq = n_pages
        flags = L.POOL_HOST_ONLY if host_only else 0
        self.desc = PoolDesc(n_layers, n_pages, n_kv_head, head_dim, page_cells, layout, max_seqs,
                             max_pages_per_seq, flags)
        h = C.c_void_p()
        check(lib.bkv_pool_create(C.byref(self.desc), C.byref(h)))
        self.handle = h

    # -- lifecycle
    def destroy(self) -> None:
        if self.handle:
            check(lib.bkv_pool_destroy(self.handle))
            self.handle = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.destroy()

    def reset(self, stream=None) -> None:
        check(lib.bkv_pool_reset(self.handle, _sh(stream)))

    def fill(self, byte: int, stream=None) -> None:
        check(lib.bkv_pool_fill(self.handle, byte, _sh(stream)))

    def bytes(self) -> int:
        return int(lib.bkv_pool_bytes(self.handle))

    def page_bytes(self, which: int) -> int:
        return int(lib.bkv_page_bytes(self.handle, which))

    def swap_page_bytes(self) -> int:
        return int(lib.bkv_swap_page_bytes(self.handle))

    def layer_ptr(self, layer: int, which: int):
        p = C.c_void_p()
        n = C.c_uint64()
        check(lib.bkv_pool_layer_ptr(self.handle, layer, which, C.byref(p), C.byref(n)))
        return p, int(n.value)

    def read_layer(self, layer: int, which: int, stream=None) -> np.ndarray:
        """Bytes of one layer's K (0) or V (1) pool."""
        p, n = self.layer_ptr(layer, which)
        out = np.empty(n, dtype=np.uint8)
        check(lib.bkv_memcpy_d2h(out.ctypes.data, p, n, _sh(stream)))
        check(lib.bkv_stream_sync(_sh(stream)))
        return out

    def write_layer(self, layer: int, which: int, data: np.ndarray, stream=None) -> None:
        p, n = self.layer_ptr(layer, which)
        data = np.ascontiguousarray(data).view(np.uint8).reshape(-1)
        assert data.nbytes == n
        check(lib.bkv_memcpy_h2d(p, data.ctypes.data, n, _sh(stream)))
        check(lib.bkv_stream_sync(_sh(stream)))

    # -- allocator
    def seq_create(self) -> int:
        s = C.c_int32()
        check(lib.bkv_seq_create(self.handle, C.byref(s)))
        return int(s.value)

    def seq_create_identity(self, n_pages: int) -> int:
        s = C.c_int32()
        check(lib.bkv_seq_create_identity(self.handle, n_pages, C.byref(s)))
        return int(s.value)

    def seq_fork(self, parent: int, n_tokens: int) -> int:
        s = C.c_int32()
        check(lib.bkv_seq_fork(self.handle, parent, n_tokens, C.byref(s)))
        return int(s.value)

    def seq_free(self, seq: int) -> None:
        check(lib.bkv_seq_free(self.handle, seq))

    def seq_reserve(self, seq: int, new_len: int, cow_capacity: int = 4):
        """Returns the list of (src, dst) copy-on-write pairs the caller must page_copy."""
        pairs = (PagePair * max(cow_capacity, 1))()
        n = C.c_int32()
        check(lib.bkv_seq_reserve(self.handle, seq, new_len, pairs, cow_capacity, C.byref(n)))
        return [(pairs[i].src, pairs[i].dst) for i in range(n.value)]

    def seq_truncate(self, seq: int, new_len: int) -> None:
        check(lib.bkv_seq_truncate(self.handle, seq, new_len))

    def seq_len(self, seq: int) -> int:
        return int(lib.bkv_seq_len(self.handle, seq))

    def seq_capacity(self, seq: int) -> int:
        return int(lib.bkv_seq_capacity(self.handle, seq))

    def seq_n_pages(self, seq: int) -> int:
        return int(lib.bkv_seq_n_pages(self.handle, seq))

    def block_table(self, seq: int) -> np.ndarray:
        n = self.seq_n_pages(seq)
        if n < 0:
            raise BkvError(L.ERR_RANGE, "sequence %d is not live" % seq)
        p = lib.bkv_seq_block_table(self.handle, seq)
        return np.ctypeslib.as_array(p, shape=(max(n, 1),))[:n].copy()

    def page_refcount(self, page: int) -> int:
        return int(lib.bkv_page_refcount(self.handle, page))

    def free_pages(self) -> int:
        return int(lib.bkv_pool_free_pages(self.handle))

    def check(self) -> None:
        check(lib.bkv_pool_check(self.handle))

    def set_free_order(self, order) -> None:
        order, po = _i32(order)
        check(lib.bkv_pool_set_free_order(self.handle, po, order.size))

    # -- per-kernel timing
    def timing_enable(self, on: bool) -> None:
        check(lib.bkv_timing_enable(self.handle, 1 if on else 0))

    def timing_reset(self) -> None:
        check(lib.bkv_timing_reset(self.handle))

    def timing_read(self, stage: int):
        n = C.c_uint64()
        ms = C.c_double()
        check(lib.bkv_timing_read(self.handle, stage, C.byref(n), C.byref(ms)))
        return int(n.value), float(ms.value)

    # -- prefix tree
    def prefix_insert(self, seq: int, tokens) -> int:
        tokens, pt = _i32(tokens)
        n = C.c_int32()
        check(lib.bkv_prefix_insert(self.handle, seq, pt, tokens.size, C.byref(n)))
        return int(n.value)

    def prefix_match(self, tokens) -> int:
        tokens, pt = _i32(tokens)
        m = C.c_int64()
        check(lib.bkv_prefix_match(self.handle, pt, tokens.size, C.byref(m)))
        return int(m.value)

    def seq_create_from_prefix(self, tokens):
        """-> (seq, matched_tokens)"""
        tokens, pt = _i32(tokens)
        s, m = C.c_int32(), C.c_int64()
        check(lib.bkv_seq_create_from_prefix(self.handle, pt, tokens.size, C.byref(s), C.byref(m)))
        return int(s.value), int(m.value)

    def prefix_evict(self, want_pages: int) -> int:
        n = C.c_int32()
        check(lib.bkv_prefix_evict(self.handle, want_pages, C.byref(n)))
        return int(n.value)

    def prefix_pin(self, tokens, pin: bool = True) -> int:
        tokens, pt = _i32(tokens)
        m = C.c_int64()
        check(lib.bkv_prefix_pin(self.handle, pt, tokens.size, 1 if pin else 0, C.byref(m)))
        return int(m.value)

    def prefix_stats(self):
        """-> (nodes, evictable_pages, pinned_nodes)"""
        a, b, c = C.c_int32(), C.c_int32(), C.c_int32()
        check(lib.bkv_prefix_stats(self.handle, C.byref(a), C.byref(b), C.byref(c)))
        return int(a.value), int(b.value), int(c.value)

    def prefix_clear(self) -> None:
        check(lib.bkv_prefix_clear(self.handle))

    def prefix_tiers(self, host_bytes: int, disk_path: str | None = None, disk_bytes: int = 0) -> None:
        """Lower tiers for evicted prefix pages: pinned host memory, then a file."""
        path = None if disk_path is None else os.fsencode(disk_path)
        check(lib.bkv_prefix_tiers(self.handle, host_bytes, path, disk_bytes))

    def prefix_prefetch(self, tokens) -> int:
        """Bring the matched chain's lower tiers back to the device; -> tokens on the device."""
        tokens, pt = _i32(tokens)
        m = C.c_int64()
        check(lib.bkv_prefix_prefetch(self.handle, pt, tokens.size, C.byref(m)))
        return int(m.value)

    def prefix_tier_stats(self):
        """-> ((device, host, disk) nodes, (to_host, to_disk, promoted, dropped) pages moved)"""
        nodes = (C.c_int32 * 3)()
        moved = (C.c_uint64 * 4)()
        check(lib.bkv_prefix_tier_stats(self.handle, nodes, moved))
        return tuple(int(x) for x in nodes), tuple(int(x) for x in moved)

    # -- hot path
    def append(self, layer: int, seqs, pos0, n_tokens, k_dev, v_dev, stream=None,
               f16_rows: bool = False) -> None:
        """k_dev / v_dev hold f32 rows, or raw binary16 rows when f16_rows is set."""
        seqs, ps = _i32(seqs)
        pos0, pp = _i64(pos0)
        n_tokens, pn = _i32(n_tokens)
        assert seqs.size == pos0.size == n_tokens.size
        fn = lib.bkv_append_f16 if f16_rows else lib.bkv_append
        check(fn(self.handle, layer, seqs.size, ps, pp, pn, _ptr(k_dev), _ptr(v_dev), _sh(stream)))

    def append_kprep(self, layer: int, seqs, pos0, n_tokens, k_dev, v_dev, gamma_dev, eps: float,
                     table_dev, n_rot: int, max_pos: int, positions_dev=None, stream=None) -> None:
        """RMSNorm(k) * gamma -> rotary at the token's position -> append, in one launch."""
        seqs, ps = _i32(seqs)
        pos0, pp = _i64(pos0)
        n_tokens, pn = _i32(n_tokens)
        assert seqs.size == pos0.size == n_tokens.size
        check(lib.bkv_append_kprep(self.handle, layer, seqs.size, ps, pp, pn, _ptr(k_dev), _ptr(v_dev),
                                   _ptr(gamma_dev), eps, _ptr(table_dev), n_rot, max_pos,
                                   _ptr(positions_dev) if positions_dev is not None else None,
                                   _sh(stream)))

    def decode_attn(self, layer: int, seqs, pos, n_q_head: int, q_dev, out_dev, scale: float,
                    gate_dev=None, gate_seq_stride: int = 0, gate_head_stride: int = 0,
                    stream=None) -> None:
        seqs, ps = _i32(seqs)
        pos, pp = _i64(pos)
        assert seqs.size == pos.size
        check(lib.bkv_decode_attn(self.handle, layer, seqs.size, ps, pp, n_q_head, _ptr(q_dev),
                                  _ptr(gate_dev), gate_seq_stride, gate_head_stride, scale,
                                  _ptr(out_dev), _sh(stream)))

    def decode_attn_static(self, layer: int, seqs, pos, n_q_head: int, q_dev, out_dev, scale: float,
                           gate_dev=None, gate_seq_stride: int = 0, gate_head_stride: int = 0,
                           stream=None) -> None:
        seqs, ps = _i32(seqs)
        pos, pp = _i64(pos)
        assert seqs.size == pos.size
        check(lib.bkv_decode_attn_static(self.handle, layer, seqs.size, ps, pp, n_q_head, _ptr(q_dev),
                                         _ptr(gate_dev), gate_seq_stride, gate_head_stride, scale,
                                         _ptr(out_dev), _sh(stream)))

    def prefill_attn(self, layer: int, seqs, pos0, n_tokens, n_q_head: int, q_dev, out_dev, scale: float,
                     gate_dev=None, gate_tok_stride: int = 0, gate_head_stride: int = 0, stream=None) -> None:
        """Causal attention of whole chunks (token t of chunk i sees cells 0..pos0[i]+t), on MFMA."""
        seqs, ps = _i32(seqs)
        pos0, pp = _i64(pos0)
        n_tokens, pn = _i32(n_tokens)
        assert seqs.size == pos0.size == n_tokens.size
        check(lib.bkv_prefill_attn(self.handle, layer, seqs.size, ps, pp, pn, n_q_head, _ptr(q_dev),
                                   _ptr(gate_dev), gate_tok_stride, gate_head_stride, scale, _ptr(out_dev),
                                   _sh(stream)))

    def decode_step(self, layer: int, seqs, pos, k_new_dev, v_new_dev, n_q_head: int, q_dev, out_dev,
                    scale: float, gate_dev=None, gate_seq_stride: int = 0, gate_head_stride: int = 0,
                    stream=None) -> None:
        """Append one token per sequence at pos and attend 0..pos, in one call."""
        seqs, ps = _i32(seqs)
        pos, pp = _i64(pos)
        assert seqs.size == pos.size
        check(lib.bkv_decode_step(self.handle, layer, seqs.size, ps, pp, _ptr(k_new_dev), _ptr(v_new_dev),
                                  n_q_head, _ptr(q_dev), _ptr(gate_dev), gate_seq_stride, gate_head_stride,
                                  scale, _ptr(out_dev), _sh(stream)))

    def decode_attn_select(self, layer: int, seqs, pos, n_q_head: int, q_dev, out_dev, scale: float,
                           ids_dev, id_stride: int, counts_dev, max_ids: int, gate_dev=None,
                           gate_seq_stride: int = 0, gate_head_stride: int = 0, stream=None) -> None:
        """Attention over per-entry lists of selected 4-cell blocks (device u32 ids / counts)."""
        seqs, ps = _i32(seqs)
        pos, pp = _i64(pos)
        assert seqs.size == pos.size
        check(lib.bkv_decode_attn_select(self.handle, layer, seqs.size, ps, pp, n_q_head, _ptr(q_dev),
                                         _ptr(gate_dev), gate_seq_stride, gate_head_stride, scale,
                                         _ptr(ids_dev), id_stride, _ptr(counts_dev), max_ids,
                                         _ptr(out_dev), _sh(stream)))

    def select_blocks(self, pos, idx_q_dev, pooled_devs, n_blocks, idx_n_head: int, idx_dim: int,
                      topk_blocks: int, ids_dev, id_stride: int, counts_dev, max_ids: int,
                      stream=None) -> None:
        """Indexer score + top-k: leaves ids / counts on the device for decode_attn_select."""
        pos, pp = _i64(pos)
        n_blocks, pn = _i32(n_blocks)
        assert pos.size == n_blocks.size == len(pooled_devs)
        ptrs = (C.c_void_p * max(len(pooled_devs), 1))(*[_ptr(x) for x in pooled_devs])
        check(lib.bkv_select_blocks(self.handle, pos.size, pp, _ptr(idx_q_dev), ptrs, pn, idx_n_head,
                                    idx_dim, topk_blocks, _ptr(ids_dev), id_stride, _ptr(counts_dev),
                                    max_ids, _sh(stream)))

    def idx_pool(self, pooled_dev, max_blocks: int, tail_dev, idx_k_dev, pos0: int, tokens: int, gamma_dev,
                 eps: float, table_dev, n_rot: int, max_pos: int, idx_dim: int = 128, stream=None) -> None:
        """Pool the indexer keys of every block this call completes; keep the incomplete tail."""
        check(lib.bkv_idx_pool(self.handle, _ptr(pooled_dev), max_blocks, _ptr(tail_dev), _ptr(idx_k_dev), pos0,
                               tokens, _ptr(gamma_dev), eps, _ptr(table_dev), n_rot, max_pos, idx_dim,
                               _sh(stream)))

    def topk_blocks(self, pos, scores_dev, n_blocks: int, topk_blocks: int, ids_dev, id_stride: int,
                    counts_dev, max_ids: int, dense: bool = False, stream=None) -> None:
        pos, pp = _i64(pos)
        check(lib.bkv_topk_blocks(self.handle, pos.size, pp, _ptr(scores_dev), n_blocks, topk_blocks,
                                  1 if dense else 0, _ptr(ids_dev), id_stride, _ptr(counts_dev), max_ids,
                                  _sh(stream)))

    def page_copy(self, pairs, stream=None) -> None:
        """pairs: iterable of (src, dst), or an int32 array of shape [n, 2]."""
        arr = np.ascontiguousarray(np.asarray(list(pairs) if not isinstance(pairs, np.ndarray)
                                              else pairs, dtype=np.int32).reshape(-1, 2))
        ptr = arr.ctypes.data_as(C.POINTER(PagePair))
        check(lib.bkv_page_copy(self.handle, ptr, arr.shape[0], _sh(stream)))

    def gather(self, layer: int, seq: int, cell0: int, n: int, stream=None):
        """Dequantised K and V rows as float32 arrays [n, n_kv, head_dim]."""
        shape = (n, self.desc.n_kv_head, self.desc.head_dim)
        count = int(np.prod(shape))
        kb = DeviceBuffer(max(count * 4, 16))
        vb = DeviceBuffer(max(count * 4, 16))
        try:
            check(lib.bkv_gather(self.handle, layer, seq, cell0, n, kb.ptr, vb.ptr, _sh(stream)))
            k = kb.download(np.float32, count, stream).reshape(shape)
            v = vb.download(np.float32, count, stream).reshape(shape)
        finally:
            kb.free()
            vb.free()
        return k, v

    # -- swap
    def host_alloc(self, nbytes: int) -> "PinnedBuffer":
        return PinnedBuffer(self, nbytes)

    def swap_out(self, pages, host: "PinnedBuffer", stream=None) -> None:
        pages, pp = _i32(pages)
        assert pages.size * self.swap_page_bytes() <= host.nbytes
        check(lib.bkv_swap_out(self.handle, pp, pages.size, host.ptr, _sh(stream)))

    def swap_in(self, pages, host: "PinnedBuffer", stream=None) -> None:
        pages, pp = _i32(pages)
        assert pages.size * self.swap_page_bytes() <= host.nbytes
        check(lib.bkv_swap_in(self.handle, pp, pages.size, host.ptr, _sh(stream)))

    def swap_wait(self) -> None:
        check(lib.bkv_swap_wait(self.handle))

    def swap_wait_for(self, timeout_ms: int) -> None:
        check(lib.bkv_swap_wait_for(self.handle, timeout_ms))

    def swap_fence(self, stream=None) -> None:
        check(lib.bkv_swap_fence(self.handle, _sh(stream)))

    def seq_evict(self, seq: int, lp0: int, n: int, host: "PinnedBuffer", stream=None) -> None:
        assert n * self.swap_page_bytes() <= host.nbytes
        check(lib.bkv_seq_evict(self.handle, seq, lp0, n, host.ptr, _sh(stream)))

    def seq_restore(self, seq: int, lp0: int, n: int, host: "PinnedBuffer", stream=None) -> None:
        assert n * self.swap_page_bytes() <= host.nbytes
        check(lib.bkv_seq_restore(self.handle, seq, lp0, n, host.ptr, _sh(stream)))


class StepPlan:
    """A decode step whose batch lives on the device (bkv_step_plan_*): capturable and replayable."""

    def __init__(self, pool: Pool, seqs, pos, horizon: int, n_q_head: int, stream=None):
        seqs, ps = _i32(seqs)
        pos, pp = _i64(pos)
        assert seqs.size == pos.size
        self.n = int(seqs.size)
        self.handle = C.c_void_p()
        check(lib.bkv_step_plan_create(pool.handle, self.n, ps, pp, horizon, n_q_head, _sh(stream),
                                       C.byref(self.handle)))

    def decode(self, layer: int, k_new_dev, v_new_dev, q_dev, out_dev, scale: float, gate_dev=None,
               gate_seq_stride: int = 0, gate_head_stride: int = 0, stream=None) -> None:
        check(lib.bkv_step_plan_decode(self.handle, layer, _ptr(k_new_dev), _ptr(v_new_dev), _ptr(q_dev),
                                       _ptr(gate_dev), gate_seq_stride, gate_head_stride, scale, _ptr(out_dev),
                                       _sh(stream)))

    def advance(self, stream=None) -> None:
        check(lib.bkv_step_plan_advance(self.handle, _sh(stream)))

    def state(self, stream=None):
        """(positions, advances done, status) once `stream` has drained."""
        pos = np.zeros(self.n, dtype=np.int64)
        steps, status = C.c_uint32(), C.c_int32()
        check(lib.bkv_step_plan_state(self.handle, _sh(stream), pos.ctypes.data_as(C.POINTER(C.c_int64)),
                                      C.byref(steps), C.byref(status)))
        return pos, int(steps.value), int(status.value)

    def destroy(self) -> None:
        if self.handle:
            check(lib.bkv_step_plan_destroy(self.handle))
            self.handle = None


class Graph:
    """Work captured from a stream (bkv_graph_*)."""

    def __init__(self, stream: Stream):
        self.stream = stream
        self.exec = None
        check(lib.bkv_graph_begin_capture(stream.handle))

    def end(self) -> "Graph":
        ex = C.c_void_p()
        check(lib.bkv_graph_end_capture(self.stream.handle, C.byref(ex)))
        self.exec = ex
        return self

    def launch(self, stream=None) -> None:
        check(lib.bkv_graph_launch(self.exec, _sh(stream if stream is not None else self.stream)))

    def destroy(self) -> None:
        if self.exec:
            check(lib.bkv_graph_destroy(self.exec))
            self.exec = None


class PinnedBuffer:
    """hipHostMalloc'd memory owned through the pool, viewable as a numpy array."""

    def __init__(self, pool: Pool, nbytes: int):
        self.pool, self.nbytes = pool, int(nbytes)
        p = C.c_void_p()
        check(lib.bkv_host_alloc(pool.handle, self.nbytes, C.byref(p)))
        self.ptr = p

    def view(self) -> np.ndarray:
        buf = (C.c_uint8 * self.nbytes).from_address(self.ptr.value)
        return np.frombuffer(buf, dtype=np.uint8)

    def free(self) -> None:
        if self.ptr:
            check(lib.bkv_host_free(self.pool.handle, self.ptr))
            self.ptr = None


def _ptr(x):
    if x is None:
        return None
    if isinstance(x, DeviceBuffer):
        return x.ptr
    return x
