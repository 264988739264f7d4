"""ctypes front-end of the CPU oracle (``bkv_oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by ``__graft_entry__.smoke()``
and by the ``cpu_baseline`` leg of ``bench.py`` as the checker / the reported CPU
baseline.  The shipped package never imports it.

Every routine here forwards to the C restatement, which cites the reference
file:line it follows.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libbkv_oracle.so")
_F16C_PATH = os.path.join(_HERE, "libf16c_ref.so")

LAYOUT_F16 = 0   # f16 K and V            (reference default)
LAYOUT_Q8V = 1   # f16 K, q8_0 V, f32 scale, 36 B / 32 values (reference BRECCIA_KV_Q8V)
LAYOUT_I8H = 2   # int8 K and V, f16 scale, 34 B / 32 values   (not in the reference)


def build(force: bool = False) -> None:
    """Compile the oracle with the committed Makefile (gcc only, no GPU)."""
    if force:
        subprocess.run(["make", "-C", _HERE, "clean"], check=True, capture_output=True)
    subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)


def _load() -> C.CDLL:
    if not os.path.exists(_LIB_PATH):
        build()
    return C.CDLL(_LIB_PATH)


_lib = _load()


class Geom(C.Structure):
    _fields_ = [("n_kv", C.c_int32), ("head_dim", C.c_int32), ("page_cells", C.c_int32)]

    def row_elems(self) -> int:
        return self.head_dim

    def rows(self, n_pages: int) -> int:
        return n_pages * self.n_kv * self.page_cells


def _p(a: np.ndarray, ty):
    return a.ctypes.data_as(C.POINTER(ty))


_lib.bkvo_f32_to_f16_bits.restype = C.c_uint16
_lib.bkvo_f32_to_f16_bits.argtypes = [C.c_float]
_lib.bkvo_f16_bits_to_f32.restype = C.c_float
_lib.bkvo_f16_bits_to_f32.argtypes = [C.c_uint16]
_lib.bkvo_to_f16.restype = C.c_float
_lib.bkvo_to_f16.argtypes = [C.c_float]
_lib.bkvo_f32_to_f16_bits_n.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p]
_lib.bkvo_f16_bits_to_f32_n.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p]
_lib.bkvo_f16_sweep_mismatches.restype = C.c_uint64
_lib.bkvo_f16_sweep_mismatches.argtypes = [C.c_uint32, C.c_uint64, C.c_void_p, C.c_int]
_lib.bkvo_to_q8_0.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p, C.c_void_p]
_lib.bkvo_to_i8h.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p, C.c_void_p]
_lib.bkvo_row_index.restype = C.c_size_t
_lib.bkvo_row_index.argtypes = [C.POINTER(Geom), C.c_int32, C.c_int32, C.c_int32]
_lib.bkvo_elem_index.restype = C.c_size_t
_lib.bkvo_elem_index.argtypes = [C.POINTER(Geom), C.c_int32, C.c_int32, C.c_int32, C.c_int32]
_lib.bkvo_i8_row_bytes.restype = C.c_size_t
_lib.bkvo_i8_row_bytes.argtypes = [C.POINTER(Geom)]
for _name in ("bkvo_append_f16", "bkvo_append_q8v", "bkvo_append_i8"):
    getattr(_lib, _name).restype = C.c_int
    getattr(_lib, _name).argtypes = [C.POINTER(Geom), C.c_void_p, C.c_void_p, C.c_void_p,
                                     C.c_int64, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p]
_lib.bkvo_gather.restype = C.c_int
_lib.bkvo_gather.argtypes = [C.POINTER(Geom), C.c_int, C.c_void_p, C.c_void_p, C.c_void_p,
                             C.c_int64, C.c_int64, C.c_void_p, C.c_void_p]
_lib.bkvo_attend.restype = C.c_int
_lib.bkvo_attend.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t,
                             C.c_int64, C.c_int32, C.c_int32, C.c_int32, C.c_void_p,
                             C.c_void_p, C.c_int]
_lib.bkvo_attend_probs.restype = C.c_int
_lib.bkvo_attend_probs.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_int64,
                                   C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_void_p,
                                   C.POINTER(C.c_size_t)]
_lib.bkvo_cells_of.restype = C.c_size_t
_lib.bkvo_cells_of.argtypes = [C.c_void_p, C.c_size_t, C.c_uint32, C.c_void_p]
_lib.bkvo_dense_ids.restype = C.c_size_t
_lib.bkvo_dense_ids.argtypes = [C.c_int64, C.c_int64, C.c_uint32, C.c_void_p]
_lib.bkvo_page_copy.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t]
_lib.bkvo_swap_out.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_void_p,
                               C.c_size_t, C.c_size_t]
_lib.bkvo_swap_in.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_void_p,
                              C.c_size_t, C.c_size_t]
_lib.bkvo_indexer_score.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int64, C.c_size_t,
                                    C.c_size_t, C.c_size_t, C.c_void_p]
_lib.bkvo_topk_blocks.restype = C.c_size_t
_lib.bkvo_topk_blocks.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_int64, C.c_void_p]
_lib.bkvo_rmsnorm.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_void_p, C.c_float,
                              C.c_void_p]
_lib.bkvo_rope_table.argtypes = [C.c_double, C.c_size_t, C.c_size_t, C.c_void_p]
_lib.bkvo_rope_apply.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_void_p,
                                 C.c_size_t, C.c_void_p, C.c_void_p]
_lib.bkvo_pool_keys.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t,
                                C.c_size_t, C.c_size_t, C.c_float, C.c_void_p]
_lib.bkvo_normalish.argtypes = [C.c_uint64, C.c_size_t, C.c_void_p]
_lib.bkvo_q8_fixture.argtypes = [C.c_void_p, C.c_size_t]
_lib.bkvo_max_threads.restype = C.c_int


def max_threads() -> int:
    return int(_lib.bkvo_max_threads())


# --------------------------------------------------------------------------- f16
def f32_to_f16_bits(x) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    _lib.bkvo_f32_to_f16_bits_n(x.ctypes.data, x.size, out.ctypes.data)
    return out


def f16_bits_to_f32(h) -> np.ndarray:
    h = np.ascontiguousarray(h, dtype=np.uint16)
    out = np.empty(h.shape, dtype=np.float32)
    _lib.bkvo_f16_bits_to_f32_n(h.ctypes.data, h.size, out.ctypes.data)
    return out


def to_f16(x) -> np.ndarray:
    """f32 -> cache f16 -> f32 (value map of the cache's storage rule)."""
    return f16_bits_to_f32(f32_to_f16_bits(x))


def f16_sweep_mismatches(first: int, expect: np.ndarray, documented_deviations: bool) -> int:
    expect = np.ascontiguousarray(expect, dtype=np.uint16)
    return int(_lib.bkvo_f16_sweep_mismatches(first, expect.size, expect.ctypes.data,
                                              1 if documented_deviations else 0))


def f16c_reference():
    """The F16C hardware convert as an independent reference, or None without the CPU flag."""
    if not os.path.exists(_F16C_PATH):
        build()
    lib = C.CDLL(_F16C_PATH)
    lib.f16c_cpu_supported.restype = C.c_int
    if not lib.f16c_cpu_supported():
        return None
    lib.f16c_convert_range.argtypes = [C.c_uint32, C.c_uint64, C.c_void_p]

    def convert(first: int, count: int) -> np.ndarray:
        assert count % 8 == 0
        out = np.empty(count, dtype=np.uint16)
        lib.f16c_convert_range(first, count, out.ctypes.data)
        return out

    return convert


# ------------------------------------------------------------------- quantisers
def to_q8_0(x):
    """Reference q8_0 (f32 scale).  Returns (dequantised f32, int8 codes, f32 scales)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    assert x.size % 32 == 0
    deq = np.empty(x.shape, dtype=np.float32)
    q = np.empty(x.shape, dtype=np.int8)
    sc = np.empty(x.size // 32, dtype=np.float32)
    _lib.bkvo_to_q8_0(x.ctypes.data, x.size, deq.ctypes.data, q.ctypes.data, sc.ctypes.data)
    return deq, q, sc


def to_i8h(x):
    """int8 with f16 scale (not in the reference).  Returns (deq f32, int8 codes, scale f16 bits)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    assert x.size % 32 == 0
    deq = np.empty(x.shape, dtype=np.float32)
    q = np.empty(x.shape, dtype=np.int8)
    sc = np.empty(x.size // 32, dtype=np.uint16)
    _lib.bkvo_to_i8h(x.ctypes.data, x.size, deq.ctypes.data, q.ctypes.data, sc.ctypes.data)
    return deq, q, sc


# ------------------------------------------------------------------ pool images
def elem_index(g: Geom, page: int, kvh: int, in_page: int, d: int) -> int:
    return int(_lib.bkvo_elem_index(C.byref(g), page, kvh, in_page, d))


def row_bytes(g: Geom, layout: int, which: str) -> int:
    """Bytes of one (page, kv head, cell) row of the K ('k') or V ('v') pool."""
    if layout == LAYOUT_F16 or (layout == LAYOUT_Q8V and which == "k"):
        return g.head_dim * 2
    if layout == LAYOUT_Q8V:
        return (g.head_dim // 32) * 36
    return int(_lib.bkvo_i8_row_bytes(C.byref(g)))


class PoolImage:
    """Host image of one layer's K and V pools in the library's byte layout."""

    def __init__(self, g: Geom, n_pages: int, layout: int = LAYOUT_F16):
        self.g, self.n_pages, self.layout = g, n_pages, layout
        rows = g.rows(n_pages)
        self.k = np.zeros(rows * row_bytes(g, layout, "k"), dtype=np.uint8)
        self.v = np.zeros(rows * row_bytes(g, layout, "v"), dtype=np.uint8)

    def page_bytes(self, which: str) -> int:
        return self.g.n_kv * self.g.page_cells * row_bytes(self.g, self.layout, which)

    def append(self, block_table, pos0: int, k, v, capacity_cells: int | None = None) -> int:
        bt = np.ascontiguousarray(block_table, dtype=np.int32)
        k = np.ascontiguousarray(k, dtype=np.float32)
        v = np.ascontiguousarray(v, dtype=np.float32)
        T = k.size // (self.g.n_kv * self.g.head_dim)
        assert k.size == v.size == T * self.g.n_kv * self.g.head_dim
        cap = bt.size * self.g.page_cells if capacity_cells is None else capacity_cells
        fn = (_lib.bkvo_append_f16, _lib.bkvo_append_q8v, _lib.bkvo_append_i8)[self.layout]
        return int(fn(C.byref(self.g), self.k.ctypes.data, self.v.ctypes.data, bt.ctypes.data,
                      cap, pos0, T, k.ctypes.data, v.ctypes.data))

    def gather(self, block_table, cell0: int, n: int):
        bt = np.ascontiguousarray(block_table, dtype=np.int32)
        ko = np.empty((n, self.g.n_kv, self.g.head_dim), dtype=np.float32)
        vo = np.empty_like(ko)
        rc = _lib.bkvo_gather(C.byref(self.g), self.layout, self.k.ctypes.data, self.v.ctypes.data,
                              bt.ctypes.data, cell0, n, ko.ctypes.data, vo.ctypes.data)
        assert rc == 0
        return ko, vo

    def page_copy(self, pairs) -> None:
        pr = np.ascontiguousarray(pairs, dtype=np.int32).reshape(-1, 2)
        for arr, which in ((self.k, "k"), (self.v, "v")):
            _lib.bkvo_page_copy(arr.ctypes.data, self.page_bytes(which), pr.ctypes.data, pr.shape[0])


# -------------------------------------------------------------------- attention
def attend(q, k, v, cells, pos: int, n_head: int, n_kv: int, hd: int, gate=None,
           threads: int = 1) -> np.ndarray:
    q = np.ascontiguousarray(q, dtype=np.float32)
    k = np.ascontiguousarray(k, dtype=np.float32)
    v = np.ascontiguousarray(v, dtype=np.float32)
    cells = np.ascontiguousarray(cells, dtype=np.uint32)
    out = np.zeros((n_head, hd), dtype=np.float32)
    gp = None
    if gate is not None:
        gate = np.ascontiguousarray(gate, dtype=np.float32)
        assert gate.size == n_head * hd
        gp = gate.ctypes.data
    assert q.size == n_head * hd
    rc = _lib.bkvo_attend(q.ctypes.data, k.ctypes.data, v.ctypes.data, cells.ctypes.data,
                          cells.size, pos, n_head, n_kv, hd, gp, out.ctypes.data, threads)
    assert rc == 0, rc
    return out


def attend_probs(q, k, cells, pos: int, h: int, n_head: int, n_kv: int, hd: int) -> np.ndarray:
    q = np.ascontiguousarray(q, dtype=np.float32)
    k = np.ascontiguousarray(k, dtype=np.float32)
    cells = np.ascontiguousarray(cells, dtype=np.uint32)
    probs = np.empty(max(cells.size, 1), dtype=np.float64)
    n = C.c_size_t(0)
    _lib.bkvo_attend_probs(q.ctypes.data, k.ctypes.data, cells.ctypes.data, cells.size, pos, h,
                           n_head, n_kv, hd, probs.ctypes.data, C.byref(n))
    return probs[: n.value]


def cells_of(blocks, idx_block: int = 4) -> np.ndarray:
    blocks = np.ascontiguousarray(blocks, dtype=np.uint32)
    out = np.empty(blocks.size * idx_block, dtype=np.uint32)
    n = _lib.bkvo_cells_of(blocks.ctypes.data, blocks.size, idx_block, out.ctypes.data)
    return out[:n]


def dense_ids(pos: int, n_kv_after: int, idx_block: int = 4) -> np.ndarray:
    out = np.empty(n_kv_after // idx_block + 2, dtype=np.uint32)
    n = _lib.bkvo_dense_ids(pos, n_kv_after, idx_block, out.ctypes.data)
    return out[:n]


def dense_cells(pos: int) -> np.ndarray:
    """The dense selection's cell list; with the causal test it is cells 0..=pos."""
    return cells_of(dense_ids(pos, pos + 1))


# -------------------------------------------------------------- test generators
# ------------------------------------------------------------------ block selection
def indexer_score(q, pooled, n_blocks: int, pos: int, idx_n_head: int = 4, idx_dim: int = 128,
                  idx_block: int = 4) -> np.ndarray:
    """float64 [n_blocks]; q: [idx_n_head, idx_dim], pooled: [>= n_blocks, idx_dim]."""
    q = np.ascontiguousarray(q, dtype=np.float32)
    pooled = np.ascontiguousarray(pooled, dtype=np.float32)
    assert q.size == idx_n_head * idx_dim and pooled.size >= n_blocks * idx_dim
    out = np.empty(n_blocks, dtype=np.float64)
    _lib.bkvo_indexer_score(q.ctypes.data, pooled.ctypes.data, n_blocks, pos, idx_n_head, idx_dim,
                            idx_block, out.ctypes.data)
    return out


def topk_blocks(scores, k: int, own_block: int | None) -> np.ndarray:
    """uint32 ids: descending score, ties to the lower block, own block appended when missed."""
    scores = np.ascontiguousarray(scores, dtype=np.float64)
    out = np.empty(k + 1, dtype=np.uint32)
    n = _lib.bkvo_topk_blocks(scores.ctypes.data, scores.size, k, -1 if own_block is None else own_block,
                              out.ctypes.data)
    return out[:n].copy()


# ------------------------------------------------------------------ K preparation
def rmsnorm(x, cols: int, gamma=None, wgroups: int | None = None, eps: float = 1e-6) -> np.ndarray:
    """Row-wise RMSNorm of x viewed as [rows, cols]; gamma is [wgroups, cols] or None."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    rows = x.size // cols
    assert rows * cols == x.size
    if gamma is None:
        wg, gp = 0, None
    else:
        gamma = np.ascontiguousarray(gamma, dtype=np.float32)
        wg = gamma.size // cols if wgroups is None else wgroups
        assert gamma.size >= wg * cols and wg > 0
        gp = gamma.ctypes.data
    out = np.empty_like(x)
    _lib.bkvo_rmsnorm(x.ctypes.data, rows, cols, wg, gp, C.c_float(eps), out.ctypes.data)
    return out


def rope_table(freq_base: float, n_rot: int, max_pos: int) -> np.ndarray:
    """float32 [max_pos, n_rot/2, 2] of (cos, sin)."""
    assert n_rot % 2 == 0
    out = np.empty((max_pos, n_rot // 2, 2), dtype=np.float32)
    _lib.bkvo_rope_table(float(freq_base), n_rot, max_pos, out.ctypes.data)
    return out


def rope_apply(x, head_dim: int, n_rot: int, table, positions) -> np.ndarray:
    """x viewed as [rows, head_dim]; positions int32 [rows]."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    rows = x.size // head_dim
    table = np.ascontiguousarray(table, dtype=np.float32)
    positions = np.ascontiguousarray(positions, dtype=np.int32)
    assert positions.size >= rows and n_rot <= head_dim and n_rot % 2 == 0
    max_pos = table.size // n_rot
    out = np.empty_like(x)
    _lib.bkvo_rope_apply(x.ctypes.data, rows, head_dim, n_rot, table.ctypes.data, max_pos,
                         positions.ctypes.data, out.ctypes.data)
    return out


def k_prep(k, n_kv: int, hd: int, gamma, eps: float, table, n_rot: int, token_pos) -> np.ndarray:
    """What reaches the cache as K: per-(token, kv head) RMSNorm with gamma[hd], then the
    rotary at the token's position (crates/breccia-kernels/src/qsa/cpu.rs:383-397).
    k: [T, n_kv, hd]; token_pos: int [T]."""
    k = np.ascontiguousarray(k, dtype=np.float32).reshape(-1, n_kv, hd)
    normed = rmsnorm(k, hd, gamma, wgroups=1, eps=eps)
    pos = np.repeat(np.asarray(token_pos, dtype=np.int32), n_kv)
    return rope_apply(normed, hd, n_rot, table, pos).reshape(k.shape)


def pool_keys(raw, gamma, table, idx_dim: int = 128, idx_block: int = 4, n_rot: int = 64,
              eps: float = 1e-6) -> np.ndarray:
    """raw: [cells, idx_dim] raw indexer keys -> pooled [cells // idx_block, idx_dim]."""
    raw = np.ascontiguousarray(raw, dtype=np.float32).reshape(-1, idx_dim)
    gamma = np.ascontiguousarray(gamma, dtype=np.float32)
    table = np.ascontiguousarray(table, dtype=np.float32)
    out = np.empty((raw.shape[0] // idx_block, idx_dim), dtype=np.float32)
    _lib.bkvo_pool_keys(raw.ctypes.data, raw.shape[0], gamma.ctypes.data, table.ctypes.data,
                        table.size // n_rot, idx_dim, idx_block, n_rot, C.c_float(eps), out.ctypes.data)
    return out


def normalish(seed: int, n: int) -> np.ndarray:
    out = np.empty(n, dtype=np.float32)
    _lib.bkvo_normalish(seed, n, out.ctypes.data)
    return out


def q8_fixture(n: int = 256) -> np.ndarray:
    out = np.empty(n, dtype=np.float32)
    _lib.bkvo_q8_fixture(out.ctypes.data, n)
    return out
