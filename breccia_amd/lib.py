"""ctypes binding of libbreccia_kv.so -- one Python function per C entry point.

There is no fallback: if the HIP library has not been built, importing this module
raises.  Nothing here computes anything on the CPU.
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libbreccia_kv.so")
BENCH_LIB_PATH = os.path.join(HERE, "libbreccia_kv_bench.so")
HEADER_PATH = os.path.join(HERE, "..", "include", "breccia_kv.h")
BENCH_HEADER_PATH = os.path.join(HERE, "..", "include", "breccia_kv_bench.h")

OK, ERR_INVALID, ERR_RANGE, ERR_NO_PAGES, ERR_STATE, ERR_NO_DEVICE, ERR_HIP, ERR_NOMEM, ERR_TIMEOUT = range(9)
STATUS_NAMES = ["OK", "INVALID", "RANGE", "NO_PAGES", "STATE", "NO_DEVICE", "HIP", "NOMEM", "TIMEOUT"]
LAYOUT_F16, LAYOUT_Q8V, LAYOUT_I8H = 0, 1, 2
POOL_HOST_ONLY = 1
MAX_BATCH = 64
MAX_KV_HEAD = 16
STATIC_WGS = 1024
(STAGE_APPEND, STAGE_ATTN_SPLIT, STAGE_ATTN_MERGE, STAGE_PAGE_COPY, STAGE_PREFILL_ATTN, STAGE_APPEND_KPREP,
 STAGE_IDX_POOL, STAGE_IDX_SCORE, STAGE_TOPK, STAGE_PAGE_STAGE) = range(10)


class BkvError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__("BKV_ERR_%s: %s" % (STATUS_NAMES[status], message))
        self.status = status
        self.message = message


class PoolDesc(C.Structure):
    _fields_ = [("n_layers", C.c_int32), ("n_pages", C.c_int32), ("n_kv_head", C.c_int32),
                ("head_dim", C.c_int32), ("page_cells", C.c_int32), ("layout", C.c_int32),
                ("max_seqs", C.c_int32), ("max_pages_per_seq", C.c_int32), ("flags", C.c_uint32)]


class PagePair(C.Structure):
    _fields_ = [("src", C.c_int32), ("dst", C.c_int32)]


def _load(path: str) -> C.CDLL:
    if not os.path.exists(path):
        raise ImportError(
            "%s is not built (%s). Build it with `python -m breccia_amd.build` "
            "(needs hipcc); there is no CPU fallback." % (os.path.basename(path), path))
    return C.CDLL(path)


_product = _load(LIB_PATH)        # the paged-KV library: include/breccia_kv.h
_bench = _load(BENCH_LIB_PATH)    # device plumbing and probes for tests and bench: include/breccia_kv_bench.h

_vp, _i32, _i64, _u64, _f32 = C.c_void_p, C.c_int32, C.c_int64, C.c_uint64, C.c_float
_pi32, _pi64 = C.POINTER(C.c_int32), C.POINTER(C.c_int64)

_SIGNATURES = {
    "bkv_last_error": (C.c_char_p, []),
    "bkv_version": (C.c_char_p, []),
    "bkv_pool_create": (C.c_int, [C.POINTER(PoolDesc), C.POINTER(_vp)]),
    "bkv_pool_destroy": (C.c_int, [_vp]),
    "bkv_pool_reset": (C.c_int, [_vp, _vp]),
    "bkv_pool_get_desc": (C.c_int, [_vp, C.POINTER(PoolDesc)]),
    "bkv_pool_bytes": (_u64, [_vp]),
    "bkv_page_bytes": (_u64, [_vp, C.c_int]),
    "bkv_pool_fill": (C.c_int, [_vp, C.c_int, _vp]),
    "bkv_pool_layer_ptr": (C.c_int, [_vp, _i32, C.c_int, C.POINTER(_vp), C.POINTER(_u64)]),
    "bkv_seq_create": (C.c_int, [_vp, _pi32]),
    "bkv_seq_create_identity": (C.c_int, [_vp, _i32, _pi32]),
    "bkv_seq_fork": (C.c_int, [_vp, _i32, _i64, _pi32]),
    "bkv_seq_free": (C.c_int, [_vp, _i32]),
    "bkv_seq_reserve": (C.c_int, [_vp, _i32, _i64, C.POINTER(PagePair), _i32, _pi32]),
    "bkv_seq_truncate": (C.c_int, [_vp, _i32, _i64]),
    "bkv_seq_len": (_i64, [_vp, _i32]),
    "bkv_seq_capacity": (_i64, [_vp, _i32]),
    "bkv_seq_n_pages": (_i32, [_vp, _i32]),
    "bkv_seq_block_table": (_pi32, [_vp, _i32]),
    "bkv_page_refcount": (_i32, [_vp, _i32]),
    "bkv_pool_free_pages": (_i32, [_vp]),
    "bkv_pool_check": (C.c_int, [_vp]),
    "bkv_pool_set_free_order": (C.c_int, [_vp, _pi32, _i32]),
    "bkv_prefix_insert": (C.c_int, [_vp, _i32, _pi32, _i64, _pi32]),
    "bkv_prefix_match": (C.c_int, [_vp, _pi32, _i64, _pi64]),
    "bkv_seq_create_from_prefix": (C.c_int, [_vp, _pi32, _i64, _pi32, _pi64]),
    "bkv_prefix_evict": (C.c_int, [_vp, _i32, _pi32]),
    "bkv_prefix_pin": (C.c_int, [_vp, _pi32, _i64, _i32, _pi64]),
    "bkv_prefix_stats": (C.c_int, [_vp, _pi32, _pi32, _pi32]),
    "bkv_prefix_clear": (C.c_int, [_vp]),
    "bkv_prefix_tiers": (C.c_int, [_vp, _u64, C.c_char_p, _u64]),
    "bkv_prefix_tier_stats": (C.c_int, [_vp, _pi32, C.POINTER(C.c_uint64)]),
    "bkv_prefix_prefetch": (C.c_int, [_vp, _pi32, _i64, _pi64]),
    "bkv_timing_enable": (C.c_int, [_vp, C.c_int]),
    "bkv_timing_reset": (C.c_int, [_vp]),
    "bkv_timing_read": (C.c_int, [_vp, C.c_int, C.POINTER(_u64), C.POINTER(C.c_double)]),
    "bkv_append": (C.c_int, [_vp, _i32, _i32, _pi32, _pi64, _pi32, _vp, _vp, _vp]),
    "bkv_append_f16": (C.c_int, [_vp, _i32, _i32, _pi32, _pi64, _pi32, _vp, _vp, _vp]),
    "bkv_append_kprep": (C.c_int, [_vp, _i32, _i32, _pi32, _pi64, _pi32, _vp, _vp, _vp, _f32, _vp, _i32,
                                   _i32, _vp, _vp]),
    "bkv_rope_table": (C.c_int, [C.c_double, _i32, _i32, _vp]),
    "bkv_decode_attn": (C.c_int, [_vp, _i32, _i32, _pi32, _pi64, _i32, _vp, _vp, _i64, _i64, _f32,
                                  _vp, _vp]),
    "bkv_decode_attn_static": (C.c_int, [_vp, _i32, _i32, _pi32, _pi64, _i32, _vp, _vp, _i64, _i64, _f32,
                                         _vp, _vp]),
    "bkv_attn_plan": (C.c_int, [_i32, _i32, _i32, _i32, _pi64, _i32, _pi32, _pi32, _pi32]),
    "bkv_prefill_attn": (C.c_int, [_vp, _i32, _i32, _pi32, _pi64, _pi32, _i32, _vp, _vp, _i64, _i64, _f32,
                                   _vp, _vp]),
    "bkv_decode_step": (C.c_int, [_vp, _i32, _i32, _pi32, _pi64, _vp, _vp, _i32, _vp, _vp, _i64, _i64, _f32,
                                  _vp, _vp]),
    "bkv_step_plan_create": (C.c_int, [_vp, _i32, _pi32, _pi64, _i32, _i32, _vp, C.POINTER(_vp)]),
    "bkv_step_plan_destroy": (C.c_int, [_vp]),
    "bkv_step_plan_decode": (C.c_int, [_vp, _i32, _vp, _vp, _vp, _vp, _i64, _i64, _f32, _vp, _vp]),
    "bkv_step_plan_advance": (C.c_int, [_vp, _vp]),
    "bkv_step_plan_state": (C.c_int, [_vp, _vp, _pi64, C.POINTER(C.c_uint32), _pi32]),
    "bkv_decode_attn_select": (C.c_int, [_vp, _i32, _i32, _pi32, _pi64, _i32, _vp, _vp, _i64, _i64, _f32,
                                         _vp, _i64, _vp, _i32, _vp, _vp]),
    "bkv_select_blocks": (C.c_int, [_vp, _i32, _pi64, _vp, C.POINTER(_vp), _pi32, _i32, _i32, _i32, _vp,
                                    _i64, _vp, _i32, _vp]),
    "bkv_idx_pool": (C.c_int, [_vp, _vp, _i32, _vp, _vp, _i64, _i32, _vp, _f32, _vp, _i32, _i32, _i32, _vp]),
    "bkv_topk_blocks": (C.c_int, [_vp, _i32, _pi64, _vp, _i32, _i32, _i32, _vp, _i64, _vp, _i32, _vp]),
    "bkv_page_copy": (C.c_int, [_vp, C.POINTER(PagePair), _i32, _vp]),
    "bkv_swap_page_bytes": (_u64, [_vp]),
    "bkv_host_alloc": (C.c_int, [_vp, _u64, C.POINTER(_vp)]),
    "bkv_host_free": (C.c_int, [_vp, _vp]),
    "bkv_swap_out": (C.c_int, [_vp, _pi32, _i32, _vp, _vp]),
    "bkv_swap_in": (C.c_int, [_vp, _pi32, _i32, _vp, _vp]),
    "bkv_swap_wait": (C.c_int, [_vp]),
    "bkv_swap_wait_for": (C.c_int, [_vp, _i64]),
    "bkv_stream_wait": (C.c_int, [_vp, _i64]),
    "bkv_wait_options": (C.c_int, [_i64, _i64]),
    "bkv_wait_options_get": (C.c_int, [_pi64, _pi64]),
    "bkv_swap_fence": (C.c_int, [_vp, _vp]),
    "bkv_seq_evict": (C.c_int, [_vp, _i32, _i32, _i32, _vp, _vp]),
    "bkv_seq_restore": (C.c_int, [_vp, _i32, _i32, _i32, _vp, _vp]),
    "bkv_gather": (C.c_int, [_vp, _i32, _i32, _i64, _i64, _vp, _vp, _vp]),
}

_BENCH_SIGNATURES = {
    "bkv_bench_last_error": (C.c_char_p, []),
    "bkv_dev_alloc": (C.c_int, [_u64, C.POINTER(_vp)]),
    "bkv_dev_free": (C.c_int, [_vp]),
    "bkv_memcpy_h2d": (C.c_int, [_vp, _vp, _u64, _vp]),
    "bkv_memcpy_d2h": (C.c_int, [_vp, _vp, _u64, _vp]),
    "bkv_stream_create": (C.c_int, [C.POINTER(_vp)]),
    "bkv_graph_begin_capture": (C.c_int, [_vp]),
    "bkv_graph_end_capture": (C.c_int, [_vp, C.POINTER(_vp)]),
    "bkv_graph_launch": (C.c_int, [_vp, _vp]),
    "bkv_graph_destroy": (C.c_int, [_vp]),
    "bkv_stream_destroy": (C.c_int, [_vp]),
    "bkv_stream_sync": (C.c_int, [_vp]),
    "bkv_device_sync": (C.c_int, []),
    "bkv_event_create": (C.c_int, [C.POINTER(_vp)]),
    "bkv_event_destroy": (C.c_int, [_vp]),
    "bkv_event_record": (C.c_int, [_vp, _vp]),
    "bkv_event_sync": (C.c_int, [_vp]),
    "bkv_event_elapsed_ms": (C.c_int, [_vp, _vp, C.POINTER(C.c_float)]),
    "bkv_device_info": (C.c_int, [C.c_char_p, _i32, _pi32, C.POINTER(_u64)]),
    "bkv_device_mem_info": (C.c_int, [C.POINTER(_u64), C.POINTER(_u64)]),
    "bkv_copy_probe": (C.c_int, [_vp, _vp, _u64, _vp]),
    "bkv_read_probe": (C.c_int, [_vp, _u64, _i32, _vp, _vp]),
}

_bench_error = None   # message of the last failed call into the bench library, until check() takes it


def _bench_call(fn):
    def call(*args):
        global _bench_error
        status = fn(*args)
        if status != OK:
            _bench_error = _bench.bkv_bench_last_error().decode("utf-8", "replace")
        return status
    return call


class _Both:
    """Every entry point of the two libraries under one name space (the names do not overlap)."""


lib = _Both()
for _name, (_res, _args) in _SIGNATURES.items():
    _fn = getattr(_product, _name)
    _fn.restype = _res
    _fn.argtypes = _args
    setattr(lib, _name, _fn)
for _name, (_res, _args) in _BENCH_SIGNATURES.items():
    _fn = getattr(_bench, _name)
    _fn.restype = _res
    _fn.argtypes = _args
    setattr(lib, _name, _bench_call(_fn) if _res is C.c_int else _fn)


def last_error() -> str:
    return _product.bkv_last_error().decode("utf-8", "replace")


def check(status: int) -> None:
    global _bench_error
    if status != OK:
        msg, _bench_error = (_bench_error, None) if _bench_error is not None else (last_error(), None)
        raise BkvError(status, msg)
