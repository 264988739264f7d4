"""Shared helpers of the test suite (independent statements used to cross-check the oracle)."""
import numpy as np


def np_cache_f16_bits(x: np.ndarray) -> np.ndarray:
    """numpy's IEEE round-to-nearest-even float16 cast with the cache rule's two documented
    deviations applied: |x| < 2^-14 -> signed zero, NaN -> signed infinity."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    bits = x.view(np.uint32)
    with np.errstate(over="ignore", invalid="ignore"):
        h = x.astype(np.float16).view(np.uint16)
    mag = bits & np.uint32(0x7FFFFFFF)
    sign = ((bits >> np.uint32(16)) & np.uint32(0x8000)).astype(np.uint16)
    h = np.where(mag < np.uint32(0x38800000), sign, h)
    h = np.where(mag > np.uint32(0x7F800000), sign | np.uint16(0x7C00), h)
    return h.astype(np.uint16)


def np_cache_f16(x: np.ndarray) -> np.ndarray:
    """Value map of the cache's f16 round trip, via numpy."""
    return np_cache_f16_bits(x).view(np.float16).astype(np.float32)


def max_rel(got: np.ndarray, want: np.ndarray) -> float:
    """The reference's error measure, crates/breccia-kernels/tests/attn_conformance.rs:102-108:
    max |g - w| / max(|w|, 1)."""
    g = np.asarray(got, dtype=np.float64)
    w = np.asarray(want, dtype=np.float64)
    return float(np.max(np.abs(g - w) / np.maximum(np.abs(w), 1.0))) if g.size else 0.0


def max_abs(got: np.ndarray, want: np.ndarray) -> float:
    g = np.asarray(got, dtype=np.float64)
    w = np.asarray(want, dtype=np.float64)
    return float(np.max(np.abs(g - w))) if g.size else 0.0
