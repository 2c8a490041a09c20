"""Comparison helpers shared by the GPU parity tests."""
import numpy as np


def rel_err_f32(got, want):
    """Max of |g-w| / max(|w|, floor) with floor = 1e-3 * rms(want): the strict
    relative error, except that outputs which cancel to (almost) zero are
    measured against a thousandth of the tensor's scale instead of themselves."""
    got = np.asarray(got, np.float64).ravel()
    want = np.asarray(want, np.float64).ravel()
    if got.size == 0:
        return 0.0
    floor = 1e-3 * float(np.sqrt(np.mean(want * want))) + 1e-30
    return float(np.max(np.abs(got - want) / np.maximum(np.abs(want), floor))) if got.size else 0.0


def rel_err_strict(got, want, min_rel=1e-3):
    """Max of |g-w| / |w| over the elements with |w| > min_rel * rms(want), no floor: the strict element-wise relative
    error wherever an output has not cancelled to (almost) nothing.  The elements it leaves out are held to the
    reference's idiom (close_idiom) by the callers."""
    got = np.asarray(got, np.float64).ravel()
    want = np.asarray(want, np.float64).ravel()
    if got.size == 0:
        return 0.0
    big = np.abs(want) > min_rel * float(np.sqrt(np.mean(want * want)))
    return float(np.max(np.abs(got[big] - want[big]) / np.abs(want[big]))) if big.any() else 0.0


def close_idiom(got, want):
    """The reference's own closeness idiom, |a-b| < 1e-5 * (1 + |b|)
    (crates/allpaka-backend/src/ops/mod.rs:25-27), over whole arrays."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    return bool(np.all(np.abs(got - want) < 1e-5 * (1.0 + np.abs(want))))


def f16_ulp_diff(got_bits, want_bits):
    """Max distance in units of fp16 codes (monotone integer mapping of the bit patterns)."""
    def key(b):
        b = np.asarray(b, np.uint16).astype(np.int32).ravel()
        return np.where(b & 0x8000, 0x8000 - b, b)
    g, w = key(got_bits), key(want_bits)
    return int(np.max(np.abs(g - w))) if g.size else 0
