"""Shared helpers for the GPU parity tests."""
import numpy as np


def assert_close(got, want, rel=1e-4, what="", scale=0.0, outlier_frac=0.0, outlier_abs=0.0):
    """The parity bar for fp32 ops: |got - want| <= rel * (|want| + rms(want)) element-wise, i.e. 1e-4 relative with
    the tensor's own scale as the floor for entries near zero.  `scale` raises that floor to the magnitude of the
    terms that cancel when the result is a small difference of large numbers (e.g. LayerNorm dx on a 2-wide row)."""
    got = np.asarray(got, dtype=np.float64).reshape(-1)
    want = np.asarray(want, dtype=np.float64).reshape(-1)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    assert np.all(np.isfinite(got) == np.isfinite(want)), what
    fin = np.isfinite(want)
    assert np.array_equal(got[~fin], want[~fin], equal_nan=True), what
    g, w = got[fin], want[fin]
    if g.size == 0:
        return
    rms = float(np.sqrt(np.mean(w * w)))
    err = np.abs(g - w)
    bound = rel * (np.abs(w) + max(rms, scale)) + 1e-30
    bad = err > bound
    if outlier_frac > 0.0:
        # ill-conditioned entries (e.g. Adam's g/(|g|+eps) where a gradient cancels to ~eps): a bounded fraction may
        # miss the tight bound but must stay within `outlier_abs`
        assert bad.mean() <= outlier_frac and (not bad.any() or err[bad].max() <= outlier_abs), \
            f"{what}: {int(bad.sum())}/{g.size} outliers, worst {err.max():.3e} (allowed {outlier_frac:.1e} of entries within {outlier_abs:.1e})"
        return
    assert not bad.any(), f"{what}: {int(bad.sum())}/{g.size} outside rel {rel}; worst err {err.max():.3e} (rms {rms:.3e})"


def py_dropout_hash(seed: int, counter: int, index: int) -> int:
    """DropoutRng.hash (packages/autograd/src/ops.ts:74-81) restated with Python floats (IEEE doubles, like a JS number) for
    the first line and arbitrary-precision ints for ToInt32 and Math.imul; returns the final h >>> 0.  Independent of the
    oracle's C version (no fmod, no fixed-width integer types)."""
    d = float(seed) + float(counter) * 2654435761.0 + float(index) * 2246822519.0    # left to right, one rounding per operation
    h = int(d) & 0xFFFFFFFF                                                           # ToInt32 keeps the low 32 bits (two's complement)
    h = ((h ^ (h >> 16)) * 0x85EBCA6B) & 0xFFFFFFFF
    h = ((h ^ (h >> 13)) * 0xC2B2AE35) & 0xFFFFFFFF
    return h ^ (h >> 16)


def py_dropout_mask(seed: int, counter: int, p: float, indices) -> np.ndarray:
    """DropoutRng.nextMask (ops.ts:41-51) for the given element indices."""
    keep = np.float32(1 / (1 - p))
    return np.array([keep if py_dropout_hash(seed, counter, int(i)) / 4294967296 > p else np.float32(0) for i in indices], np.float32)
