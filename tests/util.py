"""Shared helpers for the GPU parity tests."""
import numpy as np


def assert_close(got, want, rel=1e-4, what=""):
    """The parity bar for fp32 ops: |got - want| <= rel * (|want| + rms(want)) element-wise, i.e. 1e-4 relative with
    the tensor's own scale as the floor for entries near zero."""
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
    bound = rel * (np.abs(w) + rms) + 1e-30
    bad = err > bound
    assert not bad.any(), f"{what}: {int(bad.sum())}/{g.size} outside rel {rel}; worst err {err.max():.3e} (rms {rms:.3e})"
