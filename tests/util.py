"""Helpers shared by the parity tests: upload/download in storage dtypes and the
tolerances of the correctness bar (f32: 1e-4 relative, bf16: 2e-2 relative,
integers and indices: bit-exact)."""
import numpy as np

from oracle.dtypes import from_storage, rnd, to_storage
from rai_amd.hip import HipTensor

RTOL = {"f32": 1e-4, "f64": 1e-9, "bf16": 2e-2, "f16": 4e-3}


def up(arr, dt):
    """Carrier array (values representable in dt) -> device tensor."""
    return HipTensor.from_storage(to_storage(arr, dt), dt)


def down(t):
    return t.to_float()


def rand(rng, shape, dt, scale=1.0):
    return rnd(rng.standard_normal(shape).astype(np.float64 if dt == "f64" else np.float32) * scale, dt)


def assert_close(got, want, dt, what="", scale=None):
    """|got - want| <= rtol * max(|want|, scale) elementwise, where scale defaults
    to the largest magnitude of `want` (tensor-relative error)."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, f"{what}: shape {got.shape} vs {want.shape}"
    if want.size == 0:
        return
    fin = np.isfinite(want)
    assert np.array_equal(np.isfinite(got), fin), f"{what}: non-finite pattern differs"
    assert np.array_equal(got[~fin], want[~fin]) or np.all(np.isnan(want[~fin]) == np.isnan(got[~fin])), what
    if not fin.any():
        return
    s = float(np.max(np.abs(want[fin]))) if scale is None else scale
    tol = RTOL[dt] * max(s, 1e-30)
    err = np.abs(got[fin] - want[fin])
    bad = err > tol
    assert not bad.any(), f"{what}: max err {err.max():.3e} > tol {tol:.3e} ({bad.sum()} of {err.size} elements)"
