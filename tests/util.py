"""Helpers shared by the parity tests: upload/download in storage dtypes and the
tolerances of the correctness bar (f32: 1e-4 relative, bf16: 2e-2 relative,
integers and indices: bit-exact).  Two forms: assert_close bounds the error by the
largest magnitude of the expected tensor (contractions, reductions, norms, logits);
assert_close_elem bounds every element by its own magnitude (unary, binary, cast,
activations, RoPE)."""
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


# Per-element bound for elementwise work (unary, binary, cast, activations, RoPE): relative to each element's own
# magnitude, with an absolute floor far below the values in play, so that an error on a small element cannot hide
# behind the largest one of the tensor.
ELEM_RTOL = {"f32": 1e-4, "f64": 1e-9, "bf16": 2e-2, "f16": 4e-3}


def assert_close_elem(got, want, dt, what="", atol=None):
    """|got - want| <= rtol * |want| + atol for every element (atol defaults to rtol * 1e-3 * max|want|)."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, f"{what}: shape {got.shape} vs {want.shape}"
    if want.size == 0:
        return
    fin = np.isfinite(want)
    assert np.array_equal(np.isfinite(got), fin), f"{what}: non-finite pattern differs"
    assert np.array_equal(np.isnan(got), np.isnan(want)), f"{what}: NaN pattern differs"
    assert np.array_equal(got[~fin & ~np.isnan(want)], want[~fin & ~np.isnan(want)]), f"{what}: infinities differ"
    if not fin.any():
        return
    rtol = ELEM_RTOL[dt]
    if atol is None:
        atol = rtol * 1e-3 * float(np.max(np.abs(want[fin])))
    err = np.abs(got[fin] - want[fin])
    bound = rtol * np.abs(want[fin]) + atol
    bad = err > bound
    if bad.any():
        i = int(np.argmax(err - bound))
        raise AssertionError(f"{what}: {bad.sum()} of {err.size} elements off; worst: got {got[fin][i]!r} want "
                             f"{want[fin][i]!r} (err {err[i]:.3e} > {bound[i]:.3e})")


def progress(request, msg):
    """One line on the real stdout, past pytest's capture: long tests show they are alive."""
    cap = request.config.pluginmanager.getplugin("capturemanager")
    if cap is None:
        print(msg, flush=True)
        return
    with cap.global_and_fixture_disabled():
        print(f"\n[{request.node.name}] {msg}", end="", flush=True)


def synthetic_params(shapes, dt, seed=0, std=0.02, norm_weight=1.0, workers=8):
    """The benchmark's seeded weights (rai_amd.synthetic: N(0, std) per tensor from PCG64(seed, crc32(name)), zero
    biases, constant norm weights) as a dict name -> carrier array already rounded to dt, generated in threads."""
    from concurrent.futures import ThreadPoolExecutor

    from rai_amd import synthetic

    def make(item):
        name, shape = item
        n = int(np.prod(shape))
        if name.endswith("norm.weight"):
            a = np.full(n, norm_weight, np.float32)
        else:
            a = synthetic.tensor(name, n, seed, std)
        return name, rnd(a, dt).reshape(shape)

    with ThreadPoolExecutor(max_workers=workers) as ex:
        return dict(ex.map(make, shapes.items()))


def assert_logits_close(got, chain, exact, dt, what=""):
    """For whole-model logits at full width, where the reference's node-by-node evaluation in bf16 (`chain`: every
    primitive's result rounded to the storage dtype) is itself a few per cent away from the same computation without
    intermediate rounding (`exact`: the same stored weights, rotary tables and inputs, f32 arithmetic).  Measured on
    the 32-layer Phi-2 widths over a 512-token prefill and 12 steps: chain vs exact 1.5-3.0 % of the largest logit,
    device vs exact 1.0-2.8 %, device vs chain 1.3-2.6 %: three bf16 evaluations of the same weights, each about as far
    from the others as the dtype's tolerance after that many layers.  Whole-model logits are therefore held to one and
    a half times the dtype's tolerance, against `exact` and against `chain` alike: a fixed bound that does not grow
    with what the chain happens to measure.  Layer by layer, where no noise builds up, the chain itself is the
    reference at the plain tolerance (the single-layer tests), and so it is for every model shallow enough
    (assert_close).  Errors are relative to the largest magnitude of the expected logits, as in assert_close."""
    got, chain, exact = (np.asarray(a, dtype=np.float64) for a in (got, chain, exact))
    assert got.shape == chain.shape == exact.shape, f"{what}: shapes {got.shape} {chain.shape} {exact.shape}"
    assert np.isfinite(got).all(), f"{what}: non-finite logits"
    scale = float(np.max(np.abs(exact)))
    tol = RTOL[dt] * scale
    e_dev, e_chain, e_dc = (float(np.max(np.abs(a - b))) for a, b in ((got, exact), (chain, exact), (got, chain)))
    bound = 1.5 * tol
    assert e_dev <= bound, (f"{what}: device vs unrounded reference arithmetic {e_dev:.3e} > 1.5 x {tol:.3e} "
                            f"(chain vs the same {e_chain:.3e})")
    assert e_dc <= bound, (f"{what}: device vs node-by-node chain {e_dc:.3e} > 1.5 x {tol:.3e} "
                           f"(chain vs unrounded arithmetic {e_chain:.3e})")
    return e_dev / scale, e_chain / scale, e_dc / scale
