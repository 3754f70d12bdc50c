"""The allocation-free argmax entry point (rai_hip_argmax_static) against rai_hip_argmax, through the C ABI.

Its partial results live in a fixed device array that every call on the GPU shares and that keeps the last call's
contents, so the second call here is smaller than the first and must not see the first one's leftovers."""
import numpy as np
import pytest

from oracle import ops as oo
from oracle.dtypes import rnd
from rai_amd._lib import RaiHipError
from rai_amd.hip import HipTensor
from tests.util import down, up

pytestmark = pytest.mark.gpu


def _mallocs(hip):
    import ctypes as C
    from rai_amd import _lib
    a, b, n = C.c_uint64(0), C.c_uint64(0), C.c_uint64(0)
    _lib.call("rai_hip_mem_stats", 0, C.byref(a), C.byref(b), C.byref(n))
    return n.value


@pytest.mark.parametrize("dt", ["bf16", "f32", "f64"])
def test_argmax_static_equals_argmax_two_calls_second_smaller(hip, dt):
    from rai_amd import ops
    g = np.random.Generator(np.random.PCG64(41))
    # few distinct values: many exact ties, the first index must win; rows x long axis -> the split row kernel
    big = rnd(np.round(g.standard_normal((64, 51200)) * 3).astype(np.float32), dt)
    small = rnd(np.round(g.standard_normal((5, 7000)) * 3).astype(np.float32), dt)
    xb, xs = up(big, dt), up(small, dt)
    ob, os_ = HipTensor.empty((64,), "u32"), HipTensor.empty((5,), "u32")
    want_b, want_s = down(ops.argmax(xb, -1)), down(ops.argmax(xs, -1))     # the existing entry point
    before = _mallocs(hip)
    got_b = down(ops.argmax_static(xb, -1, ob))
    got_s = down(ops.argmax_static(xs, -1, os_))                            # second call, smaller input
    assert _mallocs(hip) == before, "the allocation-free entry point allocated device memory"
    assert np.array_equal(got_b, want_b) and np.array_equal(got_b, oo.argmax(big, -1))
    assert np.array_equal(got_s, want_s) and np.array_equal(got_s, oo.argmax(small, -1))
    # one row with a very long axis: the axis is cut into many splits
    one = rnd(g.standard_normal((1, 300000)).astype(np.float32), dt)
    o1 = HipTensor.empty((1, 1), "u32")
    assert np.array_equal(down(ops.argmax_static(up(one, dt), 1, o1, keep_dim=True)), oo.argmax(one, 1, True))


def test_argmax_static_short_axis_and_limit(hip):
    from rai_amd import ops
    g = np.random.Generator(np.random.PCG64(42))
    a = g.integers(0, 9, (70, 9)).astype(np.uint32)                         # thread-per-output kernel, no scratch
    out = HipTensor.empty((9,), "u32")
    assert np.array_equal(down(ops.argmax_static(up(a, "u32"), 0, out)), oo.argmax(a, 0))
    # more rows than the fixed array has partial-result slots: a clear error, nothing launched
    wide = up(np.zeros((65537, 1024), np.float32), "f32")
    with pytest.raises(RaiHipError) as e:
        ops.argmax_static(wide, 1, HipTensor.empty((65537,), "u32"))
    assert e.value.status == -7 and "static scratch holds" in str(e.value)
    assert not down(ops.argmax(wide, 1)).any()     # the allocating entry point takes it (two launches, grown workspace)
    ok = up(np.zeros((65536, 1024), np.float32), "f32")
    assert not down(ops.argmax_static(ok, 1, HipTensor.empty((65536,), "u32"))).any()
