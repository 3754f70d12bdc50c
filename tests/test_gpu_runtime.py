"""The device allocator behind every tensor (rai_hip_alloc / retain / release / trim / mem_stats): ref-counted blocks,
a size-class pool that hands a released block out again, blocks of up to 32 MiB cut from slabs (no hipMalloc per new
size), whole blocks returned to the driver by trim."""
import ctypes as C

import pytest

from rai_amd import _lib

pytestmark = pytest.mark.gpu


def stats():
    a, b, n = C.c_uint64(), C.c_uint64(), C.c_uint64()
    _lib.call("rai_hip_mem_stats", 0, C.byref(a), C.byref(b), C.byref(n))
    return a.value, b.value, n.value


def alloc(nbytes):
    p = C.c_void_p()
    _lib.call("rai_hip_alloc", 0, nbytes, C.byref(p))
    return p


def test_small_blocks_are_cut_from_slabs_and_pooled(hip):
    in_use0, pooled0, n0 = stats()
    # twenty sizes the pool has not seen: at most one slab's worth of hipMalloc
    sizes = [3_000_017 + 700_001 * i for i in range(20)]
    blocks = [alloc(s) for s in sizes]
    in_use1, pooled1, n1 = stats()
    assert n1 - n0 <= 2, (n0, n1)
    assert in_use1 - in_use0 >= sum(sizes)
    addrs = sorted(b.value for b in blocks)
    assert all(a % 512 == 0 for a in addrs) and len(set(addrs)) == len(addrs)
    for b in blocks:
        _lib.call("rai_hip_release", b)
    in_use2, pooled2, _ = stats()
    # everything taken is back in the pool (a warm pool may have served some of the requests itself)
    assert in_use2 == in_use0 and pooled2 - pooled1 >= sum(sizes) and pooled2 >= pooled0
    # the same sizes again come out of the pool: no hipMalloc, the same addresses
    again = [alloc(s) for s in sizes]
    assert stats()[2] == n1
    assert sorted(b.value for b in again) == addrs
    # a second reference keeps a block alive
    _lib.call("rai_hip_retain", again[0])
    for b in again:
        _lib.call("rai_hip_release", b)
    assert stats()[0] > in_use0            # again[0] is still held once
    _lib.call("rai_hip_release", again[0])
    assert stats()[0] == in_use0
    # trim keeps what was cut from a slab and hands whole blocks back
    big = alloc(96 << 20)
    _, _, n3 = stats()
    _lib.call("rai_hip_release", big)
    _, pooled3, _ = stats()
    _lib.call("rai_hip_trim", 0)
    _, pooled4, _ = stats()
    assert pooled3 - pooled4 >= (96 << 20) and pooled4 >= pooled2 - pooled1
    with pytest.raises(_lib.RaiHipError):
        _lib.call("rai_hip_release", C.c_void_p(12345))
