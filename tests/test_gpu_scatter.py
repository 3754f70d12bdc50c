"""gather / index_add / scatter_add on the device against the CPU oracle, through the C ABI: bit-exact
for every dtype, duplicates included (the device kernels add in source order and round to the storage
dtype after every addition, as the oracle's sequential loops do).  Shapes follow rai-core/tests/ops.rs
and tests/check_grad.rs plus the embedding-gradient shape at reduced size."""
import numpy as np
import pytest

from oracle import ops as oo
from rai_amd._lib import RaiHipError
from tests.util import rand, up

pytestmark = pytest.mark.gpu

DTYPES = ["u8", "u32", "i64", "f16", "bf16", "f32", "f64"]
NP_INT = {"u8": np.uint8, "u32": np.uint32, "i64": np.int64}


@pytest.fixture(scope="module")
def R(hip):
    from rai_amd import ops
    return ops


def rng(seed):
    return np.random.Generator(np.random.PCG64(seed))


def values(g, shape, dt):
    if dt in NP_INT:
        return g.integers(0, 200, shape).astype(NP_INT[dt])
    return rand(g, shape, dt, 4.0)


def same_bits(dev_tensor, want, dt):
    assert np.array_equal(dev_tensor.to_storage(), up(want, dt).to_storage())


def test_gather_known_answer(R):
    # rai-core/tests/ops.rs:156-161
    a = up(np.array([[1, 2, 3], [4, 5, 6]], np.uint32), "u32")
    idx = up(np.array([[0, 0, 0], [1, 1, 1]], np.uint32), "u32")
    assert np.array_equal(R.gather(a, 0, idx).to_storage(), [[1, 2, 3], [4, 5, 6]])


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("idt", ["u8", "u32", "i64"])
def test_gather_bit_exact(R, dt, idt):
    g = rng(31)
    x = values(g, (3, 50, 7), dt)
    for dim, shape in [(0, (5, 50, 7)), (1, (3, 131, 7)), (-1, (3, 50, 2)), (1, (3, 0, 7))]:
        ix = g.integers(0, x.shape[dim], shape).astype(NP_INT[idt])
        same_bits(R.gather(up(x, dt), dim, up(ix, idt)), oo.gather(x, dim, ix), dt)
    assert R.index_errors() == 0


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("idt", ["u8", "u32", "i64"])
def test_index_add_bit_exact_with_duplicates(R, dt, idt):
    g = rng(32)
    for xshape, dim, L in [((4, 2), 1, 3), ((40, 264), 0, 700), ((3, 9, 5), 1, 20), ((2, 6, 1100), 1, 11), ((5, 4), 0, 0)]:
        x = values(g, xshape, dt)
        sshape = list(xshape)
        sshape[dim] = L
        src = values(g, sshape, dt)
        ix = g.integers(0, xshape[dim], L).astype(NP_INT[idt])      # heavy duplication: L > extent in two cases
        same_bits(R.index_add(up(x, dt), dim, up(ix, idt), up(src, dt)), oo.index_add(x, dim, ix, src, dt), dt)
    assert R.index_errors() == 0


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("idt", ["u8", "u32", "i64"])
def test_scatter_add_bit_exact_with_duplicates(R, dt, idt):
    g = rng(33)
    # J <= 32 takes the per-element kernel, larger J the per-column kernel
    for xshape, dim, J in [((2, 2), 1, 2), ((6, 40, 9), 1, 5), ((6, 40, 9), 1, 77), ((30, 8), 0, 300), ((4, 17), 1, 1),
                           ((4, 17), 1, 0), ((3, 5, 6), 2, 33)]:
        x = values(g, xshape, dt)
        ishape = list(xshape)
        ishape[dim] = J
        ix = g.integers(0, xshape[dim], ishape).astype(NP_INT[idt])
        src = values(g, ishape, dt)
        same_bits(R.scatter_add(up(x, dt), dim, up(ix, idt), up(src, dt)), oo.scatter_add(x, dim, ix, src, dt), dt)
    assert R.index_errors() == 0


def test_bf16_sums_round_after_every_addition(R):
    x = np.array([[256.0]], np.float32)
    one = np.ones((2, 1), np.float32)
    i2 = np.array([0, 0], np.uint32)
    assert R.index_add(up(x, "bf16"), 0, up(i2, "u32"), up(one, "bf16")).to_float()[0, 0] == 256.0
    assert R.scatter_add(up(x, "bf16"), 0, up(i2.reshape(2, 1), "u32"), up(one, "bf16")).to_float()[0, 0] == 256.0
    assert R.index_add(up(x, "f32"), 0, up(i2, "u32"), up(one, "f32")).to_float()[0, 0] == 258.0


def test_embedding_gradient_shape(R):
    # the vjp of Embedding::fwd (rai-nn/src/embedding.rs:25-30 through ops/index_select.rs:40-48): cotangent rows
    # added into a zero table at the token ids, many ids repeated
    g = rng(34)
    vocab, hidden, n = 3000, 2560, 4096
    ids = g.integers(0, vocab, n).astype(np.uint32)
    ids[: n // 2] = g.integers(0, 16, n // 2)            # a few very frequent tokens
    ct = rand(g, (n, hidden), "bf16")
    zero = np.zeros((vocab, hidden), np.float32)
    got = R.index_add(up(zero, "bf16"), 0, up(ids, "u32"), up(ct, "bf16"))
    same_bits(got, oo.index_add(zero, 0, ids, ct, "bf16"), "bf16")


def test_out_of_range_indices_are_reported(R):
    x = np.arange(12, dtype=np.float32).reshape(4, 3)
    got = R.gather(up(x, "f32"), 0, up(np.array([[0, 4, 1]], np.uint32), "u32")).to_float()
    assert np.array_equal(got, [[0, 0, 5]])
    assert R.index_errors() == 1
    got = R.index_add(up(x, "f32"), 0, up(np.array([1, 9], np.uint32), "u32"), up(np.ones((2, 3), np.float32), "f32")).to_float()
    want = x.copy()
    want[1] += 1
    assert np.array_equal(got, want) and R.index_errors() == 1
    for J in (1, 40):                                   # both scatter kernels
        ix = np.zeros((J, 3), np.uint32)
        ix[0, 1] = 7
        got = R.scatter_add(up(x, "f32"), 0, up(ix, "u32"), up(np.ones((J, 3), np.float32), "f32")).to_float()
        want = x.copy()
        want[0] += J
        want[0, 1] -= 1
        assert np.array_equal(got, want) and R.index_errors() == 1
    assert R.index_errors() == 0


def test_shape_and_dtype_errors(R):
    x = up(np.zeros((4, 3), np.float32), "f32")
    with pytest.raises(RaiHipError):
        R.gather(x, 0, up(np.zeros((2, 2), np.uint32), "u32"))                 # extent off dim differs
    with pytest.raises(RaiHipError):
        R.gather(x, 0, up(np.zeros((2, 3), np.float32), "f32"))                # float index
    with pytest.raises(RaiHipError):
        R.index_add(x, 0, up(np.zeros((2,), np.uint32), "u32"), up(np.zeros((3, 3), np.float32), "f32"))
    with pytest.raises(RaiHipError):
        R.index_add(x, 0, up(np.zeros((2, 1), np.uint32), "u32"), up(np.zeros((2, 3), np.float32), "f32"))
    with pytest.raises(RaiHipError):
        R.scatter_add(x, 0, up(np.zeros((2, 3), np.uint32), "u32"), up(np.zeros((2, 2), np.float32), "f32"))
    with pytest.raises(RaiHipError):
        R.scatter_add(x, 0, up(np.zeros((2, 3), np.uint32), "u32"), up(np.zeros((2, 3), np.float64), "f64"))
    with pytest.raises(RaiHipError):
        R.gather(x.transpose(0, 1), 0, up(np.zeros((3, 4), np.uint32), "u32"))  # non-contiguous x
