"""Parity of every HIP primitive with the CPU oracle, through the C ABI.

The cases follow the reference's own op tests (rai-core/tests/ops.rs,
tests/eval.rs: same op list, small shapes, broadcasting and strided views) plus
the op-sweep shapes of the benchmark configuration at reduced size.
"""
import numpy as np
import pytest

from oracle import nn as onn
from oracle import ops as oo
from oracle.dtypes import rnd
from tests.util import assert_close, assert_close_elem, down, rand, up

pytestmark = pytest.mark.gpu

FLOATS = ["f32", "bf16", "f16", "f64"]


@pytest.fixture(scope="module")
def R(hip):
    from rai_amd import ops
    return ops


def rng(seed=1):
    return np.random.Generator(np.random.PCG64(seed))


# ------------------------------------------------------------------ creation / known answers
def test_full_arange_known_answers(R):
    # rai-core/tests/ops.rs:19-29 (test_arange) and Tensor::full / ones
    assert np.array_equal(down(R.arange(0, 10, 1, "f32")), np.arange(10, dtype=np.float32))
    assert np.array_equal(down(R.arange(10, 20, 2, "f32")), np.arange(10, 20, 2, dtype=np.float32))
    assert np.array_equal(down(R.arange(0, 10, 3, "u8")), np.array([0, 3, 6, 9], dtype=np.uint8))
    for dt in ["u8", "u32", "i64", "f16", "bf16", "f32", "f64"]:
        got = down(R.full(3, (2, 3), dt))
        assert got.shape == (2, 3) and np.all(got == 3)
    assert_close(down(R.full(1.4, (2, 3), "bf16")), rnd(np.full((2, 3), 1.4, np.float32), "bf16"), "bf16")


def test_eval_known_answer(R):
    # rai-core/tests/eval.rs:30-47: 1/2 + 2*3 - (3.1 + 3.2) = 0.2
    f = lambda v: R.full(v, (2, 2), "f32")
    z = R.binary("sub", R.binary("add", R.binary("div", f(1), f(2)), R.binary("mul", f(2), f(3))),
                 R.binary("add", f(3.1), f(3.2)))
    assert_close(down(z), np.full((2, 2), 0.2, np.float32), "f32")
    # tests/eval.rs:4-12: ones + ones + ones[3] = 3
    z = R.binary("add", R.binary("add", R.full(1, (2, 3), "f32"), R.full(1, (2, 3), "f32")), R.full(1, (3,), "f32"))
    assert np.array_equal(down(z), np.full((2, 3), 3, np.float32))


def test_matmul_known_answer(R):
    # rai-core/tests/ops.rs:80-91: ones[2,3] @ ones[3,2] = 3; :93-104 ones[2,3] @ ones[3]
    assert np.array_equal(down(R.matmul(R.full(1, (2, 3), "f32"), R.full(1, (3, 2), "f32"))), np.full((2, 2), 3.0))
    assert np.array_equal(down(R.matmul(R.full(1, (2, 3), "f32"), R.full(1, (3,), "f32"))), np.full((2,), 3.0))


def test_index_select_known_answer(R):
    # rai-core/tests/ops.rs:167-175
    t = up(np.array([[1, 2, 3], [4, 5, 6]], np.float32), "f32")
    idx = R.from_array(np.array([1, 1, 0, 0], np.uint32), "u32")
    assert np.array_equal(down(R.index_select(t, 0, idx)), np.array([[4, 5, 6], [4, 5, 6], [1, 2, 3], [1, 2, 3]]))
    assert np.array_equal(down(R.index_select(t, 1, R.from_array(np.array([2, 0], np.uint8), "u8"))),
                          np.array([[3, 1], [6, 4]]))


# ------------------------------------------------------------------ cast
@pytest.mark.parametrize("src", ["u8", "u32", "i64", "f16", "bf16", "f32", "f64"])
@pytest.mark.parametrize("dst", ["u8", "u32", "i64", "f16", "bf16", "f32", "f64"])
def test_cast(R, src, dst):
    g = rng(3)
    if src in FLOATS:
        a = g.uniform(-300, 300, (5, 37)).astype(np.float64 if src == "f64" else np.float32)
        a[0, :4] = [0.5, -0.5, 255.7, -3.9]
        a = rnd(a, src)
    else:
        hi = {"u8": 255, "u32": 100000, "i64": 100000}[src]
        a = g.integers(0, hi, (5, 37)).astype({"u8": np.uint8, "u32": np.uint32, "i64": np.int64}[src])
    got = down(R.to_dtype(up(a, src), dst))
    want = oo.to_dtype(a, src, dst)
    if dst in FLOATS:
        assert np.array_equal(np.asarray(got, np.float64), np.asarray(want, np.float64)), (src, dst)
    else:
        assert np.array_equal(got, want), (src, dst)


def test_cast_bf16_rounding_is_nearest_even(R):
    # values exactly between two bf16 neighbours must go to the even mantissa
    bits = np.array([0x3F808000, 0x3F818000, 0x3F80FFFF, 0x7F7FFFFF, 0x00000001, 0xBF808000], np.uint32)
    a = bits.view(np.float32)
    got = R.to_dtype(up(a, "f32"), "bf16").to_storage()
    assert list(got) == [0x3F80, 0x3F82, 0x3F81, 0x7F80, 0x0000, 0xBF80]


# ------------------------------------------------------------------ unary / binary
UNARY = ["sin", "cos", "neg", "square", "sqrt", "rsqrt", "abs", "exp", "log", "log2", "log10", "erf", "tanh", "sign"]
ORACLE_UN = {"sin": oo.sin, "cos": oo.cos, "neg": oo.neg, "square": oo.square, "sqrt": oo.sqrt, "rsqrt": oo.rsqrt,
             "abs": oo.abs_, "exp": oo.exp, "log": oo.log, "log2": oo.log2, "log10": oo.log10, "erf": oo.erf,
             "tanh": oo.tanh, "sign": oo.sign}


@pytest.mark.parametrize("dt", FLOATS)
@pytest.mark.parametrize("op", UNARY)
def test_unary(R, op, dt):
    a = rand(rng(5), (7, 130), dt, 2.0)
    if op in ("sqrt", "rsqrt", "log", "log2", "log10"):
        a = rnd(np.abs(a) + 0.01, dt)
    assert_close_elem(down(R.unary(op, up(a, dt))), ORACLE_UN[op](a, dt), dt, op)


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_unary_strided_input(R, dt):
    a = rand(rng(6), (6, 10, 16), dt)
    got = down(R.unary("exp", up(a, dt).transpose(0, 2).narrow(1, 2, 5)))
    assert_close_elem(got, oo.exp(np.swapaxes(a, 0, 2)[:, 2:7], dt), dt)


@pytest.mark.parametrize("dt", FLOATS)
def test_powf(R, dt):
    a = rnd(np.abs(rand(rng(7), (33, 65), dt)) + 0.1, dt)
    for e in (3.0, 0.5, -1.5):
        assert_close_elem(down(R.unary("powf", up(a, dt), e)), oo.powf(a, e, dt), dt, f"powf {e}")


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("act", ["gelu", "new_gelu", "silu", "relu"])
def test_fused_activation_matches_reference_chain(R, act, dt):
    # fused single-rounding kernel vs the reference's primitive chain (hlops/activations.rs)
    a = rand(rng(8), (64, 256), dt, 2.0)
    want = {"gelu": onn.gelu, "new_gelu": onn.new_gelu, "silu": onn.silu, "relu": onn.relu}[act](a, dt)
    # per element; the absolute floor is one rounding of the chain's largest intermediate (the reference rounds
    # tanh / erf / exp to the dtype before adding 1, which is an absolute, not a relative, error on the result)
    floor = {"f32": 2.0 ** -22, "bf16": 2.0 ** -8}[dt] * float(np.max(np.abs(a)))
    assert_close_elem(down(R.unary(act, up(a, dt))), want, dt, act, atol=floor)


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_new_gelu_primitive_chain(R, dt):
    # the same composition rai builds node by node, every node evaluated on the device
    a = rand(rng(9), (16, 128), dt, 2.0)
    x = up(a, dt)
    c = lambda v: R.to_dtype(R.full(v, x.shape, "f32"), dt)
    k = float(np.sqrt(np.float32(2.0) / np.float32(np.pi)))
    inner = R.binary("add", x, R.binary("mul", c(0.044715), R.unary("powf", x, 3.0)))
    t = R.unary("tanh", R.binary("mul", c(k), inner))
    y = R.binary("mul", R.binary("mul", c(0.5), x), R.binary("add", c(1.0), t))
    # node by node the device rounds where the reference rounds: only the library functions (powf, tanh) may differ,
    # by an ulp of their own result
    floor = {"f32": 2.0 ** -22, "bf16": 2.0 ** -8}[dt] * float(np.max(np.abs(a)))
    assert_close_elem(down(y), onn.new_gelu(a, dt), dt, "new_gelu chain", atol=floor)


BINARY = {"add": oo.add, "sub": oo.sub, "mul": oo.mul, "div": oo.div, "maximum": oo.maximum, "minimum": oo.minimum}
COMPARE = {"eq": oo.eq, "ne": oo.ne, "gt": oo.gt, "ge": oo.ge, "lt": oo.lt, "le": oo.le}


@pytest.mark.parametrize("dt", FLOATS)
@pytest.mark.parametrize("op", list(BINARY))
def test_binary_broadcast(R, op, dt):
    g = rng(10)
    a, b = rand(g, (4, 1, 96), dt), rand(g, (5, 96), dt)
    if op == "div":
        b = rnd(np.abs(b) + 0.5, dt)
    assert_close_elem(down(R.binary(op, up(a, dt), up(b, dt))), BINARY[op](a, b, dt), dt, op)
    # bias-style broadcast [M, N] + [N] and scalar-like [1]
    c = rand(g, (96,), dt)
    assert_close_elem(down(R.binary(op, up(a, dt), up(rnd(np.abs(c) + 0.5, dt), dt))),
                      BINARY[op](a, rnd(np.abs(c) + 0.5, dt), dt), dt, op)


@pytest.mark.parametrize("dt", ["u8", "u32", "i64"])
def test_binary_integers_exact(R, dt):
    g = rng(11)
    npdt = {"u8": np.uint8, "u32": np.uint32, "i64": np.int64}[dt]
    a = g.integers(0, 200, (9, 17)).astype(npdt)
    b = g.integers(1, 50, (17,)).astype(npdt)
    for op in BINARY:
        assert np.array_equal(down(R.binary(op, up(a, dt), up(b, dt))), BINARY[op](a, b, dt)), (op, dt)


@pytest.mark.parametrize("dt", ["f32", "bf16", "u32"])
def test_compare_and_where(R, dt):
    g = rng(12)
    if dt == "u32":
        a, b = g.integers(0, 5, (8, 33)).astype(np.uint32), g.integers(0, 5, (33,)).astype(np.uint32)
    else:
        a, b = rnd(np.round(rand(g, (8, 33), dt)), dt), rnd(np.round(rand(g, (33,), dt)), dt)
    for op, f in COMPARE.items():
        got = down(R.binary(op, up(a, dt), up(b, dt)))
        assert got.dtype == np.uint8 and np.array_equal(got, f(a, b, dt)), op
    cond = oo.gt(a, b, dt)
    got = down(R.where(up(cond, "u8"), up(a, dt), up(b, dt)))
    want = oo.where(cond, a, b, dt)
    assert np.array_equal(np.asarray(got, np.float64), np.asarray(want, np.float64))


def test_where_masked_fill_neg_inf(R):
    # masked_fill of rai-models/src/llm/phi2.rs:111-117 on a causal u8 mask
    s = 17
    scores = rand(rng(13), (2, 3, s, s), "f32")
    mask = (np.arange(s)[None, :] > np.arange(s)[:, None]).astype(np.uint8)
    got = down(R.where(up(mask, "u8"), R.full(-np.inf, (s, s), "f32"), up(scores, "f32")))
    assert np.array_equal(got, np.where(mask != 0, np.float32(-np.inf), scores))


# ------------------------------------------------------------------ copy / views
@pytest.mark.parametrize("dt", ["u8", "u32", "i64", "bf16", "f32", "f64"])
def test_contiguous_of_views_and_concat(R, dt):
    g = rng(14)
    if dt in FLOATS:
        a = rand(g, (3, 4, 6, 8), dt)
    else:
        a = g.integers(0, 200, (3, 4, 6, 8)).astype({"u8": np.uint8, "u32": np.uint32, "i64": np.int64}[dt])
    x = up(a, dt)
    eq = lambda got, want: np.array_equal(np.asarray(got, np.float64), np.asarray(want, np.float64))
    assert eq(down(x.transpose(1, 2).contiguous()), np.swapaxes(a, 1, 2))
    assert eq(down(x.permute((3, 0, 2, 1)).contiguous()), np.transpose(a, (3, 0, 2, 1)))
    assert eq(down(x.narrow(2, 1, 4).contiguous()), a[:, :, 1:5])
    assert eq(down(x.narrow(3, 3, 5).transpose(0, 3).contiguous()), np.swapaxes(a[..., 3:8], 0, 3))
    assert eq(down(x.narrow(1, 0, 1).broadcast_to((3, 4, 6, 8)).contiguous()), np.broadcast_to(a[:, :1], a.shape))
    assert eq(down(x.transpose(1, 2).reshape((3, 24, 8))), np.swapaxes(a, 1, 2).reshape(3, 24, 8))
    # KV-cache style cat along dim 2 (rai-models/src/llm/phi2.rs:233-243) and rotate-half cat along -1
    assert eq(down(R.concatenate([x, x.narrow(2, 0, 1)], 2)), np.concatenate([a, a[:, :, :1]], 2))
    assert eq(down(R.concatenate([x.narrow(3, 4, 4), x.narrow(3, 0, 4)], -1)),
              np.concatenate([a[..., 4:], a[..., :4]], -1))


def test_to_device_copies_a_strided_view(R):
    # ToDevice<Hip> (backend/candle.rs:776-790): this box has one GPU, so source and target are the same device
    a = rand(rng(140), (6, 10, 16), "bf16")
    x = up(a, "bf16").transpose(0, 2).narrow(1, 2, 5)
    y = R.to_device(x, 0)
    assert y.is_contiguous() and y.buf.ptr != x.buf.ptr
    assert np.array_equal(down(y), np.swapaxes(a, 0, 2)[:, 2:7])


# ------------------------------------------------------------------ reductions
@pytest.mark.parametrize("dt", FLOATS)
@pytest.mark.parametrize("dims,keep", [((-1,), True), ((-1,), False), ((0,), False), ((1,), True), ((0, 2), False),
                                       (None, False)])
def test_reduce(R, dt, dims, keep):
    a = rand(rng(15), (6, 70, 130), dt)
    x = up(a, dt)
    d = None if dims is None else tuple(dims)
    assert_close(down(R.reduce("sum", x, d, keep)), oo.reduce_sum(a, d, keep, dt), dt, "sum",
                 scale=float(np.sqrt(a.size)))
    if d is not None and len(d) == 1:
        assert np.array_equal(down(R.reduce("max", x, d, keep)).astype(np.float64),
                              oo.reduce_max(a, d, keep, dt).astype(np.float64))
        assert np.array_equal(down(R.reduce("min", x, d, keep)).astype(np.float64),
                              oo.reduce_min(a, d, keep, dt).astype(np.float64))


def test_reduce_sum_u32_exact(R):
    a = rng(16).integers(0, 1000, (5, 300)).astype(np.uint32)
    assert np.array_equal(down(R.reduce("sum", up(a, "u32"), (1,), False)), a.sum(1, dtype=np.uint32))


@pytest.mark.parametrize("dt", FLOATS)
@pytest.mark.parametrize("shape,dim", [((4, 16, 2048), -1), ((3, 5, 129), -1), ((33, 3000), -1), ((7, 300, 9), 1),
                                       ((40, 6), 0), ((2, 1), -1)])
def test_softmax(R, dt, shape, dim):
    a = rand(rng(17), shape, dt, 3.0)
    got = down(R.softmax(up(a, dt), dim))
    assert_close(got, oo.softmax(a, dim, dt), dt, "softmax", scale=1.0 if dt != "bf16" else None)
    assert_close(got.astype(np.float64).sum(dim % a.ndim), np.ones(np.delete(shape, dim % a.ndim)), dt, "rows sum to 1",
                 scale=2.0)
    lg = down(R.log_softmax(up(a, dt), dim))
    assert_close(lg, oo.log_softmax(a, dim, dt), dt, "log_softmax")


def test_softmax_extremes(R):
    a = np.array([[1e4, 1e4 - 1, -1e4, 0], [-np.inf, 0, 0, -np.inf], [5, 5, 5, 5]], np.float32)
    got = down(R.softmax(up(a, "f32"), -1))
    assert_close(got, oo.softmax(a, -1, "f32"), "f32")
    assert np.allclose(got[2], 0.25) and got[1, 0] == 0 and np.allclose(got[1, 1:3], 0.5)


@pytest.mark.parametrize("dt", ["f32", "bf16", "f16", "f64", "u32", "i64", "u8"])
@pytest.mark.parametrize("shape,dim", [((8, 51200), -1), ((3, 5000), 1), ((6, 40, 50), 1), ((70, 9), 0), ((5, 1), 1)])
def test_argmax_argmin_bit_exact(R, dt, shape, dim):
    g = rng(18)
    if dt in FLOATS:
        # few distinct values -> many exact ties; first index must win
        a = rnd(np.round(g.standard_normal(shape) * 3).astype(np.float32), dt)
    else:
        a = g.integers(0, 7, shape).astype({"u32": np.uint32, "i64": np.int64, "u8": np.uint8}[dt])
    x = up(a, dt)
    for keep in (False, True):
        got = down(R.argmax(x, dim, keep))
        assert got.dtype == np.uint32 and np.array_equal(got, oo.argmax(a, dim, keep)), ("argmax", dt, shape, dim)
        assert np.array_equal(down(R.argmin(x, dim, keep)), oo.argmin(a, dim, keep)), ("argmin", dt, shape, dim)


def test_argmax_specials(R):
    n = 4096
    a = np.zeros((6, n), np.float32)
    a[0, 100] = np.nan; a[0, 200] = 1.0            # NaN in the middle never wins
    a[1, 0] = np.nan; a[1, 7] = 5.0                # NaN at element 0 wins
    a[2, :] = -np.inf; a[2, 3000] = -1e30          # finite beats -inf
    a[3, 10] = np.inf; a[3, 4000] = np.inf         # first +inf
    a[4, :] = -0.0; a[4, 77] = 0.0                 # -0.0 == 0.0: first index
    a[5, :] = np.nan                               # all NaN -> 0
    got = down(R.argmax(up(a, "f32"), -1))
    assert list(got) == [200, 0, 3000, 10, 0, 0]
    assert np.array_equal(got, oo.argmax(a, -1))


def test_argmax_strided_view(R):
    a = rand(rng(19), (50, 3000), "f32")
    x = up(a, "f32").transpose(0, 1)  # [3000, 50], argmax over dim 0 of the view
    assert np.array_equal(down(R.argmax(x, 0)), oo.argmax(a.T, 0))


# ------------------------------------------------------------------ index_select
@pytest.mark.parametrize("dt", ["u8", "u32", "i64", "f16", "bf16", "f32", "f64"])
@pytest.mark.parametrize("idt", ["u8", "u32", "i64"])
def test_index_select_bit_exact(R, dt, idt):
    g = rng(20)
    rows, cols = (200, 264)
    if dt in FLOATS:
        table = rand(g, (rows, cols), dt)
    else:
        table = g.integers(0, 255, (rows, cols)).astype({"u8": np.uint8, "u32": np.uint32, "i64": np.int64}[dt])
    ids = g.integers(0, rows, 77).astype({"u8": np.uint8, "u32": np.uint32, "i64": np.int64}[idt])
    t = up(table, dt)
    got = R.index_select(t, 0, up(ids, idt)).to_storage()
    assert np.array_equal(got, t.to_storage()[ids.astype(np.int64)])
    ids2 = g.integers(0, cols, 9).astype(ids.dtype)
    got = R.index_select(t, 1, up(ids2, idt)).to_storage()           # generic (non-row) path
    assert np.array_equal(got, t.to_storage()[:, ids2.astype(np.int64)])
    assert R.index_errors() == 0


def test_index_select_edge_cases(R):
    table = rand(rng(21), (10, 3, 5), "f32")     # odd inner size -> scalar path
    t = up(table, "f32")
    ids = np.array([9, 0, 9, 3], np.uint32)
    assert np.array_equal(down(R.index_select(t, 0, up(ids, "u32"))), table[ids])
    assert np.array_equal(down(R.index_select(t, 1, up(np.array([2, 2], np.uint32), "u32"))), table[:, [2, 2]])
    assert down(R.index_select(t, 0, up(np.zeros((0,), np.uint32), "u32"))).shape == (0, 3, 5)   # empty index
    # transposed (non-contiguous) table
    assert np.array_equal(down(R.index_select(t.transpose(0, 2), 0, up(np.array([4, 1], np.uint32), "u32"))),
                          np.swapaxes(table, 0, 2)[[4, 1]])
    assert R.index_errors() == 0
    # out-of-range index is reported, row zero-filled, never silently read
    bad = down(R.index_select(t, 0, up(np.array([1, 10], np.uint32), "u32")))
    assert np.array_equal(bad[0], table[1]) and np.all(bad[1] == 0)
    assert R.index_errors() == 1 and R.index_errors() == 0


# ------------------------------------------------------------------ matmul / linear
@pytest.mark.parametrize("dt", FLOATS)
def test_matmul_small_vs_f64_triple_loop(R, dt):
    g = rng(22)
    a, b = rand(g, (5, 7), dt), rand(g, (7, 3), dt)
    want = np.zeros((5, 3))
    for i in range(5):
        for j in range(3):
            for k in range(7):
                want[i, j] += float(a[i, k]) * float(b[k, j])
    assert_close(down(R.matmul(up(a, dt), up(b, dt))), rnd(want, dt), dt)
    eye = np.eye(7, dtype=np.float32)
    assert np.array_equal(np.asarray(down(R.matmul(up(a, dt), up(rnd(eye, dt), dt))), np.float64),
                          np.asarray(a, np.float64))


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("m,k,n", [(1, 256, 384), (3, 2560, 640), (8, 512, 100), (17, 64, 48), (64, 320, 256),
                                   (200, 2560, 384), (130, 72, 136)])
def test_linear_layout_matmul(R, dt, m, k, n):
    # x @ W.broadcast_left(b).t()  (rai-nn/src/linear.rs:59-69): rhs is a transposed stride-0 batch view
    g = rng(23)
    x, w = rand(g, (2, m, k), dt), rand(g, (n, k), dt)
    wt = up(w, dt).broadcast_to((2, n, k)).transpose(1, 2)
    got = down(R.matmul(up(x, dt), wt))
    want = oo.matmul(x, np.swapaxes(w, 0, 1), dt)
    assert_close(got, want, dt, f"linear-matmul {m}x{k}x{n}")


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_matmul_batched_strided(R, dt):
    # attention-shaped: q[B,H,S,D] @ k[B,H,T,D].t() and p[B,H,S,T] @ v[B,H,T,D], with transposed head views
    g = rng(24)
    q, k, v = rand(g, (2, 9, 4, 80), dt), rand(g, (2, 12, 4, 80), dt), rand(g, (2, 12, 4, 80), dt)
    qd, kd, vd = (up(t, dt).transpose(1, 2) for t in (q, k, v))          # [B,H,S,D] views of [B,S,H,D]
    s = R.matmul(qd, kd.transpose(2, 3))
    qt, kt, vt = (np.swapaxes(t, 1, 2) for t in (q, k, v))
    want = oo.matmul(qt, np.swapaxes(kt, 2, 3), dt)
    assert_close(down(s), want, dt, "QK^T")
    assert_close(down(R.matmul(s, vd)), oo.matmul(want, vt, dt), dt, "PV")
    # broadcast batch on the left operand
    a, b = rand(g, (1, 6, 10), dt), rand(g, (3, 10, 4), dt)
    assert_close(down(R.matmul(up(a, dt), up(b, dt))), oo.matmul(a, b, dt), dt, "batch broadcast")


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("m", [1, 4, 9, 16, 33, 48, 64, 130])
def test_fused_linear_bias_act_residual(R, dt, m):
    g = rng(25)
    k, n = 512, 384
    x, w, b, r = rand(g, (m, k), dt), rand(g, (n, k), dt, 0.05), rand(g, (n,), dt), rand(g, (m, n), dt)
    want = oo.add(onn.new_gelu(onn.linear(x, w, b, dt), dt), r, dt)
    got = down(R.linear(up(x, dt), up(w, dt), up(b, dt), "new_gelu", up(r, dt)))
    assert_close(got, want, dt, f"linear fused m={m}")
    assert_close(down(R.linear(up(x, dt), up(w, dt))), onn.linear(x, w, None, dt), dt, "linear plain")


@pytest.mark.parametrize("kernel", ["stream", "skinny", "tile"])
@pytest.mark.parametrize("m", [9, 16, 31, 64])
@pytest.mark.parametrize("k,n", [(4096, 200), (1056, 2048), (16384, 64), (96, 50), (2048, 16384)])
def test_linear_small_batch_deep_k(R, monkeypatch, m, k, n, kernel):
    # 9..64 rows: the weight-streaming MFMA kernel by default; its two fallbacks (activations in LDS with K split over
    # blocks, and the tile kernel) are forced through the switches the library reads at every call
    if kernel != "stream":
        monkeypatch.setenv("RAI_HIP_NO_MFMA_STREAM", "1")
    if kernel == "tile":
        monkeypatch.setenv("RAI_HIP_NO_MFMA_SKINNY", "1")
    # batched-decode shapes: 9..64 activation rows against a weight matrix read once; K deep enough
    # to be split over blocks and staged in several chunks, N not a multiple of the 16-row tile
    g = rng(125)
    x, w, b = rand(g, (m, k), "bf16"), rand(g, (n, k), "bf16", 0.03), rand(g, (n,), "bf16")
    r = rand(g, (m, n), "bf16")
    assert_close(down(R.linear(up(x, "bf16"), up(w, "bf16"), up(b, "bf16"))), onn.linear(x, w, b, "bf16"), "bf16",
                 f"linear {m}x{k}x{n}")
    want = oo.add(onn.new_gelu(onn.linear(x, w, b, "bf16"), "bf16"), r, "bf16")
    got = down(R.linear(up(x, "bf16"), up(w, "bf16"), up(b, "bf16"), "new_gelu", up(r, "bf16")))
    assert_close(got, want, "bf16", f"linear fused {m}x{k}x{n}")


@pytest.mark.parametrize("m,k,n", [(32, 16384, 2048), (9, 4096, 200), (64, 16384, 64), (17, 6144, 1000)])
def test_linear_k_split_summed_by_the_last_block(R, monkeypatch, m, k, n):
    """The weight-streaming kernel with K split over blocks: the block that finishes a group of weight tiles last sums
    the partial products itself.  Same bits as the separate summing pass (RAI_HIP_NO_FUSED_SPLITK=1), call after call
    (the tickets are handed back), with and without the fused epilogue."""
    g = rng(126)
    x, w, b = rand(g, (m, k), "bf16"), rand(g, (n, k), "bf16", 0.03), rand(g, (n,), "bf16")
    r = rand(g, (m, n), "bf16")
    xd, wd, bd, rd = (up(a, "bf16") for a in (x, w, b, r))

    def run():
        return down(R.linear(xd, wd, bd)), down(R.linear(xd, wd, bd, "new_gelu", rd))

    fused = [run() for _ in range(3)]
    monkeypatch.setenv("RAI_HIP_NO_FUSED_SPLITK", "1")
    plain = run()
    for it in fused:
        np.testing.assert_array_equal(it[0], plain[0])
        np.testing.assert_array_equal(it[1], plain[1])
    assert_close(plain[0], onn.linear(x, w, b, "bf16"), "bf16", f"linear {m}x{k}x{n}")


# ------------------------------------------------------------------ norms / rope / attention
@pytest.mark.parametrize("dt", ["f32", "bf16", "f16", "f64"])
@pytest.mark.parametrize("shape", [(3, 7, 2560), (5, 1536), (4, 100), (2, 9000), (6, 2048)])
def test_layer_norm_rms_norm(R, dt, shape):
    g = rng(26)
    x = rand(g, shape, dt, 1.5)
    w = rnd(1.0 + 0.1 * g.standard_normal(shape[-1]).astype(np.float32), dt)
    b = rand(g, shape[-1:], dt, 0.1)
    assert_close(down(R.layer_norm(up(x, dt), up(w, dt), up(b, dt), 1e-5)), onn.layer_norm(x, w, b, 1e-5, dt), dt, "ln")
    assert_close(down(R.layer_norm(up(x, dt), None, None, 1e-5)), onn.layer_norm(x, None, None, 1e-5, dt), dt, "ln-na")
    assert_close(down(R.rms_norm(up(x, dt), up(w, dt), 1e-6)), onn.rms_norm(x, w, 1e-6, dt), dt, "rms")
    w0 = rnd(w - 1.0, dt)
    assert_close(down(R.rms_norm(up(x, dt), up(w0, dt), 1e-6, True)), onn.gemma_rms_norm(x, w0, 1e-6, dt), dt, "rms1p")


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_rope_matches_phi2_reference_chain(R, dt):
    from oracle import phi2
    cfg = phi2.Config(max_position_embeddings=64)
    sin, cos = phi2.rotary_tables(cfg, dt)
    x = rand(rng(27), (2, 5, 7, 80), dt)
    for offset in (0, 13):
        want = phi2.rotary(x, sin, cos, cfg.rotary_dim, offset, dt)
        got = down(R.rope(up(x, dt), up(cos, dt), up(sin, dt), cfg.rotary_dim, offset))
        assert_close_elem(got, want, dt, f"rope offset {offset}", atol=1e-6 if dt == "f32" else 1e-3)
        # transposed [B,S,H,D] storage viewed as [B,H,S,D], as produced by reshape + transpose(1,2)
        xt = up(np.ascontiguousarray(np.swapaxes(x, 1, 2)), dt).transpose(1, 2)
        assert_close_elem(down(R.rope(xt, up(cos, dt), up(sin, dt), cfg.rotary_dim, offset)), want, dt, "rope strided",
                          atol=1e-6 if dt == "f32" else 1e-3)
    # device-built f32 tables agree with the f32 reference chain
    c32, s32 = R.rope_tables(64, 32, 10000.0, "f32")
    sin32, cos32 = phi2.rotary_tables(cfg, "f32")
    assert_close(down(c32), cos32, "f32", "cos table")
    assert_close(down(s32), sin32, "f32", "sin table")


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("hq,hkv,s,t,d,causal,f32s", [(4, 4, 16, 16, 80, 1, 1), (4, 4, 1, 37, 80, 0, 1),
                                                     (6, 2, 9, 20, 128, 1, 0), (8, 1, 1, 50, 256, 0, 0),
                                                     (4, 4, 200, 200, 80, 1, 1), (3, 3, 70, 333, 80, 1, 1),
                                                     (6, 2, 129, 129, 128, 1, 0), (4, 1, 65, 100, 256, 1, 0),
                                                     (2, 2, 100, 160, 64, 0, 1), (40, 40, 130, 130, 80, 1, 1)])
def test_attention(R, dt, hq, hkv, s, t, d, causal, f32s):
    import math
    g = rng(28)
    b = 2
    q, k, v = rand(g, (b, hq, s, d), dt), rand(g, (b, hkv, t, d), dt), rand(g, (b, hkv, t, d), dt)
    scale = 1.0 / math.sqrt(d)
    kr, vr = np.repeat(k, hq // hkv, 1), np.repeat(v, hq // hkv, 1)
    mask = (np.arange(t)[None, :] > (np.arange(s)[:, None] + (t - s))) if causal else np.zeros((s, t), bool)
    if f32s:   # rai-models/src/llm/phi2.rs:244-262
        w = oo.matmul(oo.to_dtype(q, dt, "f32"), oo.mul(np.swapaxes(oo.to_dtype(kr, dt, "f32"), -1, -2),
                                                       np.float32(scale), "f32"), "f32")
        w = np.where(mask, np.float32(-np.inf), w)
        p = oo.to_dtype(oo.softmax(w, -1, "f32"), "f32", dt)
    else:      # rai-models/src/llm/qwen2.rs:205-216
        w = oo.mul(oo.matmul(q, np.swapaxes(kr, -1, -2), dt), oo.full_like(np.zeros(()), scale, dt, "f64"), dt)
        w = oo.add(w, np.where(mask, np.float32(-np.inf), np.float32(0)), dt)
        p = oo.softmax(w, -1, dt)
    want = oo.matmul(p, vr, dt).transpose(0, 2, 1, 3).reshape(b, s, hq * d)
    got = down(R.attention(up(q, dt), up(k, dt), up(v, dt), scale, causal, f32s))
    assert_close(got, want, dt, "attention")


@pytest.mark.parametrize("hq,hkv,s,t,d,causal,f32s", [(4, 4, 512, 512, 80, 1, 1), (4, 2, 300, 320, 64, 1, 0),
                                                     (3, 3, 64, 257, 80, 0, 1), (2, 2, 129, 640, 80, 1, 1)])
def test_flash_prefill_key_split_against_single_chain(R, monkeypatch, hq, hkv, s, t, d, causal, f32s):
    """Short sequences with few heads run the flash kernel with two waves per query group, one for the even and one
    for the odd key tiles, merged at the end (odd tile counts, a last tile past the context and non-square causal
    shapes included).  Both forms are held to the oracle; against each other they differ by rounding only."""
    import math
    dt = "bf16"
    g = rng(29)
    q, k, v = rand(g, (1, hq, s, d), dt), rand(g, (1, hkv, t, d), dt), rand(g, (1, hkv, t, d), dt)
    scale = 1.0 / math.sqrt(d)
    kr, vr = np.repeat(k, hq // hkv, 1), np.repeat(v, hq // hkv, 1)
    mask = (np.arange(t)[None, :] > (np.arange(s)[:, None] + (t - s))) if causal else np.zeros((s, t), bool)
    if f32s:
        w = oo.matmul(oo.to_dtype(q, dt, "f32"), oo.mul(np.swapaxes(oo.to_dtype(kr, dt, "f32"), -1, -2),
                                                       np.float32(scale), "f32"), "f32")
        p = oo.to_dtype(oo.softmax(np.where(mask, np.float32(-np.inf), w), -1, "f32"), "f32", dt)
    else:
        w = oo.mul(oo.matmul(q, np.swapaxes(kr, -1, -2), dt), oo.full_like(np.zeros(()), scale, dt, "f64"), dt)
        p = oo.softmax(oo.add(w, np.where(mask, np.float32(-np.inf), np.float32(0)), dt), -1, dt)
    want = oo.matmul(p, vr, dt).transpose(0, 2, 1, 3).reshape(1, s, hq * d)
    got = {}
    for off in ("0", "1"):
        monkeypatch.setenv("RAI_HIP_FLASH_NO_KEY_SPLIT", off)     # read per call
        got[off] = down(R.attention(up(q, dt), up(k, dt), up(v, dt), scale, causal, f32s))
        assert_close(got[off], want, dt, f"attention, key split {'off' if off == '1' else 'on'}")
    assert_close(got["0"], got["1"], dt, "key split against single chain")


# ------------------------------------------------------------------ error behaviour
def test_errors_are_reported_not_silent(R):
    from rai_amd._lib import RaiHipError
    a = up(np.zeros((2, 3), np.float32), "f32")
    with pytest.raises(RaiHipError):
        R.matmul(a, up(np.zeros((4, 2), np.float32), "f32"))       # inner dims differ
    with pytest.raises(RaiHipError):
        R.binary("add", a, up(np.zeros((2, 3), np.uint16), "bf16"))  # dtype mismatch
    with pytest.raises(RaiHipError):
        R.unary("exp", up(np.zeros((2,), np.uint32), "u32"))       # float op on ints
    with pytest.raises(RaiHipError):
        R.index_select(a, 0, up(np.zeros((2,), np.float32), "f32"))  # float index
