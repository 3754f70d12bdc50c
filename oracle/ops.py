"""Primitive operators of rai evaluated on its Cpu device, restated in NumPy.

Test infrastructure only (see oracle/__init__.py).  Every function takes carrier
arrays (see oracle/dtypes.py) and the storage dtype name `dt`; the result is
rounded to `dt` exactly once per primitive, the way each candle op rounds its
output when rai dispatches one primitive at a time
(rai-core/src/eval.rs:31-51 -> rai-core/src/backend/candle.rs).
"""
import math

import numpy as np
from scipy import special as _sp

from .dtypes import FLOAT_DTYPES, carrier, rnd


# ----------------------------------------------------------------- creation
def full(val, shape, dt):
    """Full<T>: backend/candle.rs:197-209, ops/full.rs:63-72."""
    return rnd(np.full(shape, val, dtype=carrier(dt)), dt)


def full_like(x, val, dt, val_dt="f32"):
    """full_like: ops/full.rs:85-92 — Full<T> in the scalar's own dtype, then
    ToDType to x's dtype when they differ (so a f32 constant is rounded to bf16)."""
    c = full(val, np.shape(x), val_dt)
    return c if val_dt == dt else to_dtype(c, val_dt, dt)


def arange(start, stop, step, dt):
    """Arange<T>: backend/candle.rs:241-256, ops/arange.rs:102-117."""
    n = max(0, int(math.ceil((stop - start) / step)))
    return rnd(start + step * np.arange(n, dtype=np.float64), dt) if dt in FLOAT_DTYPES else (
        (start + step * np.arange(n)).astype(carrier(dt)))


def to_dtype(x, src_dt, dst_dt):
    """ToDType<T>: backend/candle.rs:762-774.  Float -> int truncates toward zero
    and saturates (Rust `as`); float -> narrower float rounds to nearest even."""
    if src_dt == dst_dt:
        return x
    if dst_dt in FLOAT_DTYPES:
        return rnd(np.asarray(x).astype(np.float64 if dst_dt == "f64" else np.float32), dst_dt)
    info = np.iinfo(carrier(dst_dt))
    if src_dt in FLOAT_DTYPES:
        xf = np.asarray(x, dtype=np.float64)
        t = np.trunc(np.nan_to_num(xf, nan=0.0, posinf=float(info.max), neginf=float(info.min)))
        t = np.clip(t, float(info.min), float(info.max))
        # float(int64 max) rounds up to 2**63; clip in integer space afterwards
        out = np.where(t >= float(info.max), info.max, np.where(t <= float(info.min), info.min, 0)).astype(carrier(dst_dt))
        mid = (t > float(info.min)) & (t < float(info.max))
        out[mid] = t[mid].astype(carrier(dst_dt))
        return out
    return np.asarray(x).astype(carrier(dst_dt))  # int -> int wraps like Rust `as`


# ----------------------------------------------------------------- elementwise
def _bin(f):
    def op(a, b, dt):
        a, b = np.broadcast_arrays(np.asarray(a, dtype=carrier(dt)), np.asarray(b, dtype=carrier(dt)))
        with np.errstate(all="ignore"):
            return rnd(f(a, b), dt)
    return op


# Broadcast binary ops: ops/mod.rs:298-340 (broadcast per shape.rs:88-127),
# evaluated at backend/candle.rs:275-325, 736-760.
add = _bin(np.add)
sub = _bin(np.subtract)
mul = _bin(np.multiply)
maximum = _bin(np.maximum)
minimum = _bin(np.minimum)


def div(a, b, dt):
    a, b = np.broadcast_arrays(np.asarray(a, dtype=carrier(dt)), np.asarray(b, dtype=carrier(dt)))
    if dt in FLOAT_DTYPES:
        with np.errstate(all="ignore"):
            return rnd(a / b, dt)
    return np.where(b != 0, a // np.where(b == 0, 1, b), 0).astype(carrier(dt))


def _cmp(f):
    def op(a, b, dt):
        a, b = np.broadcast_arrays(np.asarray(a, dtype=carrier(dt)), np.asarray(b, dtype=carrier(dt)))
        return f(a, b).astype(np.uint8)  # candle comparisons yield U8, candle.rs:658-734
    return op


eq = _cmp(np.equal)
ne = _cmp(np.not_equal)
gt = _cmp(np.greater)
ge = _cmp(np.greater_equal)
lt = _cmp(np.less)
le = _cmp(np.less_equal)


def _un(f):
    def op(x, dt):
        with np.errstate(all="ignore"):
            return rnd(f(np.asarray(x, dtype=carrier(dt))), dt)
    return op


# Unary primitives: backend/candle.rs:445-473, 525-553, 608-656, 947-978.
sin = _un(np.sin)
cos = _un(np.cos)
neg = _un(np.negative)
square = _un(np.square)
sqrt = _un(np.sqrt)
abs_ = _un(np.abs)
exp = _un(np.exp)
log = _un(np.log)
tanh = _un(np.tanh)
erf = _un(_sp.erf)


def rsqrt(x, dt):
    """Rsqrt = sqrt then recip, two candle ops, each rounding: candle.rs:545-553."""
    s = sqrt(x, dt)
    with np.errstate(all="ignore"):
        return rnd(np.asarray(1.0, dtype=carrier(dt)) / s, dt)


def log2(x, dt):
    """candle.rs:628-636: log(x) then divide by ln 2 (an affine op in f64)."""
    with np.errstate(all="ignore"):
        return rnd(log(x, dt).astype(np.float64) / math.log(2.0), dt)


def log10(x, dt):
    with np.errstate(all="ignore"):
        return rnd(log(x, dt).astype(np.float64) / math.log(10.0), dt)


def sign(x, dt):
    """candle.rs:595-606: (x >= 0) - (x <= 0)."""
    x = np.asarray(x, dtype=carrier(dt))
    return rnd((x >= 0).astype(carrier(dt)) - (x <= 0).astype(carrier(dt)), dt)


def powf(x, e, dt):
    """Powf<T>: candle.rs:966-978 (f64 exponent applied in the element type)."""
    with np.errstate(all="ignore"):
        return rnd(np.power(np.asarray(x, dtype=carrier(dt)), carrier(dt)(e)), dt)


def where(cond, on_true, on_false, dt):
    """Where: candle.rs:901-915 (inputs ordered on_true, on_false, cond)."""
    c, t, f = np.broadcast_arrays(np.asarray(cond), on_true, on_false)
    return rnd(np.where(c != 0, t, f), dt)


# ----------------------------------------------------------------- reductions
def _dims(x, dims):
    if dims is None:
        return tuple(range(np.ndim(x)))
    if isinstance(dims, int):
        dims = (dims,)
    return tuple(d % np.ndim(x) for d in dims)


def reduce_sum(x, dims, keep_dim, dt):
    """ReduceSum: candle.rs:475-488.  Accumulates in the carrier type (f32 for
    bf16/f16: the accumulator width of candle's CPU sum is unpinned)."""
    x = np.asarray(x, dtype=carrier(dt))
    return rnd(np.sum(x, axis=_dims(x, dims), keepdims=bool(keep_dim), dtype=carrier(dt)), dt)


def reduce_max(x, dims, keep_dim, dt):
    """ReduceMax: candle.rs:490-506 (single dim in the reference)."""
    x = np.asarray(x, dtype=carrier(dt))
    return rnd(np.max(x, axis=_dims(x, dims), keepdims=bool(keep_dim)), dt)


def reduce_min(x, dims, keep_dim, dt):
    x = np.asarray(x, dtype=carrier(dt))
    return rnd(np.min(x, axis=_dims(x, dims), keepdims=bool(keep_dim)), dt)


def softmax(x, dim, dt):
    """Softmax: candle.rs:793-803 — max_keepdim, broadcast_sub, exp, sum_keepdim,
    broadcast_div: five candle ops, each rounding to the tensor dtype."""
    m = reduce_max(x, dim, True, dt)
    d = sub(x, m, dt)
    num = exp(d, dt)
    den = reduce_sum(num, dim, True, dt)
    return div(num, den, dt)


def log_softmax(x, dim, dt):
    """LogSoftmax: candle.rs:805-816."""
    m = reduce_max(x, dim, True, dt)
    d = sub(x, m, dt)
    s = reduce_sum(exp(d, dt), dim, True, dt)
    return sub(d, log(s, dt), dt)


def argmax(x, dim, keep_dim=False):
    """ArgMax: candle.rs:917-930, ops/argmax.rs:48-61.  U32 result; a sequential
    scan from element 0 that replaces the running best only on a strict `>`:
    the first maximum wins, NaN wins only from position 0."""
    x = np.asarray(x)
    d = dim % x.ndim
    xm = np.moveaxis(x, d, -1)
    if np.issubdtype(xm.dtype, np.floating):
        first_nan = np.isnan(xm[..., 0])
        safe = np.where(np.isnan(xm), -np.inf, xm)
        idx = np.argmax(safe, axis=-1)
        # a row of only -inf/NaN after element 0: argmax of all -inf is 0 already
        idx = np.where(first_nan, 0, idx)
    else:
        idx = np.argmax(xm, axis=-1)
    idx = idx.astype(np.uint32)
    return np.expand_dims(idx, d) if keep_dim else idx


def argmin(x, dim, keep_dim=False):
    """ArgMin as documented by ops/argmin.rs (the reference's candle.rs:932-944
    calls argmax here, an upstream slip that is not reproduced)."""
    x = np.asarray(x)
    d = dim % x.ndim
    xm = np.moveaxis(x, d, -1)
    if np.issubdtype(xm.dtype, np.floating):
        first_nan = np.isnan(xm[..., 0])
        safe = np.where(np.isnan(xm), np.inf, xm)
        idx = np.where(first_nan, 0, np.argmin(safe, axis=-1))
    else:
        idx = np.argmin(xm, axis=-1)
    idx = idx.astype(np.uint32)
    return np.expand_dims(idx, d) if keep_dim else idx


# ----------------------------------------------------------------- indexing / shape
def index_select(x, dim, index):
    """IndexSelect: candle.rs:867-878, ops/index_select.rs:52-61."""
    index = np.asarray(index).reshape(-1).astype(np.int64)
    if index.size and (index.min() < 0 or index.max() >= np.shape(x)[dim]):
        raise IndexError("index_select: index out of range")
    return np.take(x, index, axis=dim)


def gather(x, dim, index):
    """Gather: candle.rs:838-849, ops/gather.rs:47-60: out[.., j, ..] = x[.., index[.., j, ..], ..]; out has
    index's shape.  Known answer rai-core/tests/ops.rs:156-161."""
    x = np.asarray(x)
    index = np.asarray(index).astype(np.int64)
    d = dim % x.ndim
    if x.ndim != index.ndim or any(i != d and x.shape[i] != index.shape[i] for i in range(x.ndim)):
        raise ValueError("gather: shape mismatch")
    if index.size and (index.min() < 0 or index.max() >= x.shape[d]):
        raise IndexError("gather: index out of range")
    return np.take_along_axis(x, index, axis=d)


def _add_in_dtype(a, b, dt):
    if dt in ("bf16", "f16", "f32", "f64"):
        return rnd(a + b, dt)
    with np.errstate(over="ignore"):      # integer dtypes wrap
        return (np.asarray(a) + np.asarray(b)).astype(np.asarray(a).dtype)


def index_add(x, dim, index, source, dt):
    """IndexAdd: candle.rs:851-865, ops/index_add.rs:52-62: out = x; out[.., index[l], ..] += source[.., l, ..]
    for l in order, every sum rounded to the storage dtype ([candle, unverified]: its Cpu loop adds in place
    in the element type, source row by source row)."""
    out = np.array(x, copy=True)
    index = np.asarray(index).reshape(-1).astype(np.int64)
    d = dim % out.ndim
    source = np.asarray(source)
    want = list(out.shape)
    want[d] = index.size
    if list(source.shape) != want:
        raise ValueError("index_add: shape mismatch")
    if index.size and (index.min() < 0 or index.max() >= out.shape[d]):
        raise IndexError("index_add: index out of range")
    o = np.moveaxis(out, d, 0)          # views: writes land in `out`
    s = np.moveaxis(source, d, 0)
    for l, r in enumerate(index):
        o[r] = _add_in_dtype(o[r], s[l], dt)
    return out


def scatter_add(x, dim, index, source, dt):
    """ScatterAdd: candle.rs:990-1004, ops/scatter_add.rs:52-60: out = x;
    out[.., index[.., j, ..], ..] += source[.., j, ..] for j in order, every sum rounded to the storage dtype."""
    out = np.array(x, copy=True)
    index = np.asarray(index).astype(np.int64)
    source = np.asarray(source)
    d = dim % out.ndim
    if index.shape != source.shape or index.ndim != out.ndim or any(
            i != d and out.shape[i] != index.shape[i] for i in range(out.ndim)):
        raise ValueError("scatter_add: shape mismatch")
    if index.size and (index.min() < 0 or index.max() >= out.shape[d]):
        raise IndexError("scatter_add: index out of range")
    o = np.moveaxis(out, d, -1)         # [..., D] view
    ix = np.moveaxis(index, d, -1)
    sr = np.moveaxis(source, d, -1)
    lead = np.indices(ix.shape[:-1]) if ix.ndim > 1 else ()
    for j in range(ix.shape[-1]):
        sel = tuple(lead) + (ix[..., j],)
        o[sel] = _add_in_dtype(o[sel], sr[..., j], dt)
    return out


def narrow(x, dim, start, length):
    """Narrow: candle.rs:891-899."""
    sl = [slice(None)] * np.ndim(x)
    sl[dim % np.ndim(x)] = slice(start, start + length)
    return x[tuple(sl)]


def concatenate(xs, dim):
    """Concatenate: candle.rs:880-889, ops/concatenate.rs:54-67."""
    return np.concatenate(xs, axis=dim)


def chunk(x, n, dim):
    """hlops/chunk.rs: equal pieces of ceil(size/n) along dim."""
    d = dim % np.ndim(x)
    size = np.shape(x)[d]
    step = -(-size // n)
    return [narrow(x, d, s, min(step, size - s)) for s in range(0, size, step)]


def matmul(a, b, dt):
    """MatMul: candle.rs:327-443, ops/matmul.rs:34-70, batch broadcast
    shape.rs:130-160; rank-1 operands are promoted like ops/matmul.rs:38-52.
    f32 accumulation, one rounding of the result."""
    a = np.asarray(a, dtype=carrier(dt))
    b = np.asarray(b, dtype=carrier(dt))
    return rnd(np.matmul(a, b), dt)
