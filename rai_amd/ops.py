"""One function per rai primitive, each doing what `impl Eval<Hip, ops::X>` would:
read the evaluated inputs, allocate a fresh output of the node's inferred shape
and dtype, launch the HIP kernel through the C ABI
(reference: one `impl Eval<D, ops::X> for CandleBackend` per primitive in
rai-core/src/backend/candle.rs:197-1190).  Shapes/dtypes follow the op
definitions under rai-core/src/ops/.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from ._lib import BINARY, DTYPE_BY_NAME, REDUCE, U8, U32, UNARY, call
from .hip import HipTensor


def _d(t):
    return C.byref(t.desc()) if t is not None else None


def _dt(dtype):
    return DTYPE_BY_NAME[dtype] if isinstance(dtype, str) else int(dtype)


# ---------------------------------------------------------------- creation
def full(value, shape, dtype, dev=0):
    out = HipTensor.empty(shape, dtype, dev)
    call("rai_hip_fill", dev, _d(out), float(value))
    return out


def arange(start, stop, step, dtype, dev=0):
    n = max(0, int(np.ceil((stop - start) / step)))
    out = HipTensor.empty((n,), dtype, dev)
    call("rai_hip_arange", dev, _d(out), float(start), float(step))
    return out


def from_array(arr, dtype, dev=0):
    """FromArray<T>: backend/candle.rs:258-273 (host -> device upload)."""
    return HipTensor.from_storage(arr, dtype, dev)


def to_device(x, dev):
    """ToDevice<Hip> (backend/candle.rs:776-790): a contiguous copy of x on HIP device `dev`."""
    out = HipTensor.empty(x.shape, x.dtype, dev)
    call("rai_hip_to_device", x.dev, _d(x), int(dev), _d(out))
    return out


def to_dtype(x, dtype):
    dt = _dt(dtype)
    if dt == x.dtype:
        return x
    out = HipTensor.empty(x.shape, dt, x.dev)
    call("rai_hip_cast", x.dev, _d(x), _d(out))
    return out


# ---------------------------------------------------------------- elementwise
def unary(name, x, param=0.0):
    out = HipTensor.empty(x.shape, x.dtype, x.dev)
    call("rai_hip_unary", x.dev, UNARY[name], _d(x), _d(out), float(param))
    return out


def broadcast_shapes(a, b):
    """rai-core/src/shape.rs:88-127."""
    ra, rb = len(a), len(b)
    a = (1,) * (max(ra, rb) - ra) + tuple(a)
    b = (1,) * (max(ra, rb) - rb) + tuple(b)
    out = []
    for l, r in zip(a, b):
        if l == r or r == 1:
            out.append(l)
        elif l == 1:
            out.append(r)
        else:
            raise ValueError(f"incompatible shapes {a} {b}")
    return tuple(out)


def binary(name, a, b):
    shape = broadcast_shapes(a.shape, b.shape)
    op = BINARY[name]
    out = HipTensor.empty(shape, U8 if op >= BINARY["eq"] else a.dtype, a.dev)
    call("rai_hip_binary", a.dev, op, _d(a.broadcast_to(shape)), _d(b.broadcast_to(shape)), _d(out))
    return out


def where(cond, on_true, on_false):
    shape = broadcast_shapes(broadcast_shapes(cond.shape, on_true.shape), on_false.shape)
    out = HipTensor.empty(shape, on_true.dtype, cond.dev)
    call("rai_hip_where", cond.dev, _d(cond.broadcast_to(shape)), _d(on_true.broadcast_to(shape)),
         _d(on_false.broadcast_to(shape)), _d(out))
    return out


# ---------------------------------------------------------------- reductions
def _reduced_shape(shape, dims, keep):
    return tuple(1 if i in dims else s for i, s in enumerate(shape) if keep or i not in dims)


def reduce(name, x, dims=None, keep_dim=False):
    dims = tuple(range(x.rank)) if dims is None else ((dims,) if isinstance(dims, int) else tuple(dims))
    dims = tuple(d % x.rank for d in dims)
    out = HipTensor.empty(_reduced_shape(x.shape, dims, keep_dim), x.dtype, x.dev)
    arr = (C.c_int32 * len(dims))(*dims)
    call("rai_hip_reduce", x.dev, REDUCE[name], _d(x), arr, len(dims), int(keep_dim), _d(out))
    return out


def softmax(x, dim):
    out = HipTensor.empty(x.shape, x.dtype, x.dev)
    call("rai_hip_softmax", x.dev, _d(x), int(dim), _d(out))
    return out


def log_softmax(x, dim):
    out = HipTensor.empty(x.shape, x.dtype, x.dev)
    call("rai_hip_log_softmax", x.dev, _d(x), int(dim), _d(out))
    return out


def argmax(x, dim, keep_dim=False, _fn="rai_hip_argmax"):
    d = dim % x.rank
    out = HipTensor.empty(_reduced_shape(x.shape, (d,), keep_dim), U32, x.dev)
    call(_fn, x.dev, _d(x), d, int(keep_dim), _d(out))
    return out


def sample_argmax(logits, context=None, repeat_penalty=1.10):
    """apply_repeat_penalty + sample_argmax of examples/phi2/src/main.rs:29-50: logits [rows, vocab],
    context [rows, n] u32 or None -> tokens [rows] u32."""
    out = HipTensor.empty((logits.shape[0],), U32, logits.dev)
    call("rai_hip_sample_argmax", logits.dev, _d(logits), None if context is None else _d(context),
         float(repeat_penalty), _d(out))
    return out


def argmin(x, dim, keep_dim=False):
    return argmax(x, dim, keep_dim, "rai_hip_argmin")


def argmax_static(x, dim, out, keep_dim=False):
    """rai_hip_argmax_static: argmax into the caller's `out`, with no allocation inside the library."""
    call("rai_hip_argmax_static", x.dev, _d(x), dim % x.rank, int(keep_dim), _d(out))
    return out


# ---------------------------------------------------------------- indexing
def index_select(x, dim, index):
    d = dim % x.rank
    shape = list(x.shape)
    shape[d] = index.numel()
    out = HipTensor.empty(shape, x.dtype, x.dev)
    call("rai_hip_index_select", x.dev, _d(x), _d(index), d, _d(out))
    return out


def gather(x, dim, index):
    """Tensor::gather (ops/gather.rs:47-60): out has index's shape."""
    d = dim % x.rank
    out = HipTensor.empty(index.shape, x.dtype, x.dev)
    call("rai_hip_gather", x.dev, _d(x), _d(index), d, _d(out))
    return out


def index_add(x, dim, index, source):
    """Tensor::index_add (ops/index_add.rs:52-62)."""
    d = dim % x.rank
    out = HipTensor.empty(x.shape, x.dtype, x.dev)
    call("rai_hip_index_add", x.dev, _d(x), _d(index), _d(source), d, _d(out))
    return out


def scatter_add(x, dim, index, source):
    """Tensor::scatter_add (ops/scatter_add.rs:52-60)."""
    d = dim % x.rank
    out = HipTensor.empty(x.shape, x.dtype, x.dev)
    call("rai_hip_scatter_add", x.dev, _d(x), _d(index), _d(source), d, _d(out))
    return out


def index_errors(dev=0):
    n = C.c_uint64(0)
    call("rai_hip_index_errors", dev, C.byref(n))
    return n.value


def concatenate(xs, dim):
    """Concatenate: one strided copy per piece into a narrowed view of the output."""
    d = dim % xs[0].rank
    shape = list(xs[0].shape)
    shape[d] = sum(x.shape[d] for x in xs)
    out = HipTensor.empty(shape, xs[0].dtype, xs[0].dev)
    at = 0
    for x in xs:
        call("rai_hip_copy", x.dev, _d(x), _d(out.narrow(d, at, x.shape[d])))
        at += x.shape[d]
    return out


# ---------------------------------------------------------------- contraction
def matmul(a, b):
    """ops/matmul.rs:34-70 with batch broadcast shape.rs:130-160."""
    if a.rank == 1:
        return matmul(a.reshape((1,) + a.shape), b).reshape(b.shape[:-2] + b.shape[-1:])
    if b.rank == 1:
        return matmul(a, b.reshape(b.shape + (1,))).reshape(a.shape[:-1])
    batch = broadcast_shapes(a.shape[:-2], b.shape[:-2])
    out = HipTensor.empty(batch + (a.shape[-2], b.shape[-1]), a.dtype, a.dev)
    call("rai_hip_matmul", a.dev, _d(a.broadcast_to(batch + a.shape[-2:])), _d(b.broadcast_to(batch + b.shape[-2:])),
         _d(out))
    return out


# ---------------------------------------------------------------- fused compositions
def linear(x, w, bias=None, act=None, residual=None):
    out = HipTensor.empty(x.shape[:-1] + (w.shape[0],), x.dtype, x.dev)
    call("rai_hip_linear", x.dev, _d(x), _d(w), _d(bias), -1 if act is None else UNARY[act], _d(residual), _d(out))
    return out


def linear_packed(x, w, bias=None, bias2=None, act=None, act_from=0, residual=None, glu=False, n1=None, k_splits=0):
    """rai_hip_linear_packed: several Linears over one input as one contraction.  Returns out1, or
    (out1, out2) when n1 < N splits the columns over two outputs."""
    m, n = x.shape[0], w.shape[0]
    n1 = n // 2 if glu else (n if n1 is None else n1)
    out1 = HipTensor.empty((m, n1), x.dtype, x.dev)
    out2 = None if glu or n1 == n else HipTensor.empty((m, n - n1), x.dtype, x.dev)
    call("rai_hip_linear_packed", x.dev, _d(x), _d(w), _d(bias), _d(bias2), -1 if act is None else UNARY[act],
         int(act_from), _d(residual), int(glu), int(k_splits), _d(out1), _d(out2))
    return out1 if out2 is None else (out1, out2)


def layer_norm(x, w, b, eps):
    out = HipTensor.empty(x.shape, x.dtype, x.dev)
    call("rai_hip_layer_norm", x.dev, _d(x), _d(w), _d(b), float(eps), _d(out))
    return out


def rms_norm(x, w, eps, add_one=False):
    out = HipTensor.empty(x.shape, x.dtype, x.dev)
    call("rai_hip_rms_norm", x.dev, _d(x), _d(w), float(eps), int(add_one), _d(out))
    return out


def rope_tables(max_pos, rot_dim, theta, dtype, f64_powf=False, dev=0):
    cos = HipTensor.empty((max_pos, rot_dim), dtype, dev)
    sin = HipTensor.empty((max_pos, rot_dim), dtype, dev)
    call("rai_hip_rope_tables", dev, float(theta), int(rot_dim), int(f64_powf), _d(cos), _d(sin))
    return cos, sin


def rope(x, cos, sin, rot_dim, offset):
    out = HipTensor.empty(x.shape, x.dtype, x.dev)
    call("rai_hip_rope", x.dev, _d(x), _d(cos), _d(sin), int(rot_dim), int(offset), _d(out))
    return out


def attention(q, k, v, scale, causal, f32_scores):
    b, hq, s, d = q.shape
    out = HipTensor.empty((b, s, hq * d), q.dtype, q.dev)
    call("rai_hip_attention", q.dev, _d(q), _d(k), _d(v), float(scale), int(causal), int(f32_scores), _d(out))
    return out
