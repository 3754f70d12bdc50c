"""Lazy tensors on the `Hip` device: the host-side mirror of rai-core's `Tensor`.

Building an expression only records nodes (rai-core/src/ops/*.rs); arithmetic
happens when `eval()` / `as_vec()` walks the graph in topological order and
dispatches each node to its rule (rai-core/src/eval.rs:31-51), here through
the C ABI of include/rai_graph.h.  Scalars on the right or left of an operator
become `full_like` constants followed by a dtype cast, as impl_std_ops! does
(rai-core/src/ops/mod.rs:203-296, full.rs:85-92).  The high-level ops below
are the reference's decompositions, node for node:
  mean / var            rai-core/src/hlops/mean.rs:4-7, var.rs:33-38 (ddof 0)
  new_gelu, gelu, silu  rai-core/src/hlops/activations.rs:5-32
  layer_norm, rms_norm  rai-nn/src/layer_norm.rs:32-42, rms_norm.rs:18-22
  linear                rai-nn/src/linear.rs:59-69
"""
from __future__ import annotations

import ctypes as C
import math

import numpy as np

from . import _lib
from ._lib import BF16, BINARY, DTYPE_BY_NAME, DTYPE_NAMES, DTYPE_SIZE, F16, F32, F64, I64, REDUCE, U8, U32, UNARY, \
    GraphStats, RaiHipError, TensorDesc, check

OP_KINDS = ["Full", "Arange", "FromArray", "ToDType", "Unary", "Binary", "MatMul", "Softmax", "LogSoftmax", "Reduce",
            "ArgMax", "ArgMin", "IndexSelect", "Narrow", "Concatenate", "Where", "Transpose", "Reshape", "Permute",
            "Broadcast", "ToContiguous", "Err", "Gather", "IndexAdd", "ScatterAdd", "ToDevice"]
OP = {n: i for i, n in enumerate(OP_KINDS)}
_NP = {U8: np.uint8, U32: np.uint32, I64: np.int64, F16: np.float16, BF16: np.uint16, F32: np.float32, F64: np.float64}


def _dt(d):
    return DTYPE_BY_NAME[d] if isinstance(d, str) else int(d)


def _shape_arr(shape):
    return (C.c_int64 * max(len(shape), 1))(*shape), len(shape)


class F64Scalar:
    """An f64 scalar operand (`x * 0.5f64` in the reference): becomes Full<f64> + ToDType, not Full<f32>."""

    def __init__(self, value):
        self.value = float(value)


class Tensor:
    """Handle of one graph node (a new reference; released with the Python object)."""

    def __init__(self, handle):
        if not handle:
            raise RaiHipError(-6, "null tensor handle")
        self._h = C.c_void_p(handle)

    def __del__(self):
        try:
            if getattr(self, "_h", None):
                _lib.load().rai_tensor_release(self._h)
                self._h = None
        except Exception:
            pass

    # ------------------------------------------------------------ creation
    @staticmethod
    def full(value, shape, dtype="f32", dev=0):
        arr, rank = _shape_arr(shape)
        return Tensor(_lib.load().rai_full(float(value), _dt(dtype), arr, rank, dev))

    @staticmethod
    def ones(shape, dtype="f32", dev=0):
        return Tensor.full(1.0, shape, dtype, dev)

    @staticmethod
    def zeros(shape, dtype="f32", dev=0):
        return Tensor.full(0.0, shape, dtype, dev)

    @staticmethod
    def arange(start, stop, step=1.0, dtype="f32", dev=0):
        return Tensor(_lib.load().rai_arange(float(start), float(stop), float(step), _dt(dtype), dev))

    @staticmethod
    def from_array(storage, dtype, dev=0):
        """`storage`: host array in the dtype's storage form (bf16 = uint16 bit patterns)."""
        dt = _dt(dtype)
        a = np.ascontiguousarray(storage, dtype=_NP[dt])
        arr, rank = _shape_arr(a.shape)
        return Tensor(_lib.load().rai_from_array(a.ctypes.data_as(C.c_void_p), dt, arr, rank, dev))

    @staticmethod
    def from_storage(desc, buf, dev=0):
        """An already evaluated node over existing device storage: `desc` a TensorDesc view into `buf`, an allocation
        of rai_hip_alloc (what a front end with tensor objects of its own hands over; the node retains `buf`)."""
        return Tensor(_lib.load().rai_from_storage(C.byref(desc), buf, dev))

    def buffer(self):
        """The allocation an evaluated node's view points into (None before evaluation)."""
        return _lib.load().rai_tensor_buffer(self._h)

    # ------------------------------------------------------------ metadata
    @property
    def shape(self):
        out = (C.c_int64 * 8)()
        r = _lib.load().rai_tensor_shape(self._h, out)
        return tuple(out[i] for i in range(r))

    @property
    def dtype(self):
        return DTYPE_NAMES[_lib.load().rai_tensor_dtype(self._h)]

    @property
    def device(self):
        return int(_lib.load().rai_tensor_device(self._h))

    @property
    def op(self):
        return OP_KINDS[_lib.load().rai_tensor_op(self._h)]

    @property
    def id(self):
        return int(_lib.load().rai_tensor_id(self._h))

    @property
    def error(self):
        e = _lib.load().rai_tensor_error(self._h)
        return e.decode() if e else None

    def is_evaluated(self):
        return bool(_lib.load().rai_tensor_is_evaluated(self._h))

    def num_inputs(self):
        return int(_lib.load().rai_tensor_num_inputs(self._h))

    def elem_count(self):
        return int(np.prod(self.shape, dtype=np.int64)) if self.shape else 1

    def storage(self):
        d = TensorDesc()
        check(_lib.load().rai_tensor_storage(self._h, C.byref(d)))
        return d

    # ------------------------------------------------------------ evaluation
    def eval(self, retain_graph=False):
        eval_all([self], retain_graph)
        return self

    def as_storage(self):
        """Tensor::as_vec in storage form (evaluates if needed)."""
        dt = _dt(self.dtype)
        out = np.empty(self.shape, _NP[dt])
        check(_lib.load().rai_tensor_to_host(self._h, out.ctypes.data_as(C.c_void_p), out.nbytes))
        return out

    def as_numpy(self):
        """Values as float64 / integer NumPy array."""
        s = self.as_storage()
        if self.dtype == "bf16":
            return (s.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        return s.astype(np.float64) if self.dtype in ("f16", "f32", "f64") else s

    # ------------------------------------------------------------ primitives
    def to_dtype(self, dtype):
        return Tensor(_lib.load().rai_to_dtype(self._h, _dt(dtype)))

    def _unary(self, name, param=0.0):
        return Tensor(_lib.load().rai_unary(UNARY[name], self._h, float(param)))

    def sin(self): return self._unary("sin")
    def cos(self): return self._unary("cos")
    def neg(self): return self._unary("neg")
    def square(self): return self._unary("square")
    def sqrt(self): return self._unary("sqrt")
    def rsqrt(self): return self._unary("rsqrt")
    def abs(self): return self._unary("abs")
    def exp(self): return self._unary("exp")
    def log(self): return self._unary("log")
    def erf(self): return self._unary("erf")
    def tanh(self): return self._unary("tanh")
    def powf(self, e): return self._unary("powf", e)
    def __neg__(self): return self.neg()

    def full_like(self, value, scalar_dtype="f32"):
        """Full<T> of this shape for a scalar of Rust type T (f32 or f64), cast to this dtype when it differs
        (full.rs:85-92)."""
        c = Tensor.full(value, self.shape, scalar_dtype)
        return c if self.dtype == scalar_dtype else c.to_dtype(self.dtype)

    def _binary(self, name, other, swap=False):
        # a bare Python float stands for an f32 scalar; F64(x) marks the f64 scalars of the reference's model code
        if isinstance(other, F64Scalar):
            o = self.full_like(other.value, "f64")
        else:
            o = other if isinstance(other, Tensor) else self.full_like(other)
        a, b = (o, self) if swap else (self, o)
        return Tensor(_lib.load().rai_binary(BINARY[name], a._h, b._h))

    def __add__(self, o): return self._binary("add", o)
    def __radd__(self, o): return self._binary("add", o, True)
    def __sub__(self, o): return self._binary("sub", o)
    def __rsub__(self, o): return self._binary("sub", o, True)
    def __mul__(self, o): return self._binary("mul", o)
    def __rmul__(self, o): return self._binary("mul", o, True)
    def __truediv__(self, o): return self._binary("div", o)
    def __rtruediv__(self, o): return self._binary("div", o, True)
    def maximum(self, o): return self._binary("maximum", o)
    def minimum(self, o): return self._binary("minimum", o)
    def eq(self, o): return self._binary("eq", o)
    def gt(self, o): return self._binary("gt", o)
    def lt(self, o): return self._binary("lt", o)

    def matmul(self, o):
        return Tensor(_lib.load().rai_matmul(self._h, o._h))

    def __matmul__(self, o): return self.matmul(o)

    def softmax(self, dim=-1):
        return Tensor(_lib.load().rai_softmax(self._h, dim))

    def log_softmax(self, dim=-1):
        return Tensor(_lib.load().rai_log_softmax(self._h, dim))

    def _reduce(self, name, dims, keep_dim):
        dims = list(range(len(self.shape))) if dims is None else ([dims] if isinstance(dims, int) else list(dims))
        arr = (C.c_int32 * max(len(dims), 1))(*dims)
        return Tensor(_lib.load().rai_reduce(REDUCE[name], self._h, arr, len(dims), int(keep_dim)))

    def sum(self, dims=None, keep_dim=False): return self._reduce("sum", dims, keep_dim)
    def max(self, dims=None, keep_dim=False): return self._reduce("max", dims, keep_dim)
    def min(self, dims=None, keep_dim=False): return self._reduce("min", dims, keep_dim)

    def argmax(self, dim=-1, keep_dim=False):
        return Tensor(_lib.load().rai_argmax(self._h, dim, int(keep_dim)))

    def argmin(self, dim=-1, keep_dim=False):
        return Tensor(_lib.load().rai_argmin(self._h, dim, int(keep_dim)))

    def index_select(self, dim, index):
        return Tensor(_lib.load().rai_index_select(self._h, dim, index._h))

    def gather(self, dim, index):
        return Tensor(_lib.load().rai_gather(self._h, dim, index._h))

    def index_add(self, dim, index, source):
        return Tensor(_lib.load().rai_index_add(self._h, dim, index._h, source._h))

    def scatter_add(self, dim, index, source):
        return Tensor(_lib.load().rai_scatter_add(self._h, dim, index._h, source._h))

    def narrow(self, dim, start, length):
        return Tensor(_lib.load().rai_narrow(self._h, dim, start, length))

    def where_cond(self, on_true, on_false):
        return Tensor(_lib.load().rai_where(self._h, on_true._h, on_false._h))

    def transpose(self, d0, d1):
        return Tensor(_lib.load().rai_transpose(self._h, d0, d1))

    def t(self):
        return self.transpose(-2, -1)

    def reshape(self, shape):
        arr, rank = _shape_arr(shape)
        return Tensor(_lib.load().rai_reshape(self._h, arr, rank))

    def permute(self, dims):
        arr = (C.c_int32 * len(dims))(*dims)
        return Tensor(_lib.load().rai_permute(self._h, arr, len(dims)))

    def broadcast_to(self, shape):
        arr, rank = _shape_arr(shape)
        return Tensor(_lib.load().rai_broadcast_to(self._h, arr, rank))

    def to_contiguous(self):
        return Tensor(_lib.load().rai_to_contiguous(self._h))

    def to_device(self, dev):
        """Tensor::to_device (ops/to_device.rs:48-59): the same tensor when it already lives on Hip(dev)."""
        return Tensor(_lib.load().rai_to_device(self._h, int(dev)))

    # ------------------------------------------------------------ high-level ops (the reference's decompositions)
    def flatten(self):
        return self.reshape((self.elem_count(),))

    def unsqueeze(self, dim):
        s = list(self.shape)
        # a negative dim inserts *after* that position (hlops/unsqueeze.rs:5-13)
        d = dim if dim >= 0 else len(s) + dim + 1
        s.insert(d, 1)
        return self.reshape(s)

    def mean(self, dims=None, keep_dim=False):
        dl = list(range(len(self.shape))) if dims is None else ([dims] if isinstance(dims, int) else list(dims))
        n = 1
        for d in dl:
            n *= self.shape[d]
        return self.sum(dims, keep_dim) / float(n)

    def var(self, dims=None, keep_dim=False, ddof=0):
        dl = list(range(len(self.shape))) if dims is None else ([dims] if isinstance(dims, int) else list(dims))
        n = 1
        for d in dl:
            n *= self.shape[d]
        m = self.mean(dims, True)
        s = (self - m).square().sum(dims, keep_dim)
        return s / float(n - ddof)

    def new_gelu(self):
        # 0.5 * x * (1 + tanh(sqrt(2/pi) * (x + 0.044715 * x^3))), f32 constants (activations.rs:25-27)
        k = float(np.float32(math.sqrt(2.0 / math.pi)))
        return 0.5 * self * (1.0 + (k * (self + float(np.float32(0.044715)) * self.powf(3.0))).tanh())

    def gelu(self):
        return self * 0.5 * (1.0 + (self / float(np.float32(math.sqrt(2.0)))).erf())

    def silu(self):
        return self / ((-self).exp() + 1.0)

    def relu(self):
        return self.maximum(self.full_like(0.0))


def cat(tensors, dim):
    arr = (C.c_void_p * len(tensors))(*[t._h for t in tensors])
    return Tensor(_lib.load().rai_concatenate(arr, len(tensors), dim))


def eval_all(tensors, retain_graph=False):
    arr = (C.c_void_p * max(len(tensors), 1))(*[t._h for t in tensors])
    check(_lib.load().rai_eval(arr, len(tensors), int(retain_graph)))


def eval_order(tensors):
    """Ids of the nodes eval() would visit, in order (utils.rs:35-66)."""
    arr = (C.c_void_p * max(len(tensors), 1))(*[t._h for t in tensors])
    n = C.c_int32(0)
    ids = (C.c_uint64 * 4096)()
    check(_lib.load().rai_graph_eval_order(arr, len(tensors), ids, 4096, C.byref(n)))
    return [int(ids[i]) for i in range(min(n.value, 4096))]


def set_fusion(enabled):
    check(_lib.load().rai_graph_set_fusion(int(bool(enabled))))


def set_compose(enabled):
    """Composition pass on / off: Linear + bias, LayerNorm, RmsNorm, rotary embedding and the attention block as one
    fused launch each (tolerance-level agreement with node-by-node evaluation)."""
    check(_lib.load().rai_graph_set_compose(int(bool(enabled))))


def stats(reset=False):
    s = GraphStats()
    check(_lib.load().rai_graph_get_stats(C.byref(s), int(reset)))
    return {"nodes_evaluated": s.nodes_evaluated, "kernel_launches": s.kernel_launches,
            "fused_regions": s.fused_regions, "fused_nodes": s.fused_nodes,
            "composed_regions": s.composed_regions, "composed_nodes": s.composed_nodes,
            "plan_ms": s.plan_ns * 1e-6, "run_ms": s.run_ns * 1e-6}


def dispatch_unregister(op):
    check(_lib.load().rai_dispatch_unregister(OP[op]))


def dispatch_register_builtin(op):
    check(_lib.load().rai_dispatch_register_builtin(OP[op]))


def dispatch_has_rule(op):
    return bool(_lib.load().rai_dispatch_has_rule(OP[op]))


# ---------------------------------------------------------------- rai-nn modules as functions
def linear(x, weight, bias=None):
    """x @ broadcast_left(W).t() + b (rai-nn/src/linear.rs:59-69)."""
    w = weight
    if len(x.shape) > 2:
        w = weight.broadcast_to(tuple(x.shape[:-2]) + tuple(weight.shape))
    y = x.matmul(w.t())
    return y + bias if bias is not None else y


def layer_norm(x, weight, bias, eps):
    """w * ((x - mean) * rsqrt(var + eps)) + b over the last dim (rai-nn/src/layer_norm.rs:32-42)."""
    mean = x.mean(-1, True)
    var = x.var(-1, True)
    xs = (x - mean) * (var + eps).rsqrt()
    y = weight * xs if weight is not None else xs
    return y + bias if bias is not None else y


def rms_norm(x, weight, eps):
    """s = 1 / sqrt(n); weight * x * rsqrt(sum((x * s)^2) + eps) (rai-nn/src/rms_norm.rs:18-22)."""
    n = x.shape[-1]
    s = (x * (1.0 / math.sqrt(n))).square().sum(-1, True)
    return weight * x * (s + eps).rsqrt()


def embedding(ids, table):
    """flatten ids -> index_select dim 0 -> reshape [.., H] (rai-nn/src/embedding.rs:25-30)."""
    flat = ids.flatten()
    out = table.index_select(0, flat)
    return out.reshape(tuple(ids.shape) + (table.shape[1],))
