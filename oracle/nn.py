"""rai-nn modules and rai-core hlops restated as compositions of oracle.ops.

Test infrastructure only (see oracle/__init__.py).  Every step is a separate
primitive with its own storage rounding, as in the reference where the lazy
graph is evaluated node by node.
"""
import math

import numpy as np

from . import ops
from .dtypes import carrier


def mean(x, dim, keep_dim, dt):
    """hlops/mean.rs:4-7: sum(args) / elem_count, the divisor is a f64 scalar
    turned into a Full<F64>.to_dtype(x) tensor (ops/mod.rs:262-276)."""
    n = np.shape(x)[dim]
    return ops.div(ops.reduce_sum(x, dim, keep_dim, dt), ops.full_like(np.zeros(()), float(n), dt, "f64"), dt)


def var(x, dim, keep_dim, dt, ddof=0):
    """hlops/var.rs:33-38: population variance, divisor is a f32 scalar."""
    n = np.shape(x)[dim]
    m = mean(x, dim, keep_dim, dt)
    s = ops.reduce_sum(ops.square(ops.sub(x, m, dt), dt), dim, keep_dim, dt)
    return ops.div(s, ops.full_like(np.zeros(()), float(n - ddof), dt, "f32"), dt)


def layer_norm(x, weight, bias, eps, dt):
    """LayerNorm::fwd rai-nn/src/layer_norm.rs:32-42."""
    m = mean(x, -1, True, dt)
    v = var(x, -1, True, dt)
    xn = ops.mul(ops.sub(x, m, dt), ops.rsqrt(ops.add(v, ops.full_like(np.zeros(()), eps, dt, "f64"), dt), dt), dt)
    if weight is None:
        return xn
    return ops.add(ops.mul(weight, xn, dt), bias, dt)


def rms_norm(x, weight, eps, dt):
    """RmsNorm::fwd rai-nn/src/rms_norm.rs:18-22:
    s = 1/sqrt(n); n = rsqrt(sum((x*s)^2) + eps); weight * x * n."""
    s = 1.0 / math.sqrt(np.shape(x)[-1])
    xs = ops.mul(x, ops.full_like(np.zeros(()), s, dt, "f64"), dt)
    n = ops.rsqrt(ops.add(ops.reduce_sum(ops.square(xs, dt), -1, True, dt), ops.full_like(np.zeros(()), eps, dt, "f64"), dt), dt)
    return ops.mul(ops.mul(weight, x, dt), n, dt)


def gemma_rms_norm(x, weight, eps, dt):
    """RmsNorm::fwd rai-models/src/llm/gemma.rs:42-54: upcast to f32 for bf16/f16
    inputs, x / sqrt(mean(x^2) + eps), cast back, times (weight + 1)."""
    internal = "f32" if dt in ("bf16", "f16") else dt
    hidden = np.shape(x)[-1]
    xi = ops.to_dtype(x, dt, internal)
    norm = ops.div(ops.reduce_sum(ops.square(xi, internal), -1, True, internal),
                   ops.full_like(np.zeros(()), float(hidden), internal, "f64"), internal)
    xn = ops.div(xi, ops.sqrt(ops.add(norm, ops.full_like(np.zeros(()), eps, internal, "f64"), internal), internal), internal)
    xn = ops.to_dtype(xn, internal, dt)
    return ops.mul(xn, ops.add(weight, ops.full_like(np.zeros(()), 1.0, dt, "f64"), dt), dt)


def linear(x, weight, bias, dt):
    """Linear::fwd rai-nn/src/linear.rs:59-69: x @ W^T (+ bias), W is [out, in]."""
    y = ops.matmul(x, np.swapaxes(weight, -1, -2), dt)
    return y if bias is None else ops.add(y, bias, dt)


def embedding(ids, weight):
    """Embedding::fwd rai-nn/src/embedding.rs:25-30."""
    ids = np.asarray(ids)
    out = ops.index_select(weight, 0, ids.reshape(-1))
    return out.reshape(tuple(ids.shape) + (weight.shape[-1],))


def _c(val, dt, val_dt="f32"):
    return ops.full_like(np.zeros(()), val, dt, val_dt)


def gelu(x, dt):
    """hlops/activations.rs:20-22: x * 0.5 * (1 + erf(x / sqrt(2))) with f32 scalars."""
    inner = ops.erf(ops.div(x, _c(np.float32(2.0) ** np.float32(0.5), dt), dt), dt)
    return ops.mul(ops.mul(x, _c(0.5, dt), dt), ops.add(_c(1.0, dt), inner, dt), dt)


def new_gelu(x, dt):
    """hlops/activations.rs:25-27:
    0.5 * x * (1 + tanh(sqrt(2/pi) * (x + 0.044715 * x.powf(3))))  (f32 scalars)."""
    k = np.sqrt(np.float32(2.0) / np.float32(np.pi)).astype(np.float32)
    x3 = ops.powf(x, 3.0, dt)
    inner = ops.add(x, ops.mul(_c(np.float32(0.044715), dt), x3, dt), dt)
    t = ops.tanh(ops.mul(_c(k, dt), inner, dt), dt)
    return ops.mul(ops.mul(_c(0.5, dt), x, dt), ops.add(_c(1.0, dt), t, dt), dt)


def silu(x, dt):
    """hlops/activations.rs:30-32: x / (exp(-x) + 1)."""
    return ops.div(x, ops.add(ops.exp(ops.neg(x, dt), dt), _c(1.0, dt), dt), dt)


def relu(x, dt):
    """hlops/activations.rs:5-7."""
    return ops.maximum(x, np.zeros_like(np.asarray(x, dtype=carrier(dt))), dt)


ACTIVATIONS = {"gelu": gelu, "gelu_new": new_gelu, "new_gelu": new_gelu, "silu": silu, "relu": relu}


def activation(name):
    """Activation parsing rai-nn/src/activations.rs:5-17 (alias gelu_new)."""
    return ACTIVATIONS[name]
