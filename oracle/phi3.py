"""Phi-3 restated from rai-models/src/llm/phi3.rs (TEST INFRASTRUCTURE ONLY, like the rest of this
package): the sequential pre-norm block of Qwen2 with a fused qkv_proj and a fused gate_up_proj, no
biases, rai-nn RmsNorm, an untied bias-free lm_head.  Builds on oracle/qwen2.py for everything the two
files share (rotary application, mask, attention contractions).

Pinned by tests/test_oracle_phi3.py against Hugging Face transformers' Phi3ForCausalLM built locally
from an in-memory config and loaded with the oracle's seeded weights (parameter names coincide with
rai's, phi3.rs:262-270 + rai-core/src/nn.rs:183-205).
"""
import math

import numpy as np

from . import nn, ops
from . import qwen2 as _q
from .dtypes import rnd


class Config(_q.Config):
    """phi3.rs:9-30; head_dim = hidden_size / num_attention_heads (:26-29)."""

    def __init__(self, vocab_size, hidden_size, intermediate_size, num_hidden_layers, num_attention_heads,
                 num_key_value_heads, hidden_act="silu", max_position_embeddings=4096, rms_norm_eps=1e-5,
                 rope_theta=10000.0):
        _q.Config.__init__(self, "qwen2", vocab_size, hidden_size, intermediate_size, num_hidden_layers,
                           num_attention_heads, num_key_value_heads, hidden_act, max_position_embeddings, rms_norm_eps,
                           rope_theta, None)
        self.arch = "phi3"


def param_shapes(cfg):
    """Names per phi3.rs:262-270 (model.embed_tokens, model.layers, model.norm, lm_head) and the field names
    of Attention :114-117, MLP :79-82, DecoderLayer :232-237."""
    h, i, v = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    qd, kd = cfg.num_attention_heads * cfg.head_dim, cfg.num_key_value_heads * cfg.head_dim
    out = {"model.embed_tokens.weight": (v, h)}
    for l in range(cfg.num_hidden_layers):
        p = f"model.layers.{l}."
        out[p + "self_attn.qkv_proj.weight"] = (qd + 2 * kd, h)
        out[p + "self_attn.o_proj.weight"] = (h, qd)
        out[p + "mlp.gate_up_proj.weight"] = (2 * i, h)
        out[p + "mlp.down_proj.weight"] = (h, i)
        out[p + "input_layernorm.weight"] = (h,)
        out[p + "post_attention_layernorm.weight"] = (h,)
    out["model.norm.weight"] = (h,)
    out["lm_head.weight"] = (v, h)
    return out


def rotary_tables(cfg, dt):
    """RotaryEmbedding::new phi3.rs:41-62: inv_freq as an f64 tensor cast to the model dtype (one rounding
    from f64), then positions and the outer product in the model dtype."""
    dim = cfg.head_dim
    inv = np.array([1.0 / cfg.rope_theta ** (i / dim) for i in range(0, dim, 2)], np.float64)
    inv = ops.to_dtype(inv.reshape(1, -1), "f64", dt)
    t = ops.to_dtype(np.arange(cfg.max_position_embeddings, dtype=np.uint32), "u32", dt).reshape(-1, 1)
    freqs = ops.matmul(t, inv, dt)
    freqs = np.concatenate([freqs, freqs], axis=-1)
    return ops.sin(freqs, dt), ops.cos(freqs, dt)


class Model(_q.Model):
    def __init__(self, cfg, params, dt):
        self.cfg, self.p, self.dt = cfg, params, dt
        self.sin, self.cos = rotary_tables(cfg, dt)
        self.kv = [None] * cfg.num_hidden_layers
        self.act = nn.activation(cfg.hidden_act)

    def _attention(self, l, xs, mask, offset):
        """Attention::fwd phi3.rs:164-215: one projection, narrowed into q | k | v."""
        cfg, dt, p = self.cfg, self.dt, self.p
        pre = f"model.layers.{l}.self_attn."
        b, s, _ = xs.shape
        nh, nkv, hd = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
        qkv = nn.linear(xs, p[pre + "qkv_proj.weight"], None, dt)
        q = ops.narrow(qkv, -1, 0, nh * hd).reshape(b, s, nh, hd).transpose(0, 2, 1, 3)
        k = ops.narrow(qkv, -1, nh * hd, nkv * hd).reshape(b, s, nkv, hd).transpose(0, 2, 1, 3)
        v = ops.narrow(qkv, -1, (nh + nkv) * hd, nkv * hd).reshape(b, s, nkv, hd).transpose(0, 2, 1, 3)
        q = _q.apply_rotary(q, self.sin, self.cos, offset, dt)
        k = _q.apply_rotary(k, self.sin, self.cos, offset, dt)
        if self.kv[l] is not None:
            k = np.concatenate([self.kv[l][0], k], axis=2)
            v = np.concatenate([self.kv[l][1], v], axis=2)
        self.kv[l] = (k, v)
        n_rep = nh // nkv
        if n_rep > 1:  # repeat_kv phi3.rs:152-162
            k = np.repeat(k, n_rep, axis=1)
            v = np.repeat(v, n_rep, axis=1)
        scale = np.float32(1.0) / np.float32(math.sqrt(np.float32(hd)))       # f32 scalar, phi3.rs:202
        w = ops.mul(ops.matmul(q, np.swapaxes(k, -1, -2), dt), ops.full_like(np.zeros(()), float(scale), dt, "f32"), dt)
        if mask is not None:
            w = ops.add(w, mask, dt)
        w = ops.softmax(w, -1, dt)
        o = ops.matmul(w, v, dt).transpose(0, 2, 1, 3).reshape(b, s, nh * hd)
        return nn.linear(o, p[pre + "o_proj.weight"], None, dt)

    def layer(self, l, xs, mask, offset):
        """DecoderLayer::fwd phi3.rs:257-265 and MLP::fwd :97-103 (up * act(gate))."""
        dt, p, i = self.dt, self.p, self.cfg.intermediate_size
        pre = f"model.layers.{l}."
        h = self._attention(l, self._norm(xs, p[pre + "input_layernorm.weight"]), mask, offset)
        xs = ops.add(h, xs, dt)
        y = self._norm(xs, p[pre + "post_attention_layernorm.weight"])
        gu = nn.linear(y, p[pre + "mlp.gate_up_proj.weight"], None, dt)
        gate, up = ops.narrow(gu, -1, 0, i), ops.narrow(gu, -1, i, i)
        mlp = nn.linear(ops.mul(up, self.act(gate, dt), dt), p[pre + "mlp.down_proj.weight"], None, dt)
        return ops.add(xs, mlp, dt)


greedy_decode = _q.greedy_decode


def random_params(cfg, dt, seed=0, std=0.02):
    """N(0, std) matrices, unit norm weights."""
    rng = np.random.Generator(np.random.PCG64(seed))
    out = {}
    for name, shape in param_shapes(cfg).items():
        if name.endswith("norm.weight"):
            a = np.ones(shape, np.float32)
        else:
            a = rng.standard_normal(shape, dtype=np.float32) * np.float32(std)
        out[name] = rnd(a, dt)
    return out
