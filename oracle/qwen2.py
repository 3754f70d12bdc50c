"""Qwen2 and Gemma decoders (rai-models/src/llm/qwen2.rs, gemma.rs) restated over
oracle.ops / oracle.nn.  Test infrastructure only (see oracle/__init__.py).

The two files share their structure (sequential pre-norm block, full-dimension
rotary embedding, additive causal mask, scores/softmax in the model dtype,
gated MLP); they differ in the norm (rai-nn RmsNorm vs Gemma's f32-internal
(1 + w) variant), q/k/v biases, embedding scaling and the tied head.

qwen2.rs hard-codes num_kv_groups = 1 and sizes k/v projections hidden->hidden
(qwen2.rs:138-139,150), so it cannot express a grouped-query configuration; for
num_key_value_heads < num_attention_heads this restatement follows gemma.rs
(:167, :191-201: kv projections of num_kv_heads*head_dim and repeat_kv).
"""
import math

import numpy as np

from . import nn, ops
from .dtypes import rnd


class Config:
    """Union of qwen2.rs:8-24 and gemma.rs:12-27."""

    def __init__(self, arch, vocab_size, hidden_size, intermediate_size, num_hidden_layers, num_attention_heads,
                 num_key_value_heads, hidden_act, max_position_embeddings=4096, rms_norm_eps=1e-6, rope_theta=10000.0,
                 head_dim=None):
        assert arch in ("qwen2", "gemma")
        self.arch = arch
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.num_hidden_layers = num_hidden_layers
        self.num_attention_heads = num_attention_heads
        self.num_key_value_heads = num_key_value_heads
        self.hidden_act = hidden_act
        self.max_position_embeddings = max_position_embeddings
        self.rms_norm_eps = rms_norm_eps
        self.rope_theta = rope_theta
        self.head_dim = head_dim or hidden_size // num_attention_heads


def param_shapes(cfg):
    """Names per qwen2.rs:276-282 / gemma.rs:309-319 and rai-core/src/nn.rs:183-205."""
    h, i, v = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    qd, kd = cfg.num_attention_heads * cfg.head_dim, cfg.num_key_value_heads * cfg.head_dim
    out = {"model.embed_tokens.weight": (v, h)}
    for l in range(cfg.num_hidden_layers):
        p = f"model.layers.{l}."
        out[p + "self_attn.q_proj.weight"] = (qd, h)
        out[p + "self_attn.k_proj.weight"] = (kd, h)
        out[p + "self_attn.v_proj.weight"] = (kd, h)
        if cfg.arch == "qwen2":
            out[p + "self_attn.q_proj.bias"] = (qd,)
            out[p + "self_attn.k_proj.bias"] = (kd,)
            out[p + "self_attn.v_proj.bias"] = (kd,)
        out[p + "self_attn.o_proj.weight"] = (h, qd)
        out[p + "mlp.gate_proj.weight"] = (i, h)
        out[p + "mlp.up_proj.weight"] = (i, h)
        out[p + "mlp.down_proj.weight"] = (h, i)
        out[p + "input_layernorm.weight"] = (h,)
        out[p + "post_attention_layernorm.weight"] = (h,)
    out["model.norm.weight"] = (h,)
    if cfg.arch == "qwen2":
        out["lm_head.weight"] = (v, h)
    return out


def rotary_tables(cfg, dt):
    """RotaryEmbedding::new qwen2.rs:40-58 / gemma.rs:72-90: inv_freq from an f64 powf
    cast to f32, then positions and the outer product IN THE MODEL DTYPE."""
    dim = cfg.head_dim
    inv = np.array([np.float32(1.0) / np.float32(cfg.rope_theta ** (i / dim)) for i in range(0, dim, 2)], np.float32)
    inv = ops.to_dtype(inv.reshape(1, -1), "f32", dt)
    t = ops.to_dtype(np.arange(cfg.max_position_embeddings, dtype=np.uint32), "u32", dt).reshape(-1, 1)
    freqs = ops.matmul(t, inv, dt)
    freqs = np.concatenate([freqs, freqs], axis=-1)
    return ops.sin(freqs, dt), ops.cos(freqs, dt)


def rotate_half(xs, dt):
    """qwen2.rs:32-37."""
    half = xs.shape[-1] // 2
    return np.concatenate([ops.neg(xs[..., half:], dt), xs[..., :half]], axis=-1)


def apply_rotary(x, sin, cos, offset, dt):
    """RotaryEmbedding::fwd qwen2.rs:60-71: q * cos + rotate_half(q) * sin."""
    s = x.shape[2]
    c, sn = cos[offset:offset + s][None, None], sin[offset:offset + s][None, None]
    return ops.add(ops.mul(x, c, dt), ops.mul(rotate_half(x, dt), sn, dt), dt)


def causal_mask(tgt, offset, dt):
    """prepare_decoder_attention_mask qwen2.rs:306-336 / gemma.rs:341-362 (no sliding
    window in play for contexts below it): f32 -inf above the diagonal, zero
    padding for the cached positions, cast to the model dtype."""
    i = np.arange(tgt)[:, None]
    j = np.arange(tgt)[None, :]
    m = np.where(i < j, np.float32(-np.inf), np.float32(0)).astype(np.float32)
    if offset > 0:
        m = np.concatenate([np.zeros((tgt, offset), np.float32), m], axis=-1)
    return ops.to_dtype(m, "f32", dt)


class Model:
    def __init__(self, cfg, params, dt):
        self.cfg, self.p, self.dt = cfg, params, dt
        self.sin, self.cos = rotary_tables(cfg, dt)
        self.kv = [None] * cfg.num_hidden_layers
        self.act = nn.activation(cfg.hidden_act)

    def clear_kv_cache(self):
        self.kv = [None] * self.cfg.num_hidden_layers

    def _norm(self, x, w):
        if self.cfg.arch == "gemma":
            return nn.gemma_rms_norm(x, w, self.cfg.rms_norm_eps, self.dt)
        return nn.rms_norm(x, w, self.cfg.rms_norm_eps, self.dt)

    def _attention(self, l, xs, mask, offset):
        """Attention::fwd qwen2.rs:166-221 / gemma.rs:203-259."""
        cfg, dt, p = self.cfg, self.dt, self.p
        pre = f"model.layers.{l}.self_attn."
        b, s, _ = xs.shape
        nh, nkv, hd = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
        q = nn.linear(xs, p[pre + "q_proj.weight"], p.get(pre + "q_proj.bias"), dt)
        k = nn.linear(xs, p[pre + "k_proj.weight"], p.get(pre + "k_proj.bias"), dt)
        v = nn.linear(xs, p[pre + "v_proj.weight"], p.get(pre + "v_proj.bias"), dt)
        q = q.reshape(b, s, nh, hd).transpose(0, 2, 1, 3)
        k = k.reshape(b, s, nkv, hd).transpose(0, 2, 1, 3)
        v = v.reshape(b, s, nkv, hd).transpose(0, 2, 1, 3)
        q = apply_rotary(q, self.sin, self.cos, offset, dt)
        k = apply_rotary(k, self.sin, self.cos, offset, dt)
        if self.kv[l] is not None:
            k = np.concatenate([self.kv[l][0], k], axis=2)
            v = np.concatenate([self.kv[l][1], v], axis=2)
        self.kv[l] = (k, v)
        n_rep = nh // nkv
        if n_rep > 1:  # repeat_kv gemma.rs:191-201
            k = np.repeat(k, n_rep, axis=1)
            v = np.repeat(v, n_rep, axis=1)
        scale = 1.0 / math.sqrt(hd)
        w = ops.mul(ops.matmul(q, np.swapaxes(k, -1, -2), dt), ops.full_like(np.zeros(()), scale, dt, "f64"), dt)
        if mask is not None:
            w = ops.add(w, mask, dt)
        w = ops.softmax(w, -1, dt)
        o = ops.matmul(w, v, dt).transpose(0, 2, 1, 3).reshape(b, s, nh * hd)
        return nn.linear(o, p[pre + "o_proj.weight"], None, dt)

    def layer(self, l, xs, mask, offset):
        """DecoderLayer::fwd qwen2.rs:253-266 / gemma.rs:286-299."""
        dt, p = self.dt, self.p
        pre = f"model.layers.{l}."
        h = self._attention(l, self._norm(xs, p[pre + "input_layernorm.weight"]), mask, offset)
        xs = ops.add(h, xs, dt)
        y = self._norm(xs, p[pre + "post_attention_layernorm.weight"])
        lhs = self.act(nn.linear(y, p[pre + "mlp.gate_proj.weight"], None, dt), dt)
        rhs = nn.linear(y, p[pre + "mlp.up_proj.weight"], None, dt)
        mlp = nn.linear(ops.mul(lhs, rhs, dt), p[pre + "mlp.down_proj.weight"], None, dt)
        return ops.add(xs, mlp, dt)

    def fwd(self, ids):
        """Model::fwd qwen2.rs:338-359 / gemma.rs:364-386: logits of the last position, [B, vocab]."""
        cfg, dt, p = self.cfg, self.dt, self.p
        ids = np.asarray(ids)
        s = ids.shape[1]
        offset = 0 if self.kv[0] is None else self.kv[0][0].shape[2]
        mask = None if s <= 1 else causal_mask(s, offset, dt)
        xs = nn.embedding(ids, p["model.embed_tokens.weight"])
        if cfg.arch == "gemma":  # gemma.rs:379: xs * sqrt(hidden) with a f64 scalar cast to the model dtype
            xs = ops.mul(xs, ops.full_like(np.zeros(()), math.sqrt(cfg.hidden_size), dt, "f64"), dt)
        for l in range(cfg.num_hidden_layers):
            xs = self.layer(l, xs, mask, offset)
        xs = self._norm(ops.narrow(xs, 1, s - 1, 1), p["model.norm.weight"])
        head = p["model.embed_tokens.weight"] if cfg.arch == "gemma" else p["lm_head.weight"]
        return nn.linear(xs, head, None, dt)[:, 0, :]


def greedy_decode(model, prompt, n_new):
    """examples/qwen2/src/main.rs / gemma main.rs decode loop with plain argmax."""
    prompt = np.asarray(prompt, dtype=np.uint32)
    model.clear_kv_cache()
    tokens, logits_all = [], []
    ctx = prompt
    for _ in range(n_new):
        logits = model.fwd(ctx)
        nxt = ops.argmax(logits, -1)
        tokens.append(nxt)
        logits_all.append(logits)
        ctx = nxt.reshape(-1, 1)
    return np.stack(tokens, axis=1), logits_all


def random_params(cfg, dt, seed=0, std=0.02):
    """N(0, std) matrices; norm weights 1 for Qwen2, 0 for Gemma (so 1 + w = 1); zero biases."""
    rng = np.random.Generator(np.random.PCG64(seed))
    out = {}
    for name, shape in param_shapes(cfg).items():
        if name.endswith("norm.weight"):
            a = np.zeros(shape, np.float32) if cfg.arch == "gemma" else np.ones(shape, np.float32)
        elif name.endswith(".bias"):
            a = np.zeros(shape, np.float32)
        else:
            a = rng.standard_normal(shape, dtype=np.float32) * np.float32(std)
        out[name] = rnd(a, dt)
    return out
