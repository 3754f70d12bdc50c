"""Phi-2 decoder (rai-models/src/llm/phi2.rs) restated over oracle.ops / oracle.nn.

Test infrastructure only (see oracle/__init__.py).
"""
import math

import numpy as np

from . import nn, ops
from .dtypes import rnd


class Config:
    """phi2.rs:9-24 (serde Config)."""

    def __init__(self, vocab_size=51200, hidden_size=2560, intermediate_size=10240, num_hidden_layers=32,
                 num_attention_heads=32, num_key_value_heads=None, hidden_act="gelu_new",
                 max_position_embeddings=2048, layer_norm_eps=1e-5, tie_word_embeddings=False, rope_theta=10000.0,
                 partial_rotary_factor=0.4, qk_layernorm=False):
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.num_hidden_layers = num_hidden_layers
        self.num_attention_heads = num_attention_heads
        self.num_key_value_heads = num_key_value_heads or num_attention_heads
        self.hidden_act = hidden_act
        self.max_position_embeddings = max_position_embeddings
        self.layer_norm_eps = layer_norm_eps
        self.tie_word_embeddings = tie_word_embeddings
        self.rope_theta = rope_theta
        self.partial_rotary_factor = partial_rotary_factor
        self.qk_layernorm = qk_layernorm

    @property
    def head_dim(self):
        return self.hidden_size // self.num_attention_heads

    @property
    def rotary_dim(self):
        return int(self.partial_rotary_factor * self.head_dim)


def param_shapes(cfg):
    """Parameter names as produced by #[derive(Module)] with the renames at
    phi2.rs:307-313 and the naming rule rai-core/src/nn.rs:183-205,256-268."""
    h, i, v = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    kv = cfg.num_key_value_heads * cfg.head_dim
    out = {"model.embed_tokens.weight": (v, h)}
    for l in range(cfg.num_hidden_layers):
        p = f"model.layers.{l}."
        out[p + "self_attn.q_proj.weight"] = (h, h)
        out[p + "self_attn.q_proj.bias"] = (h,)
        out[p + "self_attn.k_proj.weight"] = (kv, h)
        out[p + "self_attn.k_proj.bias"] = (kv,)
        out[p + "self_attn.v_proj.weight"] = (kv, h)
        out[p + "self_attn.v_proj.bias"] = (kv,)
        out[p + "self_attn.dense.weight"] = (h, h)
        out[p + "self_attn.dense.bias"] = (h,)
        if cfg.qk_layernorm:   # phi2.rs:163-169: LayerNorm::new(head_dim, ..)
            for n in ("q_layernorm", "k_layernorm"):
                out[p + f"self_attn.{n}.weight"] = (cfg.head_dim,)
                out[p + f"self_attn.{n}.bias"] = (cfg.head_dim,)
        out[p + "mlp.fc1.weight"] = (i, h)
        out[p + "mlp.fc1.bias"] = (i,)
        out[p + "mlp.fc2.weight"] = (h, i)
        out[p + "mlp.fc2.bias"] = (h,)
        out[p + "input_layernorm.weight"] = (h,)
        out[p + "input_layernorm.bias"] = (h,)
    out["model.final_layernorm.weight"] = (h,)
    out["model.final_layernorm.bias"] = (h,)
    out["lm_head.weight"] = (v, h)
    out["lm_head.bias"] = (v,)
    return out


def rotary_tables(cfg, dt):
    """RotaryEmbedding::new phi2.rs:44-64: inv_freq via f32 powf, positions and the
    outer product computed IN THE MODEL DTYPE, cat(freqs, freqs), sin / cos."""
    dim = cfg.rotary_dim
    theta = np.float32(cfg.rope_theta)
    inv = np.array([np.float32(1.0) / np.power(theta, np.float32(i) / np.float32(dim), dtype=np.float32)
                    for i in range(0, dim, 2)], dtype=np.float32)
    inv = ops.to_dtype(inv.reshape(1, -1), "f32", dt)
    t = ops.to_dtype(np.arange(cfg.max_position_embeddings, dtype=np.uint32), "u32", dt).reshape(-1, 1)
    freqs = ops.matmul(t, inv, dt)
    emb = np.concatenate([freqs, freqs], axis=-1)
    return ops.sin(emb, dt), ops.cos(emb, dt)


def rotary(xs, sin, cos, dim, offset, dt):
    """RotaryEmbedding::fwd phi2.rs:66-77 (NeoX rotate-half on the first `dim`)."""
    seq_len, headdim = xs.shape[2], xs.shape[3]
    xs_rot = ops.narrow(xs, 3, 0, dim)
    xs_pass = ops.narrow(xs, 3, dim, headdim - dim)
    xs1, xs2 = ops.chunk(xs_rot, 2, -1)
    c = ops.narrow(cos, 0, offset, seq_len)
    s = ops.narrow(sin, 0, offset, seq_len)
    rotate_half = np.concatenate([ops.neg(xs2, dt), xs1], axis=-1)
    xs_rot = ops.add(ops.mul(xs_rot, c, dt), ops.mul(rotate_half, s, dt), dt)
    return np.concatenate([xs_rot, xs_pass], axis=-1)


def get_mask(size):
    """phi2.rs:104-109: u8 [S,S], 1 where j > i."""
    i = np.arange(size)[:, None]
    j = np.arange(size)[None, :]
    return (j > i).astype(np.uint8)


class Model:
    """phi2.rs:302-353.  `params` maps the names of param_shapes() to carrier arrays."""

    def __init__(self, cfg, params, dt):
        self.cfg, self.p, self.dt = cfg, params, dt
        self.sin, self.cos = rotary_tables(cfg, dt)
        self.kv = [None] * cfg.num_hidden_layers
        self.act = nn.activation(cfg.hidden_act)

    def clear_kv_cache(self):
        self.kv = [None] * self.cfg.num_hidden_layers

    def _attention(self, l, xs, mask):
        cfg, dt, p = self.cfg, self.dt, self.p
        pre = f"model.layers.{l}.self_attn."
        b, s, _ = xs.shape
        nh, nkv, hd = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
        q = nn.linear(xs, p[pre + "q_proj.weight"], p[pre + "q_proj.bias"], dt)
        k = nn.linear(xs, p[pre + "k_proj.weight"], p[pre + "k_proj.bias"], dt)
        v = nn.linear(xs, p[pre + "v_proj.weight"], p[pre + "v_proj.bias"], dt)
        if cfg.qk_layernorm:
            # phi2.rs:207-216 applies the LayerNorm (parameters of head_dim elements) to the projections BEFORE they
            # are split into heads, i.e. over a last dim of heads * head_dim: broadcasting the [head_dim] weight against
            # it is an IncompatibleShape error node unless there is a single head.  Restated as is.
            if nh * hd != hd or nkv * hd != hd:
                raise ValueError(f"IncompatibleShape {{ lhs: [{hd}], rhs: [{b}, {s}, {nh * hd}] }}")
            q = nn.layer_norm(q, p[pre + "q_layernorm.weight"], p[pre + "q_layernorm.bias"], cfg.layer_norm_eps, dt)
            k = nn.layer_norm(k, p[pre + "k_layernorm.weight"], p[pre + "k_layernorm.bias"], cfg.layer_norm_eps, dt)
        q = q.reshape(b, s, nh, hd).transpose(0, 2, 1, 3)
        k = k.reshape(b, s, nkv, hd).transpose(0, 2, 1, 3)
        v = v.reshape(b, s, nkv, hd).transpose(0, 2, 1, 3)
        offset = 0 if self.kv[l] is None else self.kv[l][0].shape[2]
        q = rotary(q, self.sin, self.cos, cfg.rotary_dim, offset, dt)
        k = rotary(k, self.sin, self.cos, cfg.rotary_dim, offset, dt)
        if self.kv[l] is not None:
            k = np.concatenate([self.kv[l][0], k], axis=2)
            v = np.concatenate([self.kv[l][1], v], axis=2)
        self.kv[l] = (k, v)
        n_rep = nh // nkv
        if n_rep > 1:  # repeat_kv phi2.rs:190-200
            k = np.repeat(k, n_rep, axis=1)
            v = np.repeat(v, n_rep, axis=1)
        # phi2.rs:248-251: q.f32 @ (k.f32.t() * scale), scale is a f64 scalar -> Full<F64>.to_dtype(F32)
        scale = 1.0 / math.sqrt(hd)
        qf = ops.to_dtype(q, dt, "f32")
        kf = ops.mul(np.swapaxes(ops.to_dtype(k, dt, "f32"), -1, -2), ops.full_like(np.zeros(()), scale, "f32", "f64"), "f32")
        w = ops.matmul(qf, kf, "f32")
        if mask is not None:  # masked_fill phi2.rs:111-117
            w = ops.where(np.broadcast_to(mask, w.shape), np.float32(-np.inf), w, "f32")
        w = ops.to_dtype(ops.softmax(w, -1, "f32"), "f32", dt)
        o = ops.matmul(w, v, dt).transpose(0, 2, 1, 3).reshape(b, s, nh * hd)
        return nn.linear(o, p[pre + "dense.weight"], p[pre + "dense.bias"], dt)

    def layer(self, l, xs, mask):
        """DecoderLayer::fwd phi2.rs:293-299: one LayerNorm, attn + mlp + residual."""
        dt, p = self.dt, self.p
        pre = f"model.layers.{l}."
        ln = nn.layer_norm(xs, p[pre + "input_layernorm.weight"], p[pre + "input_layernorm.bias"],
                           self.cfg.layer_norm_eps, dt)
        attn = self._attention(l, ln, mask)
        h = nn.linear(ln, p[pre + "mlp.fc1.weight"], p[pre + "mlp.fc1.bias"], dt)
        h = self.act(h, dt)
        mlp = nn.linear(h, p[pre + "mlp.fc2.weight"], p[pre + "mlp.fc2.bias"], dt)
        return ops.add(ops.add(attn, mlp, dt), xs, dt)

    def hidden(self, ids):
        """Everything of Model::fwd up to the final LayerNorm input."""
        ids = np.asarray(ids)
        s = ids.shape[1]
        xs = nn.embedding(ids, self.p["model.embed_tokens.weight"])
        mask = None if s <= 1 else get_mask(s)
        for l in range(self.cfg.num_hidden_layers):
            xs = self.layer(l, xs, mask)
        return xs

    def fwd(self, ids):
        """Model::fwd phi2.rs:334-347: logits of the last position, [B, vocab]."""
        p, dt = self.p, self.dt
        xs = self.hidden(ids)
        s = xs.shape[1]
        xs = nn.layer_norm(xs, p["model.final_layernorm.weight"], p["model.final_layernorm.bias"],
                           self.cfg.layer_norm_eps, dt)
        xs = ops.narrow(xs, 1, s - 1, 1)
        head_w = p["model.embed_tokens.weight"] if self.cfg.tie_word_embeddings else p["lm_head.weight"]
        head_b = None if self.cfg.tie_word_embeddings else p.get("lm_head.bias")
        return nn.linear(xs, head_w, head_b, dt)[:, 0, :]


def greedy_decode(model, prompt, n_new):
    """examples/phi2/src/main.rs:75-95 with plain argmax (no repeat penalty):
    the whole prompt first, then one token per step; returns [B, n_new] u32 and
    the per-step logits."""
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
    """Synthetic weights: N(0, std) matrices and embeddings, zero biases, unit
    LayerNorm weights; generated in f32 from PCG64(seed) in param_shapes() order
    and rounded to `dt`."""
    rng = np.random.Generator(np.random.PCG64(seed))
    out = {}
    for name, shape in param_shapes(cfg).items():
        if name.endswith("layernorm.weight"):
            a = np.ones(shape, dtype=np.float32)
        elif name.endswith(".bias"):
            a = np.zeros(shape, dtype=np.float32)
        else:
            a = rng.standard_normal(shape, dtype=np.float32) * np.float32(std)
        out[name] = rnd(a, dt)
    return out
