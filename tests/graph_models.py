"""Phi-2 written against the lazy `Tensor` API, node for node as
rai-models/src/llm/phi2.rs builds it (RotaryEmbedding :44-78, masked_fill :111-117,
Attention::fwd :202-264, MLP :99-101, DecoderLayer::fwd :293-299, Model::fwd :334-347),
and Qwen2 / Gemma as rai-models/src/llm/qwen2.rs and gemma.rs build them (SeqGraph).

Nothing here computes: every call records graph nodes; `eval()` / `as_storage()`
runs them on the Hip device through the dispatcher.  This is the reference's own
execution scheme (one primitive per node, KV cache by concatenation) and serves
as the functional drop-in path; the fused decoder drivers are the fast path.
"""
from __future__ import annotations

import math

import numpy as np

from rai_amd import graph as g
from rai_amd.graph import F64Scalar, Tensor, cat


class Phi2Graph:
    def __init__(self, cfg, params, dtype):
        """cfg: object with the fields of phi2.rs:9-24; params: name -> Tensor (model dtype)."""
        self.cfg, self.p, self.dt = cfg, params, dtype
        self.kv = [None] * cfg.num_hidden_layers
        dim = cfg.rotary_dim
        theta = np.float32(cfg.rope_theta)
        inv = np.array([np.float32(1.0) / np.power(theta, np.float32(i) / np.float32(dim), dtype=np.float32)
                        for i in range(0, dim, 2)], dtype=np.float32)
        inv_freq = Tensor.from_array(inv.reshape(1, -1), "f32").to_dtype(dtype)
        t = Tensor.arange(0, cfg.max_position_embeddings, 1, "u32").to_dtype(dtype).reshape(
            (cfg.max_position_embeddings, 1))
        freqs = t.matmul(inv_freq)
        emb = cat([freqs, freqs], -1)
        self.sin, self.cos = emb.sin(), emb.cos()

    def clear_kv_cache(self):
        self.kv = [None] * self.cfg.num_hidden_layers

    def _rotary(self, xs, offset):
        dim = self.cfg.rotary_dim
        _, _, seq_len, headdim = xs.shape
        xs_rot = xs.narrow(3, 0, dim)
        xs_pass = xs.narrow(3, dim, headdim - dim)
        xs1, xs2 = xs_rot.narrow(3, 0, dim // 2), xs_rot.narrow(3, dim // 2, dim // 2)
        c = self.cos.narrow(0, offset, seq_len)
        s = self.sin.narrow(0, offset, seq_len)
        rotate_half = cat([-xs2, xs1], -1)
        xs_rot = xs_rot * c + rotate_half * s
        return cat([xs_rot, xs_pass], -1)

    def _linear(self, x, name):
        return g.linear(x, self.p[name + ".weight"], self.p.get(name + ".bias"))

    def _attention(self, l, xs, mask):
        cfg, dt = self.cfg, self.dt
        pre = f"model.layers.{l}.self_attn."
        b, s, _ = xs.shape
        nh, nkv, hd = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
        q, k = self._linear(xs, pre + "q_proj"), self._linear(xs, pre + "k_proj")
        if getattr(cfg, "qk_layernorm", False):   # phi2.rs:207-216: on the un-split projections
            q = g.layer_norm(q, self.p[pre + "q_layernorm.weight"], self.p[pre + "q_layernorm.bias"], cfg.layer_norm_eps)
            k = g.layer_norm(k, self.p[pre + "k_layernorm.weight"], self.p[pre + "k_layernorm.bias"], cfg.layer_norm_eps)
        q = q.reshape((b, s, nh, hd)).transpose(1, 2)
        k = k.reshape((b, s, nkv, hd)).transpose(1, 2)
        v = self._linear(xs, pre + "v_proj").reshape((b, s, nkv, hd)).transpose(1, 2)
        offset = 0 if self.kv[l] is None else self.kv[l][0].shape[2]
        q, k = self._rotary(q, offset), self._rotary(k, offset)
        if self.kv[l] is not None:
            k = cat([self.kv[l][0], k], 2)
            v = cat([self.kv[l][1], v], 2)
        self.kv[l] = (k, v)
        n_rep = nh // nkv
        if n_rep > 1:  # repeat_kv phi2.rs:190-200
            t = k.shape[2]
            k = k.unsqueeze(2).broadcast_to((b, nkv, n_rep, t, hd)).reshape((b, nh, t, hd))
            v = v.unsqueeze(2).broadcast_to((b, nkv, n_rep, t, hd)).reshape((b, nh, t, hd))
        scale = 1.0 / math.sqrt(hd)
        w = q.to_dtype("f32").matmul(k.to_dtype("f32").t() * scale)
        if mask is not None:
            m = mask.broadcast_to(w.shape)
            w = m.where_cond(w.full_like(float("-inf")), w)
        w = w.softmax(-1).to_dtype(dt)
        o = w.matmul(v).transpose(1, 2).reshape((b, s, nh * hd))
        return self._linear(o, pre + "dense")

    def _layer(self, l, xs, mask):
        pre = f"model.layers.{l}."
        ln = g.layer_norm(xs, self.p[pre + "input_layernorm.weight"], self.p[pre + "input_layernorm.bias"],
                          self.cfg.layer_norm_eps)
        attn = self._attention(l, ln, mask)
        h = self._linear(ln, pre + "mlp.fc1")
        h = {"gelu_new": h.new_gelu, "gelu": h.gelu, "silu": h.silu, "relu": h.relu}[self.cfg.hidden_act]()
        mlp = self._linear(h, pre + "mlp.fc2")
        return attn + mlp + xs

    def fwd(self, ids):
        """ids: u32 Tensor [B, S] -> logits Tensor [B, 1, vocab] of the last position (unevaluated)."""
        s = ids.shape[1]
        xs = g.embedding(ids, self.p["model.embed_tokens.weight"])
        mask = None
        if s > 1:  # get_mask phi2.rs:104-109: u8 [S, S], 1 above the diagonal
            mask = Tensor.from_array(np.triu(np.ones((s, s), np.uint8), 1), "u8")
        for l in range(self.cfg.num_hidden_layers):
            xs = self._layer(l, xs, mask)
        xs = g.layer_norm(xs, self.p["model.final_layernorm.weight"], self.p["model.final_layernorm.bias"],
                          self.cfg.layer_norm_eps)
        xs = xs.narrow(1, s - 1, 1)
        if self.cfg.tie_word_embeddings:
            return g.linear(xs, self.p["model.embed_tokens.weight"], None)
        return g.linear(xs, self.p["lm_head.weight"], self.p.get("lm_head.bias"))


class SeqGraph:
    """Qwen2 (qwen2.rs) and Gemma (gemma.rs): sequential pre-norm block, rotary embedding over the whole head, additive
    causal mask, scores and softmax in the model dtype, gated MLP.  Grouped-query configurations follow gemma.rs
    (kv projections of num_kv_heads * head_dim and repeat_kv, :167, :191-201), which qwen2.rs cannot express."""

    def __init__(self, cfg, params, dtype):
        """cfg: arch ("qwen2" | "gemma") + the fields of qwen2.rs:9-23 / gemma.rs:12-26; params: name -> Tensor."""
        self.cfg, self.p, self.dt = cfg, params, dtype
        self.kv = [None] * cfg.num_hidden_layers
        dim = cfg.head_dim
        # RotaryEmbedding::new qwen2.rs:40-58: f64 powf cast to f32, positions and outer product in the model dtype
        inv = np.array([np.float32(1.0) / np.float32(cfg.rope_theta ** (i / dim)) for i in range(0, dim, 2)], np.float32)
        inv_freq = Tensor.from_array(inv.reshape(1, -1), "f32").to_dtype(dtype)
        t = Tensor.arange(0, cfg.max_position_embeddings, 1, "u32").to_dtype(dtype).reshape(
            (cfg.max_position_embeddings, 1))
        freqs = t.matmul(inv_freq)
        freqs = cat([freqs, freqs], -1)
        self.sin, self.cos = freqs.sin(), freqs.cos()

    def clear_kv_cache(self):
        self.kv = [None] * self.cfg.num_hidden_layers

    @staticmethod
    def _rotate_half(xs):   # qwen2.rs:32-37
        d = xs.shape[-1]
        xs1, xs2 = xs.narrow(-1, 0, d // 2), xs.narrow(-1, d // 2, d - d // 2)
        return cat([-xs2, xs1], -1)

    def _rotary(self, q, k, offset):   # RotaryEmbedding::fwd qwen2.rs:60-71
        s = q.shape[2]
        cos = self.cos.narrow(0, offset, s).unsqueeze(0).unsqueeze(0)
        sin = self.sin.narrow(0, offset, s).unsqueeze(0).unsqueeze(0)
        return q * cos + self._rotate_half(q) * sin, k * cos + self._rotate_half(k) * sin

    def _norm(self, x, w):
        eps = self.cfg.rms_norm_eps
        if self.cfg.arch != "gemma":
            return g.rms_norm(x, w, eps)           # rai-nn RmsNorm (rms_norm.rs:18-22)
        # RmsNorm::fwd gemma.rs:42-54: f32 inside for 16-bit inputs, x / sqrt(mean(x^2) + eps), cast back, (w + 1)
        internal = "f32" if self.dt in ("bf16", "f16") else self.dt
        xi = x.to_dtype(internal)
        norm_x = xi.square().sum(-1, True) / F64Scalar(x.shape[-1])
        x_normed = xi / (norm_x + F64Scalar(eps)).sqrt()
        return x_normed.to_dtype(self.dt) * (w + F64Scalar(1.0))

    @staticmethod
    def _repeat_kv(xs, n_rep):   # gemma.rs:191-201
        if n_rep == 1:
            return xs
        b, nkv, t, hd = xs.shape
        return xs.unsqueeze(2).broadcast_to((b, nkv, n_rep, t, hd)).reshape((b, nkv * n_rep, t, hd))

    def _linear(self, x, name):
        return g.linear(x, self.p[name + ".weight"], self.p.get(name + ".bias"))

    def _attention(self, l, xs, mask, offset):   # Attention::fwd qwen2.rs:166-221 / gemma.rs:203-259
        cfg = self.cfg
        pre = f"model.layers.{l}.self_attn."
        b, s, _ = xs.shape
        nh, nkv, hd = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
        q = self._linear(xs, pre + "q_proj").reshape((b, s, nh, hd)).transpose(1, 2)
        k = self._linear(xs, pre + "k_proj").reshape((b, s, nkv, hd)).transpose(1, 2)
        v = self._linear(xs, pre + "v_proj").reshape((b, s, nkv, hd)).transpose(1, 2)
        q, k = self._rotary(q, k, offset)
        if self.kv[l] is not None:
            k = cat([self.kv[l][0], k], 2)
            v = cat([self.kv[l][1], v], 2)
        self.kv[l] = (k, v)
        k, v = self._repeat_kv(k, nh // nkv), self._repeat_kv(v, nh // nkv)
        w = q.matmul(k.transpose(2, 3)) * F64Scalar(1.0 / math.sqrt(hd))
        if mask is not None:
            w = w + mask
        o = w.softmax(-1).matmul(v)
        return self._linear(o.transpose(1, 2).reshape((b, s, nh * hd)), pre + "o_proj")

    def _layer(self, l, xs, mask, offset):   # DecoderLayer::fwd qwen2.rs:253-266 / gemma.rs:286-299
        pre = f"model.layers.{l}."
        h = self._attention(l, self._norm(xs, self.p[pre + "input_layernorm.weight"]), mask, offset)
        xs = h + xs
        y = self._norm(xs, self.p[pre + "post_attention_layernorm.weight"])
        gate = self._linear(y, pre + "mlp.gate_proj")
        lhs = {"gelu_new": gate.new_gelu, "gelu": gate.gelu, "silu": gate.silu, "relu": gate.relu}[self.cfg.hidden_act]()
        rhs = self._linear(y, pre + "mlp.up_proj")
        return xs + self._linear(lhs * rhs, pre + "mlp.down_proj")

    def _mask(self, b, tgt, offset):   # prepare_decoder_attention_mask qwen2.rs:306-336 / gemma.rs:341-362
        m = np.where(np.arange(tgt)[:, None] < np.arange(tgt)[None, :], np.float32(-np.inf), np.float32(0))
        mask = Tensor.from_array(m.astype(np.float32), "f32")
        if offset > 0:
            mask = cat([Tensor.zeros((tgt, offset), "f32"), mask], -1)
        return mask.broadcast_to((b, 1, tgt, tgt + offset)).to_dtype(self.dt)

    def fwd(self, ids):
        """ids: u32 Tensor [B, S] -> logits Tensor [B, 1, vocab] of the last position (unevaluated)."""
        cfg = self.cfg
        b, s = ids.shape
        offset = 0 if self.kv[0] is None else self.kv[0][0].shape[2]
        mask = None if s <= 1 else self._mask(b, s, offset)
        xs = g.embedding(ids, self.p["model.embed_tokens.weight"])
        if cfg.arch == "gemma":   # gemma.rs:379
            xs = xs * F64Scalar(math.sqrt(cfg.hidden_size))
        for l in range(cfg.num_hidden_layers):
            xs = self._layer(l, xs, mask, offset)
        xs = self._norm(xs.narrow(1, s - 1, 1), self.p["model.norm.weight"])
        head = self.p["model.embed_tokens.weight"] if cfg.arch == "gemma" else self.p["lm_head.weight"]
        return g.linear(xs, head, None)
