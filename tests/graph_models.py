"""Phi-2 written against the lazy `Tensor` API, node for node as
rai-models/src/llm/phi2.rs builds it (RotaryEmbedding :44-78, masked_fill :111-117,
Attention::fwd :202-264, MLP :99-101, DecoderLayer::fwd :293-299, Model::fwd :334-347).

Nothing here computes: every call records graph nodes; `eval()` / `as_storage()`
runs them on the Hip device through the dispatcher.  This is the reference's own
execution scheme (one primitive per node, KV cache by concatenation) and serves
as the functional drop-in path; the fused decoder drivers are the fast path.
"""
from __future__ import annotations

import math

import numpy as np

from rai_amd import graph as g
from rai_amd.graph import Tensor, cat


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
