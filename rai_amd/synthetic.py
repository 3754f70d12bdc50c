"""Seeded synthetic weights and prompts for the decoder drivers.

Weights are N(0, std) for matrices and embeddings, zero biases, unit norm
weights, drawn per tensor from PCG64 seeded with (seed, crc32(name)) so any
subset of tensors can be regenerated independently (a CPU comparator can build
only the layers it times).  Values are returned in the storage form the C ABI
expects (bf16 as uint16 bit patterns).
"""
from __future__ import annotations

import zlib
from concurrent.futures import ThreadPoolExecutor

import numpy as np


def f32_to_bf16_bits(x):
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    r = (u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16)
    return r.astype(np.uint16)


def to_storage(a, dtype):
    if dtype == "bf16":
        return f32_to_bf16_bits(a).reshape(a.shape)
    if dtype == "f16":
        return a.astype(np.float16)
    if dtype == "f32":
        return np.ascontiguousarray(a, dtype=np.float32)
    raise ValueError(dtype)


def tensor(name, numel, seed=0, std=0.02):
    """float32 values of one named parameter (flat)."""
    if name.endswith("norm.weight"):
        return np.ones(numel, np.float32)
    if name.endswith(".bias"):
        return np.zeros(numel, np.float32)
    rng = np.random.Generator(np.random.PCG64([seed, zlib.crc32(name.encode())]))
    out = rng.standard_normal(numel, dtype=np.float32)
    out *= np.float32(std)
    return out


def load_random_params(decoder, seed=0, std=0.02, workers=8):
    """Generate and upload every parameter the decoder expects."""
    names = decoder.param_names()
    dt = decoder.dtype

    def make(item):
        name, numel = item
        return name, to_storage(tensor(name, numel, seed, std), dt)

    items = sorted(names.items(), key=lambda kv: -kv[1])
    with ThreadPoolExecutor(max_workers=workers) as ex:
        # bounded look-ahead keeps host memory to a few tensors at a time
        pending = []
        it = iter(items)
        for _ in range(workers):
            nxt = next(it, None)
            if nxt is not None:
                pending.append(ex.submit(make, nxt))
        while pending:
            name, arr = pending.pop(0).result()
            decoder.load_param(name, arr)
            nxt = next(it, None)
            if nxt is not None:
                pending.append(ex.submit(make, nxt))


def prompt(vocab_size, batch, length, seed=1):
    rng = np.random.Generator(np.random.PCG64(seed))
    return rng.integers(0, vocab_size, (batch, length)).astype(np.uint32)


class Phi2Shape:
    """The fields of the Phi-2 configuration (rai-models/src/llm/phi2.rs:9-24) that fix parameter and cache shapes."""

    def __init__(self, vocab_size=51200, hidden_size=2560, intermediate_size=10240, num_hidden_layers=32,
                 num_attention_heads=32, num_key_value_heads=None, hidden_act="gelu_new", max_position_embeddings=2048,
                 layer_norm_eps=1e-5, tie_word_embeddings=False, rope_theta=10000.0, partial_rotary_factor=0.4,
                 qk_layernorm=False):
        self.vocab_size, self.hidden_size, self.intermediate_size = vocab_size, hidden_size, intermediate_size
        self.num_hidden_layers, self.num_attention_heads = num_hidden_layers, num_attention_heads
        self.num_key_value_heads = num_key_value_heads or num_attention_heads
        self.hidden_act, self.max_position_embeddings = hidden_act, max_position_embeddings
        self.layer_norm_eps, self.tie_word_embeddings, self.rope_theta = layer_norm_eps, tie_word_embeddings, rope_theta
        self.partial_rotary_factor, self.qk_layernorm = partial_rotary_factor, qk_layernorm
        self.head_dim = hidden_size // num_attention_heads
        self.rotary_dim = int(partial_rotary_factor * self.head_dim)


def phi2_param_shapes(cfg):
    """Parameter name -> shape of a Phi-2 model, by the names the reference's modules give them
    (rai-models/src/llm/phi2.rs:307-313 with the naming rule of rai-core/src/nn.rs:183-205)."""
    h, i, v = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    kv = cfg.num_key_value_heads * cfg.head_dim
    out = {"model.embed_tokens.weight": (v, h)}
    for l in range(cfg.num_hidden_layers):
        p = f"model.layers.{l}."
        for name, rows in (("q_proj", h), ("k_proj", kv), ("v_proj", kv), ("dense", h)):
            out[p + f"self_attn.{name}.weight"] = (rows, h)
            out[p + f"self_attn.{name}.bias"] = (rows,)
        out[p + "mlp.fc1.weight"], out[p + "mlp.fc1.bias"] = (i, h), (i,)
        out[p + "mlp.fc2.weight"], out[p + "mlp.fc2.bias"] = (h, i), (h,)
        out[p + "input_layernorm.weight"], out[p + "input_layernorm.bias"] = (h,), (h,)
    out["model.final_layernorm.weight"], out["model.final_layernorm.bias"] = (h,), (h,)
    if not cfg.tie_word_embeddings:
        out["lm_head.weight"], out["lm_head.bias"] = (v, h), (v,)
    return out
