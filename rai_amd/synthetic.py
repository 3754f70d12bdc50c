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
