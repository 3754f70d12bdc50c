#!/usr/bin/env python3
"""Headline benchmark: Phi-2-architecture bf16 greedy decode / prefill on one MI355X.

Workload (one "step"): the full 32-layer Phi-2-architecture model, random-init
N(0, 0.02) bf16 weights, batch 1, KV cache, a 512-token uniform-random prompt
(prefill) followed by 128 greedy tokens (decode), all on the device through the
C ABI of librai_hip.so.  Weights, prompt and KV cache are resident in HBM when
the timed region starts.

Prints ONE JSON line.  `value` is decode tokens/s; prefill tokens/s, the
roofline of the dominant kernel (the weight-streaming decode kernel, HBM-bound)
and a CPU baseline (the NumPy oracle restating rai's Cpu path, timed on this
host on a bounded sample) ride along in the same object.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PHI2 = dict(vocab_size=51200, hidden_size=2560, intermediate_size=10240, num_hidden_layers=32,
            num_attention_heads=32, rotary_dim=32, max_position_embeddings=2048, hidden_act="gelu_new",
            rope_theta=10000.0, norm_eps=1e-5)
PROMPT, NEW = 512, 128
# HBM traffic of the dominant kernel relative to its algorithmic bytes, from rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE (two runs), each scaled by what the same counter reads for a plain 256 MiB copy kernel
# (profiles/phi2_decode_step_hbm_traffic_pmc.md): 5.255 GB fetched + 4.7 MB written against 5.224 GB.
TRAFFIC_OVER_ALGORITHMIC = 1.0069
HBM_PEAK_GBS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0


def decode_bytes_per_token(cfg, ctx):
    """Algorithmic HBM bytes of one decode token at context length ctx (bf16):
    every layer's weights and biases once, the lm_head, one embedding row and the
    K/V rows of the cached context."""
    h, i, v, l = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"], cfg["num_hidden_layers"]
    layer = 4 * h * h + 4 * h + 2 * h * i + i + h + 2 * h      # q,k,v,dense + biases, fc1, fc2 + biases, LayerNorm
    head = v * h + v + 2 * h
    kv = l * 2 * h * ctx
    return 2.0 * (l * layer + head + h + kv)


def prefill_flops(cfg, s):
    h, i, v, l = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"], cfg["num_hidden_layers"]
    nh = cfg["num_attention_heads"]
    hd = h // nh
    lin = 2.0 * (4 * h * h + 2 * h * i) * l * s
    attn = l * 4.0 * nh * s * s * hd
    return lin + attn + 2.0 * v * h


def check_first_tokens(tokens):
    """The greedy tokens of this workload against the CPU oracle's (tests/golden/phi2_bench_first_tokens.json, written
    by tests/golden/make_phi2_bench_tokens.py from the oracle alone; tests/test_gpu_config2_phi2_full.py checks the
    fixture itself).  A token may differ only where the oracle's own two best logits are a near tie at the bf16
    tolerance; the sequences may part ways after that.  Anything else ends the run: a fast wrong answer is no result."""
    path = os.path.join(ROOT, "tests", "golden", "phi2_bench_first_tokens.json")
    with open(path) as f:
        gold = json.load(f)
    for s, want in enumerate(gold["tokens"]):
        if int(tokens[s]) != want:
            if gold["top2_gap"][s] <= 2e-2 * gold["max_abs_logit"][s]:
                return f"identical for {s} tokens, then a near tie of the oracle's logits (gap {gold['top2_gap'][s]:.4f})"
            sys.exit(f"bench.py: greedy token {s} is {int(tokens[s])}, the CPU oracle says {want} "
                     f"(top-2 gap {gold['top2_gap'][s]:.4f}): refusing to report a throughput")
    return f"identical for all {len(gold['tokens'])} checked tokens"


def cpu_baseline(steps_decode=2, layers=2):
    """The oracle (a NumPy port of rai's Cpu evaluation, bf16 storage with f32
    math) timed on this host on a bounded sample: the first `layers` decoder
    layers plus embedding and lm_head, 512-token prefill, then `steps_decode`
    decode tokens; the per-layer times are scaled to 32 layers."""
    from oracle import phi2
    # threads = physical cores of this host, capped by the share the environment grants (OMP_NUM_THREADS); the BLAS
    # pool NumPy's matmul runs on is set to that count and the count it reports back is what goes into the line
    import psutil
    from threadpoolctl import threadpool_info, threadpool_limits
    want = min(psutil.cpu_count(logical=False) or os.cpu_count() or 1,
               int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)))
    threadpool_limits(limits=want)
    pools = [p["num_threads"] for p in threadpool_info() if p.get("user_api") == "blas"]
    threads = max(pools) if pools else want
    cfg = phi2.Config(num_hidden_layers=layers)
    params = phi2.random_params(cfg, "bf16", seed=0)
    model = phi2.Model(cfg, params, "bf16")
    ids = np.random.Generator(np.random.PCG64(1)).integers(0, cfg.vocab_size, (1, PROMPT)).astype(np.uint32)

    def timed_layers(x, mask):
        t0 = time.perf_counter()
        for l in range(layers):
            x = model.layer(l, x, mask)
        return x, time.perf_counter() - t0

    from oracle import nn as onn, ops as oo
    t0 = time.perf_counter()
    x = onn.embedding(ids, params["model.embed_tokens.weight"])
    t_embed = time.perf_counter() - t0
    x, t_pre_layers = timed_layers(x, phi2.get_mask(PROMPT))

    def head(x):
        t0 = time.perf_counter()
        y = onn.layer_norm(x, params["model.final_layernorm.weight"], params["model.final_layernorm.bias"], 1e-5, "bf16")
        y = oo.narrow(y, 1, y.shape[1] - 1, 1)
        logits = onn.linear(y, params["lm_head.weight"], params["lm_head.bias"], "bf16")
        tok = oo.argmax(logits[:, 0, :], -1)
        return tok, time.perf_counter() - t0

    tok, t_head = head(x)
    prefill_s = t_embed + t_pre_layers * (32.0 / layers) + t_head
    dec_layers, dec_head = 0.0, 0.0
    for _ in range(steps_decode):
        x = onn.embedding(tok.reshape(1, 1), params["model.embed_tokens.weight"])
        x, tl = timed_layers(x, None)
        tok, th = head(x)
        dec_layers += tl
        dec_head += th
    decode_s_per_tok = (dec_layers * (32.0 / layers) + dec_head) / steps_decode
    return {
        "value": round(1.0 / decode_s_per_tok, 4),
        "unit": "tokens/s (decode)",
        "prefill_tokens_per_s": round(PROMPT / prefill_s, 2),
        "cores": threads,
        "kind": "port",
        "sample": f"NumPy oracle of rai's Cpu path (bf16 storage, f32 math): {layers} of 32 layers + embedding + "
                  f"lm_head timed, 512-token prefill then {steps_decode} decode tokens, layer time scaled x{32 // layers}",
    }


# ------------------------------------------------------------------------------------------------
# Secondary workloads (not the headline line): the other configurations of the same hot path.
QWEN2_15B = dict(vocab_size=151936, hidden_size=1536, intermediate_size=8960, num_hidden_layers=28,
                 num_attention_heads=12, num_key_value_heads=2, head_dim=128, rotary_dim=128,
                 max_position_embeddings=2048, hidden_act="silu", rope_theta=1e6, norm_eps=1e-6)
GEMMA_2B = dict(vocab_size=256000, hidden_size=2048, intermediate_size=16384, num_hidden_layers=18,
                num_attention_heads=8, num_key_value_heads=1, head_dim=256, rotary_dim=256,
                max_position_embeddings=4096, hidden_act="gelu", rope_theta=10000.0, norm_eps=1e-6,
                tie_word_embeddings=True)


def _line(metric, value, unit, steps, warmup, ms_per_step, workload, extra):
    out = {"metric": metric, "value": round(value, 2), "unit": unit, "n_gpus": 1, "steps": steps, "warmup": warmup,
           "ms_per_step": round(ms_per_step, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
           "dtype": "bf16", "data": "synthetic", "config": {"workload": workload}}
    out.update(extra)
    print(json.dumps(out), flush=True)


def run_qwen2_prefill(args):
    """Qwen2-1.5B architecture, bf16, batched prefill 16 x 1024 with causal mask."""
    from rai_amd import synthetic
    from rai_amd.hip import sync
    from rai_amd.models import Decoder
    B, S = 16, 1024
    cfg = QWEN2_15B
    dec = Decoder("qwen2", "bf16", max_batch=B, max_context=S, **cfg)
    synthetic.load_random_params(dec, seed=0)
    ids = synthetic.prompt(cfg["vocab_size"], B, S, seed=1)
    times = []
    for it in range(args.warmup + args.steps):
        dec.clear_kv_cache()
        sync()
        t0 = time.perf_counter()
        _, tok = dec.forward(ids, want_logits=False)   # returns after the tokens are on the host
        dt = time.perf_counter() - t0
        if it >= args.warmup:
            times.append(dt)
    t = float(np.mean(times))
    h, i, v, l = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"], cfg["num_hidden_layers"]
    qd, kd = cfg["num_attention_heads"] * cfg["head_dim"], cfg["num_key_value_heads"] * cfg["head_dim"]
    lin = 2.0 * (h * (qd + 2 * kd) + qd * h + 3 * h * i) * l * B * S
    attn = l * 4.0 * cfg["num_attention_heads"] * B * S * S * cfg["head_dim"]
    flops = lin + attn + 2.0 * B * v * h
    _line("Qwen2-1.5B bf16 batched prefill tok/s on 1 MI355X", B * S / t, "tokens/s", args.steps, args.warmup, t * 1e3,
          "Qwen2-1.5B architecture 28L bf16, prefill batch 16 x 1024 tokens, causal, GQA 12/2 (random-init N(0,0.02))",
          {"prefill_ms": round(t * 1e3, 3), "prefill_tflops": round(flops / t / 1e12, 1),
           "prefill_frac_of_bf16_mfma_peak": round(flops / t / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
           "first_tokens": [int(x) for x in tok[:8]]})
    dec.close()


def run_gemma_decode(args):
    """Gemma-2B architecture, bf16, greedy decode at batch 32 on a 2048-token context per sequence, 64 steps."""
    from rai_amd import synthetic
    from rai_amd.models import Decoder
    B, CTX, NEWT = 32, 2048, 64
    cfg = GEMMA_2B
    dec = Decoder("gemma", "bf16", max_batch=B, max_context=CTX + NEWT, **cfg)
    synthetic.load_random_params(dec, seed=0)
    prompt = synthetic.prompt(cfg["vocab_size"], B, CTX, seed=1)
    pre, dcd = [], []
    wall0 = time.perf_counter()
    for it in range(args.warmup + args.steps):
        if it == args.warmup:
            wall0 = time.perf_counter()
        toks, p, d = dec.generate(prompt, NEWT)
        if it >= args.warmup:
            pre.append(p)
            dcd.append(d)
    wall = time.perf_counter() - wall0
    d_ms = float(np.mean(dcd)) / (NEWT - 1)
    h, i, v, l = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"], cfg["num_hidden_layers"]
    qd, kd = cfg["num_attention_heads"] * cfg["head_dim"], cfg["num_key_value_heads"] * cfg["head_dim"]
    weights = 2.0 * (l * (h * (qd + 2 * kd) + qd * h + 3 * h * i + 2 * h) + v * h + h)
    kv = 2.0 * l * B * 2 * kd * (CTX + NEWT / 2.0)
    step_bytes = weights + kv
    _line("Gemma-2B bf16 batch-32 decode tok/s on 1 MI355X", B / (d_ms / 1e3), "tokens/s", args.steps, args.warmup,
          wall * 1e3 / max(args.steps, 1),
          "Gemma-2B architecture 18L bf16, greedy decode batch 32, 2048-token context per sequence, 64 steps, "
          "MQA 8/1 x 256, tied 256000-way head (random-init N(0,0.02))",
          {"decode_ms_per_step": round(d_ms, 4), "decode_step_bytes": int(step_bytes),
           "decode_frac_of_hbm_roofline": round(step_bytes / (d_ms / 1e3) / 1e9 / HBM_PEAK_GBS, 4),
           "prefill_tokens_per_s": round(B * CTX / (float(np.mean(pre)) / 1e3), 1),
           "first_tokens": [int(x) for x in toks[0, :8]]})
    dec.close()


def run_ops(args):
    """Primitive sweep, bf16 and f32.  Every op is launched through the C ABI into an output allocated beforehand,
    with the tensor descriptors built once, so the timed loop holds launches only: `loop_us` is the hipEvent time of
    a back-to-back loop divided by its length (launch rate or kernel time, whichever is longer), `single_us` one
    launch between two events.  The kernels' own durations are in the rocprofv3 kernel trace of this same command
    (profiles/op_sweep_kernel_trace.md)."""
    import ctypes as C

    from rai_amd import _lib, ops
    from rai_amd._lib import REDUCE, UNARY  # noqa: F401
    from rai_amd.hip import HipTensor, sync
    _lib.call("rai_hip_init", 0)
    lib = _lib.load()
    rng = np.random.default_rng(0)

    def rnd(shape, dt, scale=1.0):
        a = rng.standard_normal(shape, dtype=np.float32) * np.float32(scale)
        if dt == "bf16":
            return HipTensor.from_storage((a.view(np.uint32) >> 16).astype(np.uint16), "bf16")
        return HipTensor.from_storage(a, "f32")

    def launcher(name, *args):
        """A zero-argument callable that performs exactly one C-ABI call with everything prepared."""
        fn = getattr(lib, name)
        keep = [a.desc() if isinstance(a, HipTensor) else a for a in args]
        cargs = [C.byref(k) if isinstance(k, _lib.TensorDesc) else k for k in keep]

        def go():
            st = fn(*cargs)
            if st != 0:
                _lib.check(st)
        go.keep = (keep, args)
        return go

    def timed(fn, iters):
        t = C.c_void_p()
        _lib.call("rai_hip_timer_create", 0, C.byref(t))
        for _ in range(3):
            fn()
        _lib.call("rai_hip_timer_start", t)
        for _ in range(iters):
            fn()
        _lib.call("rai_hip_timer_stop", t)
        ms = C.c_float()
        _lib.call("rai_hip_timer_elapsed_ms", t, C.byref(ms))
        loop_us = ms.value * 1e3 / iters
        sync()
        _lib.call("rai_hip_timer_start", t)
        fn()
        _lib.call("rai_hip_timer_stop", t)
        _lib.call("rai_hip_timer_elapsed_ms", t, C.byref(ms))
        _lib.call("rai_hip_timer_destroy", t)
        return loop_us, ms.value * 1e3

    rows = []

    def hbm(op, dt, by, fn, iters=100):
        lu, su = timed(fn, iters)
        rows.append(dict(op=op, dtype=dt, loop_us=lu, single_us=su, bound="hbm", achieved=by / lu / 1e3, unit="GB/s",
                         frac=by / lu / 1e3 / HBM_PEAK_GBS, bytes=int(by)))

    for dt, es in (("bf16", 2), ("f32", 4)):
        a, b = rnd((4096, 2560), dt), rnd((2560, 10240), dt)
        out = HipTensor.empty((4096, 10240), dt)
        fl = 2.0 * 4096 * 2560 * 10240
        peak = MFMA_BF16_PEAK_TFLOPS if dt == "bf16" else 157.3
        lu, su = timed(launcher("rai_hip_matmul", 0, a, b, out), 10)
        rows.append(dict(op="matmul [4096,2560]x[2560,10240]", dtype=dt, loop_us=lu, single_us=su, bound="mfma",
                         achieved=fl / lu / 1e6, unit="TFLOP/s", frac=fl / lu / 1e6 / peak))
        w = rnd((10240, 2560), dt)
        lu, su = timed(launcher("rai_hip_linear", 0, a, w, None, -1, None, out), 10)
        rows.append(dict(op="linear x[4096,2560] . W[10240,2560]^T", dtype=dt, loop_us=lu, single_us=su, bound="mfma",
                         achieved=fl / lu / 1e6, unit="TFLOP/s", frac=fl / lu / 1e6 / peak))
        del a, b, w, out
        x = rnd((32, 128, 2048), dt, 3.0)
        out = HipTensor.empty(x.shape, dt)
        hbm("softmax [32,128,2048]", dt, 2.0 * x.numel() * es, launcher("rai_hip_softmax", 0, x, 2, out))
        x = rnd((4096, 2560), dt)
        out = HipTensor.empty(x.shape, dt)
        w1, b1 = rnd((2560,), dt), rnd((2560,), dt)
        by = 2.0 * x.numel() * es
        hbm("layer_norm [4096,2560]", dt, by, launcher("rai_hip_layer_norm", 0, x, w1, b1, 1e-5, out))
        hbm("rms_norm [4096,2560]", dt, by, launcher("rai_hip_rms_norm", 0, x, w1, 1e-6, 0, out))
        x = rnd((1, 32, 2048, 80), dt)
        out = HipTensor.empty(x.shape, dt)
        cos, sin = ops.rope_tables(2048, 32, 10000.0, dt)
        hbm("rope [1,32,2048,80] rot 32", dt, 2.0 * x.numel() * es, launcher("rai_hip_rope", 0, x, cos, sin, 32, 0, out))
        table = rnd((51200, 2560), dt)
        ids = HipTensor.from_storage(rng.integers(0, 51200, 4096).astype(np.uint32), "u32")
        out = HipTensor.empty((4096, 2560), dt)
        hbm("index_select 4096 of [51200,2560]", dt, 2.0 * 4096 * 2560 * es + 4096 * 4,
            launcher("rai_hip_index_select", 0, table, ids, 0, out))
        # the gradient of that embedding lookup: cotangent rows added into the table at the ids
        ct = rnd((4096, 2560), dt)
        out = HipTensor.empty(table.shape, dt)
        hbm("index_add 4096 rows into [51200,2560]", dt, (2.0 * 51200 * 2560 + 4096 * 2560) * es,
            launcher("rai_hip_index_add", 0, table, ids, ct, 0, out), 20)
        del table, ct, out
        x = rnd((64, 51200), dt)
        out = HipTensor.empty((64,), "u32")
        hbm("argmax [64,51200]", dt, 1.0 * x.numel() * es, launcher("rai_hip_argmax", 0, x, 1, 0, out))
        hbm("argmax_static [64,51200]", dt, 1.0 * x.numel() * es, launcher("rai_hip_argmax_static", 0, x, 1, 0, out))
    sync()
    for r in rows:
        r.update(loop_us=round(r["loop_us"], 2), single_us=round(r["single_us"], 2), achieved=round(r["achieved"], 1),
                 frac=round(r["frac"], 4))
    mm = rows[1]
    _line("bf16 linear [4096,2560]x[2560,10240] TFLOP/s on 1 MI355X", mm["achieved"], "TFLOP/s", 10, 3, mm["loop_us"] / 1e3,
          "primitive sweep, bf16 and f32: matmul / linear, softmax, LayerNorm, RMSNorm, RoPE, index_select, argmax",
          {"ops": rows})


def run_gemm_tiles(args):
    """The bf16 tile GEMM on the Phi-2 prefill shapes (and the op-sweep shape), every tile shape forced in turn
    through RAI_HIP_GEMM_TILE, Linear with bias and gelu_new as the q|k|v|fc1 product has them: shows what tile
    quantisation at M = 512 costs and that no tile shape escapes it."""
    import ctypes as C

    from rai_amd import _lib
    from rai_amd._lib import UNARY
    from rai_amd.hip import HipTensor, sync
    _lib.call("rai_hip_init", 0)
    lib = _lib.load()
    rng = np.random.default_rng(0)

    def rnd(shape):
        a = rng.standard_normal(shape, dtype=np.float32)
        return HipTensor.from_storage((a.view(np.uint32) >> 16).astype(np.uint16), "bf16")

    shapes = [(512, 17920, 2560), (512, 10240, 2560), (512, 7680, 2560), (512, 2560, 12800), (4096, 10240, 2560)]
    tiles = ["128x128", "128x128k64", "256x128", "256x192", "256x256", "256x256x8w", "256x256x8wk64", "streamk", "streamk64", None]
    rows = []
    for m, n, k in shapes:
        x, b, out = rnd((m, k)), rnd((n,)), HipTensor.empty((m, n), "bf16")
        # "cold": the launches rotate over enough copies of the weight (> 600 MB together) that none is still in the
        # 256 MB memory-side cache when its turn comes, as inside a model; "warm": one weight, resident after warm-up
        w0 = rnd((n, k))
        copies = [w0] + ([rnd((n, k)) for _ in range(-(-600_000_000 // (2 * n * k)) - 1)] if args.cold else [])
        dx, db, do = x.desc(), b.desc(), out.desc()
        dws = [c.desc() for c in copies]
        for tile in tiles:
            if tile is None:
                os.environ.pop("RAI_HIP_GEMM_TILE", None)
            else:
                os.environ["RAI_HIP_GEMM_TILE"] = tile

            turn = [0]

            def go():
                dw = dws[turn[0] % len(dws)]
                turn[0] += 1
                _lib.check(lib.rai_hip_linear(0, C.byref(dx), C.byref(dw), C.byref(db), UNARY["new_gelu"], None, C.byref(do)))
            if tile is not None and lib.rai_hip_linear(0, C.byref(dx), C.byref(dws[0]), C.byref(db), UNARY["new_gelu"], None,
                                                        C.byref(do)) != 0:
                continue        # this form does not apply to the shape (stream-K, K tiles of 64 with K split)
            t = C.c_void_p()
            _lib.call("rai_hip_timer_create", 0, C.byref(t))
            for _ in range(10):
                go()
            _lib.call("rai_hip_timer_start", t)
            for _ in range(50):
                go()
            _lib.call("rai_hip_timer_stop", t)
            ms = C.c_float()
            _lib.call("rai_hip_timer_elapsed_ms", t, C.byref(ms))
            _lib.call("rai_hip_timer_destroy", t)
            us = ms.value * 1e3 / 50
            rows.append({"shape": f"{m}x{n}x{k}", "tile": tile or "auto", "us": round(us, 1),
                         "tflops": round(2.0 * m * n * k / us / 1e6, 1)})
    os.environ.pop("RAI_HIP_GEMM_TILE", None)
    sync()
    best = max(r["tflops"] for r in rows if r["shape"] == "512x17920x2560")
    _line("bf16 Linear 512x17920x2560 (+bias, gelu_new) TFLOP/s on 1 MI355X", best, "TFLOP/s", 50, 10, 0.0,
          "tile GEMM, every tile shape forced in turn on the Phi-2 prefill shapes",
          {"weights": "cold (rotating copies)" if args.cold else "warm (one copy)", "tiles": rows})


def run_peaks(args):
    """What this GPU sustains with no workload around the loop (rai_hip_measure_peak, include/rai_hip_peaks.h): matrix
    pipes alone and with LDS fragment reads beside them, LDS reads alone, a plain 1 GiB read and copy, and 64 KB tile
    staging global -> LDS by every CU at once, both ways.  The roofline fractions elsewhere are against the published
    peaks; these are the ceilings the kernels actually meet."""
    from rai_amd import _lib
    from rai_amd.hip import measure_peak
    _lib.call("rai_hip_init", 0)
    launches = max(10, args.steps)
    out = {}
    gib = 1 << 30
    for label, kind, nbytes in (("mfma_bf16", "mfma_bf16", 0), ("mfma_bf16_lds", "mfma_bf16_lds", 0), ("lds_read", "lds_read", 0),
                                ("hbm_read", "hbm_read", gib), ("hbm_copy", "hbm_copy", gib),
                                ("stage_dma_2MiB", "stage_dma", 2 << 20), ("stage_vgpr_2MiB", "stage_vgpr", 2 << 20),
                                ("stage_dma_32MiB", "stage_dma", 32 << 20), ("stage_vgpr_32MiB", "stage_vgpr", 32 << 20),
                                ("gemm_loop_2MiB", "gemm_loop", 2 << 20), ("gemm_loop_32MiB", "gemm_loop", 32 << 20),
                                ("gemm_loop_1GiB", "gemm_loop", 1 << 30)):
        for _ in range(max(0, args.warmup)):
            measure_peak(kind, nbytes, 1)
        sec, work = measure_peak(kind, nbytes, launches)
        rate = work / sec
        if kind.startswith("mfma") or kind == "gemm_loop":
            out[label] = {"TFLOP/s": round(rate / 1e12, 1), "frac_of_2.5_PFLOP/s": round(rate / 2.5e15, 3), "us_per_launch": round(sec * 1e6, 1)}
        elif kind == "hbm_copy":
            out[label] = {"GB/s_read_plus_written": round(2 * rate / 1e9, 1), "frac_of_8_TB/s": round(2 * rate / 8e12, 3),
                         "us_per_launch": round(sec * 1e6, 1)}
        elif kind == "hbm_read":
            out[label] = {"GB/s": round(rate / 1e9, 1), "frac_of_8_TB/s": round(rate / 8e12, 3), "us_per_launch": round(sec * 1e6, 1)}
        else:
            out[label] = {"GB/s_per_CU": round(rate / 1e9 / 256, 1), "GB/s": round(rate / 1e9, 1), "us_per_launch": round(sec * 1e6, 1)}
    mf = out["mfma_bf16"]
    _line("bf16 MFMA ceiling measured on 1 MI355X (matrix pipes alone)", mf["TFLOP/s"], "TFLOP/s", launches, args.warmup,
          mf["us_per_launch"] / 1e3, "ceiling loops of rai_hip_measure_peak: no model, no tensors", {"peaks": out})


def run_phi2_graph(args, n_new=16):
    """The drop-in path: Phi-2 recorded node for node through the lazy-graph API the way rai-models/src/llm/phi2.rs
    builds it (tests/graph_models.py, KV cache by concatenation) and evaluated by the C++ evaluator with its
    composition and elementwise passes.  Greedy decode, batch 1, 512-token prompt; the time per token includes
    recording the graph from Python (ctypes), which a Rust front end would do far faster."""
    from rai_amd import graph as g, synthetic
    from rai_amd.graph import Tensor
    from tests.graph_models import Phi2Graph     # the stand-in for the reference's unchanged model file
    cfg = synthetic.Phi2Shape(num_hidden_layers=args.layers)
    params = {}
    for name, shape in synthetic.phi2_param_shapes(cfg).items():
        a = synthetic.to_storage(synthetic.tensor(name, int(np.prod(shape)), 0, 0.02), "bf16").reshape(shape)
        params[name] = Tensor.from_array(a, "bf16")
    g.eval_all(list(params.values()))
    model = Phi2Graph(cfg, params, "bf16")
    prompt = synthetic.prompt(cfg.vocab_size, 1, PROMPT, seed=1)
    out = {}
    for label, compose in (("composed", True), ("node_by_node", False)):
        g.set_compose(compose)
        model.clear_kv_cache()
        ids = prompt
        toks, t_rec, t_eval, launches, nodes, t_plan, t_run = [], 0.0, 0.0, 0, 0, 0.0, 0.0
        steps = n_new if compose else min(n_new, 4)
        for step in range(steps + 1):
            g.stats(reset=True)
            t0 = time.perf_counter()
            nxt = model.fwd(Tensor.from_array(ids, "u32")).argmax(-1)
            t1 = time.perf_counter()
            tok = nxt.as_storage().reshape(-1)
            t2 = time.perf_counter()
            st = g.stats()
            if step == 0:
                out[f"{label}_prefill_ms"] = round((t2 - t0) * 1e3, 2)
            else:
                t_rec += t1 - t0
                t_eval += t2 - t1
                launches += st["kernel_launches"]
                t_plan += st["plan_ms"]
                t_run += st["run_ms"]
                nodes += st["nodes_evaluated"] + st["fused_nodes"] + st["composed_nodes"]
            toks.append(int(tok[0]))
            ids = tok.reshape(1, 1).astype(np.uint32)
        out[f"{label}_decode_tokens_per_s"] = round(steps / (t_rec + t_eval), 2)
        out[f"{label}_record_ms_per_token"] = round(t_rec / steps * 1e3, 3)
        out[f"{label}_eval_ms_per_token"] = round(t_eval / steps * 1e3, 3)
        out[f"{label}_launches_per_token"] = round(launches / steps, 1)
        out[f"{label}_host_plan_ms_per_token"] = round(t_plan / steps, 3)
        out[f"{label}_host_run_ms_per_token"] = round(t_run / steps, 3)
        out[f"{label}_first_tokens"] = toks[:8]
    g.set_compose(True)
    out["recorded_nodes_per_token"] = round(nodes / steps, 1)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--pmc-calibrate", action="store_true",
                    help="also run a plain device copy of 256 MiB three times (k_copy): the known-size reference "
                         "for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE readings")
    ap.add_argument("--layers", type=int, default=PHI2["num_hidden_layers"],
                    help="debug only: fewer layers (the JSON line then says so and is not the headline workload)")
    ap.add_argument("--graph-tokens", type=int, default=16,
                    help="tokens decoded through the lazy-graph path for the graph_decode_* fields (0: skip)")
    ap.add_argument("--cold", action="store_true",
                    help="gemm-tiles: rotate over weight copies so every launch reads its weight from HBM, as in a model")
    ap.add_argument("--workload", default="phi2-decode", choices=["phi2-decode", "qwen2-prefill", "gemma-decode", "ops", "gemm-tiles", "peaks"],
                    help="phi2-decode is the headline line; the others are the remaining configurations of the path")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU; --gpus must be 1 (multi-GPU sharding is a design note only)")
    if args.workload == "qwen2-prefill":
        return run_qwen2_prefill(args)
    if args.workload == "gemma-decode":
        return run_gemma_decode(args)
    if args.workload == "ops":
        return run_ops(args)
    if args.workload == "gemm-tiles":
        return run_gemm_tiles(args)
    if args.workload == "peaks":
        return run_peaks(args)

    from rai_amd import synthetic
    from rai_amd.hip import sync
    from rai_amd.models import Decoder

    cfg = dict(PHI2)
    cfg["num_hidden_layers"] = args.layers
    t0 = time.perf_counter()
    dec = Decoder("phi2", "bf16", max_batch=1, max_context=PROMPT + NEW, **cfg)
    synthetic.load_random_params(dec, seed=0)
    sync()
    load_s = time.perf_counter() - t0
    prompt = synthetic.prompt(cfg["vocab_size"], 1, PROMPT, seed=1)

    for _ in range(args.warmup):
        dec.generate(prompt, NEW)
    sync()
    wall0 = time.perf_counter()
    pre_ms, dec_ms, toks = [], [], None
    for _ in range(args.steps):
        toks, p, d = dec.generate(prompt, NEW)
        pre_ms.append(p)
        dec_ms.append(d)
    sync()
    wall = time.perf_counter() - wall0
    pre = float(np.mean(pre_ms))
    dcd = float(np.mean(dec_ms))
    decode_tok_s = (NEW - 1) / (dcd / 1e3)     # the prefill produces token 0; NEW-1 single-token steps follow
    prefill_tok_s = PROMPT / (pre / 1e3)
    # the same loop with the example's token choice (repeat penalty 1.10 over the last 64 tokens, last maximum)
    dec.generate_sampled(prompt, NEW)
    _, _, _, samp_ms = dec.generate_sampled(prompt, NEW)

    # dominant kernel: the persistent per-token kernel that runs all layers of a decode step (weights, biases,
    # norm parameters and the KV cache of the current context once per launch), timed live with one hipEvent
    # pair per launch on the library's stream, at the context length the generate call ended with
    us, bytes_per_launch = dec.time_decode_step(sweeps=20)
    achieved = bytes_per_launch / (us * 1e-6) / 1e9
    gemv_us, gemv_bytes = dec.time_decode_linear(sweeps=10)   # the launch-per-primitive path's streaming kernels
    mean_ctx = PROMPT + (NEW - 1) / 2.0 + 1
    step_bytes = decode_bytes_per_token(cfg, mean_ctx)
    out = {
        "metric": "Phi-2 bf16 decode tok/s on 1 MI355X",
        "value": round(decode_tok_s, 2),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall * 1e3 / args.steps, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"Phi-2 architecture {args.layers}L bf16, batch 1, KV cache, {PROMPT}-token prompt + "
                               f"{NEW} greedy tokens (random-init N(0,0.02), uniform-random prompt)",
                   "prompt_len": PROMPT, "new_tokens": NEW, "batch": 1},
        "decode_ms_per_token": round(dcd / (NEW - 1), 4),
        "decode_frac_of_hbm_roofline": round(step_bytes / (dcd / 1e3 / (NEW - 1)) / 1e9 / HBM_PEAK_GBS, 4),
        "prefill_tokens_per_s": round(prefill_tok_s, 1),
        "prefill_ms": round(pre, 3),
        "prefill_frac_of_bf16_mfma_peak": round(prefill_flops(cfg, PROMPT) / (pre / 1e3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
        "weights_load_s": round(load_s, 1),
        "first_tokens": [int(t) for t in toks[0, :17]],
        "sampled_decode_tokens_per_s": round((NEW - 1) / (samp_ms / 1e3), 2),
        "roofline": {
            "kernel": "k_phi2_decode_step (persistent kernel: all 32 layers of one decode step, blocks exchange "
                      "tagged packets instead of grid barriers, weight ring prefetched across segments, "
                      "attention inputs published ahead of the fc1 stream)",
            "bound": "hbm",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            "traffic": int(bytes_per_launch * TRAFFIC_OVER_ALGORITHMIC),
            "us_per_launch": round(us, 3),
            "bytes_per_launch": int(bytes_per_launch),
        },
        "decode_gemv_kernels": {"us_per_launch": round(gemv_us, 3), "bytes_per_launch": int(gemv_bytes),
                                "GB_per_s": round(gemv_bytes / (gemv_us * 1e-6) / 1e9, 1)},
    }
    dec.close()
    if args.layers == PHI2["num_hidden_layers"]:
        out["tokens_match_oracle"] = check_first_tokens(toks[0])
    if args.pmc_calibrate:
        import ctypes as C

        from rai_amd import _lib, ops
        from rai_amd.hip import HipTensor
        src = ops.full(1.0, (64 * 1024 * 1024,), "f32")
        dst = HipTensor.empty((64 * 1024 * 1024,), "f32")
        for _ in range(3):
            _lib.call("rai_hip_copy", 0, C.byref(src.desc()), C.byref(dst.desc()))
        sync()
    if args.graph_tokens > 0:
        out["graph_path"] = run_phi2_graph(args, args.graph_tokens)
        out["graph_decode_tokens_per_s"] = out["graph_path"]["composed_decode_tokens_per_s"]
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
