"""Qwen2-1.5B and Gemma-2B at their full widths (two layers of each, so that the CPU oracle stays affordable):

* Qwen2-1.5B architecture, bf16: batched prefill of 16 x 1024 tokens with the causal mask: hidden 1536,
  12 query / 2 KV heads of 128, SwiGLU 8960, RMSNorm eps 1e-6, RoPE theta 1e6, vocabulary 151936.
* Gemma-2B architecture, bf16: decode at batch 32 on a 2048-token context per sequence: hidden 2048, 8 query /
  1 KV head of 256, GeGLU 16384, RMSNorm with (1 + w), embedding scaled by sqrt(2048), tied 256000-way head.

The device runs the whole batch; sequences are independent of each other through every operator, so the oracle
(rai-models/src/llm/qwen2.rs, gemma.rs restated) is run on a few of the sequences and compared row by row.
"""
import numpy as np
import pytest

from oracle import qwen2
from oracle.dtypes import rnd, to_storage
from tests.test_gpu_phi2 import check_tokens
from tests.util import assert_close, assert_logits_close, progress, synthetic_params

pytestmark = pytest.mark.gpu


def build(cfg, max_batch, max_context, request):
    from rai_amd.models import Decoder
    dt = "bf16"
    progress(request, "generating seeded weights")
    params = synthetic_params(qwen2.param_shapes(cfg), dt, seed=0, norm_weight=0.0 if cfg.arch == "gemma" else 1.0)
    g = np.random.Generator(np.random.PCG64(77))
    for k in params:   # biases and norm weights away from their trivial values
        if k.endswith(".bias"):
            params[k] = rnd(0.02 * g.standard_normal(params[k].shape).astype(np.float32), dt)
        elif k.endswith("norm.weight"):
            params[k] = rnd(params[k] + 0.1 * g.standard_normal(params[k].shape).astype(np.float32), dt)
    dec = Decoder(cfg.arch, dt, vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size,
                  intermediate_size=cfg.intermediate_size, num_hidden_layers=cfg.num_hidden_layers,
                  num_attention_heads=cfg.num_attention_heads, num_key_value_heads=cfg.num_key_value_heads,
                  head_dim=cfg.head_dim, rotary_dim=cfg.head_dim, max_position_embeddings=cfg.max_position_embeddings,
                  hidden_act=cfg.hidden_act, tie_word_embeddings=cfg.arch == "gemma", rope_theta=cfg.rope_theta,
                  norm_eps=cfg.rms_norm_eps, max_batch=max_batch, max_context=max_context)
    names = dec.param_names()
    assert set(names) == set(params)
    for n in names:
        dec.load_param(n, to_storage(params[n], dt))
    return dec, params


def test_qwen2_1p5b_widths_prefill_16x1024(hip, request):
    cfg = qwen2.Config("qwen2", 151936, 1536, 8960, 2, 12, 2, "silu", max_position_embeddings=2048, rope_theta=1e6,
                       head_dim=128)
    dec, params = build(cfg, 16, 1024 + 8, request)
    ids = np.random.Generator(np.random.PCG64(31)).integers(0, cfg.vocab_size, (16, 1024)).astype(np.uint32)
    logits, tok = dec.forward(ids)                 # 16384 rows: eight-wave 256x256 tiles, GQA flash attention
    assert logits.shape == (16, cfg.vocab_size)
    rows = [0, 6, 15]
    progress(request, f"oracle prefill of sequences {rows}")
    ref = qwen2.Model(cfg, params, "bf16")
    # the same stored weights and the same (bf16) rotary tables, f32 arithmetic without intermediate rounding: at
    # this width and length the bf16 node-by-node chain is ~2 % (of the largest logit) away from it by itself
    exact = qwen2.Model(cfg, params, "f32")
    exact.sin, exact.cos = ref.sin, ref.cos
    want = ref.fwd(ids[rows])
    errs = assert_logits_close(logits[rows], want, exact.fwd(ids[rows]), "bf16", "Qwen2-1.5B widths, prefill 16 x 1024")
    progress(request, "relative errors: device vs unrounded %.4f, chain vs unrounded %.4f, device vs chain %.4f" % errs)
    check_tokens(tok[rows], want, "bf16")
    # one decode step on top of the 1024-token cache for all 16 sequences
    nxt = tok.copy().reshape(16, 1)
    nxt[rows, 0] = np.argmax(want, -1).astype(np.uint32)
    logits, tok = dec.forward(nxt)
    want = ref.fwd(nxt[rows])
    assert_logits_close(logits[rows], want, exact.fwd(nxt[rows]), "bf16", "decode step at context 1024")
    check_tokens(tok[rows], want, "bf16")
    dec.close()


def test_gemma_2b_widths_decode_batch32_context2048(hip, request):
    cfg = qwen2.Config("gemma", 256000, 2048, 16384, 2, 8, 1, "gelu", max_position_embeddings=4096, head_dim=256)
    B, CTX = 32, 2048
    dec, params = build(cfg, B, CTX + 8, request)
    ids = np.random.Generator(np.random.PCG64(32)).integers(0, cfg.vocab_size, (B, CTX)).astype(np.uint32)
    progress(request, "device prefill 32 x 2048")
    logits, tok = dec.forward(ids)
    rows = [0, 13, 31]
    progress(request, f"oracle prefill of sequences {rows}")
    ref = qwen2.Model(cfg, params, "bf16")
    want = ref.fwd(ids[rows])
    assert_close(logits[rows], want, "bf16", "Gemma-2B widths, prefill 32 x 2048: logits")
    check_tokens(tok[rows], want, "bf16")
    for step in range(4):                          # batch-32 decode: weight-streaming MFMA Linears, MQA decode attention,
        nxt = tok.copy().reshape(B, 1)             # 256000-row tied head, device argmax
        nxt[rows, 0] = np.argmax(want, -1).astype(np.uint32)
        logits, tok = dec.forward(nxt)
        want = ref.fwd(nxt[rows])
        assert_close(logits[rows], want, "bf16", f"decode step {step} at context {CTX + step}")
        check_tokens(tok[rows], want, "bf16")
        # every row's token is the argmax of that row's own logits (first maximum), bit-exactly
        assert np.array_equal(tok, np.argmax(logits, -1).astype(np.uint32))
    assert dec.context_len() == CTX + 4
    dec.close()


@pytest.mark.parametrize("arch", ["qwen2", "gemma"])
def test_single_layer_full_width_against_the_chain(hip, request, arch):
    """One layer at the full widths (Qwen2-1.5B: 1536 / 8960, 12 / 2 heads of 128, 2 x 1024 positions; Gemma-2B: 2048 /
    16384, 8 / 1 heads of 256, 2 x 512 positions; bf16) fed with rows of residual-stream size, against the
    node-by-node bf16 chain of the same layer.  Without depth no rounding noise builds up, so the plain 2e-2 bound
    applies, to the layer's output and to what the layer adds to its input."""
    if arch == "qwen2":
        cfg = qwen2.Config("qwen2", 512, 1536, 8960, 1, 12, 2, "silu", max_position_embeddings=2048, rope_theta=1e6, head_dim=128)
        B, S = 2, 1024
    else:
        cfg = qwen2.Config("gemma", 512, 2048, 16384, 1, 8, 1, "gelu", max_position_embeddings=4096, head_dim=256)
        B, S = 2, 512
    dec, params = build(cfg, B, S, request)
    g = np.random.Generator(np.random.PCG64(43))
    x = rnd(g.standard_normal((B, S, cfg.hidden_size)).astype(np.float32), "bf16")
    got, _, _ = dec.forward_hidden(hidden_in=to_storage(x, "bf16"))
    progress(request, "oracle: one layer, bf16 chain")
    ref = qwen2.Model(cfg, params, "bf16")
    want = ref.layer(0, x, qwen2.causal_mask(S, 0, "bf16"), 0)
    assert_close(got, want, "bf16", f"{arch} layer output vs the bf16 chain")
    ulp = float(np.max(np.abs(want))) * 2.0 ** -8     # one rounding of the output: no error of the layer
    d_got, d_want = got.astype(np.float64) - x, want.astype(np.float64) - x
    err, scale = float(np.max(np.abs(d_got - d_want))), float(np.max(np.abs(d_want)))
    progress(request, "layer contribution: max error %.3e of %.3e (%.4f), one output rounding %.3e" % (err, scale, err / scale, ulp))
    assert err <= 2e-2 * scale + ulp, f"attention + MLP contribution off by {err:.3e} (scale {scale:.3e})"
    dec.close()


@pytest.mark.parametrize("arch", ["gemma", "qwen2"])
def test_decode_chain_against_launch_per_linear(hip, request, monkeypatch, arch):
    """Batched decode steps through the persistent decode chain kernel (o_proj, gate|up, down, the sum of its K splits
    and the next layer's q|k|v as phases of one launch) against the same steps with one launch per Linear: the same
    weight-stream arithmetic, so the logits agree to within the rounding of the regrouped K-split sum and the tokens are
    the same; and against the oracle on a few sequences."""
    if arch == "gemma":
        cfg = qwen2.Config("gemma", 4096, 2048, 16384, 3, 8, 1, "gelu", max_position_embeddings=256, head_dim=256)
        B = 32
    else:
        cfg = qwen2.Config("qwen2", 4096, 1536, 8960, 3, 12, 2, "silu", max_position_embeddings=256, rope_theta=1e6, head_dim=128)
        B = 16
    CTX, STEPS = 40, 3
    ids = np.random.Generator(np.random.PCG64(51)).integers(0, cfg.vocab_size, (B, CTX)).astype(np.uint32)
    runs = {}
    for label, on in (("chain", "1"), ("per linear", None)):
        if on:
            monkeypatch.setenv("RAI_HIP_CHAIN", on)
        else:
            monkeypatch.delenv("RAI_HIP_CHAIN", raising=False)
        dec, params = build(cfg, B, CTX + STEPS + 1, request)
        logits, tok = dec.forward(ids)
        steps = []
        for _ in range(STEPS):
            logits, tok = dec.forward(tok.reshape(B, 1))
            steps.append((logits.copy(), tok.copy()))
        runs[label] = steps
        dec.close()
    for s, ((lc, tc), (lp, tp)) in enumerate(zip(runs["chain"], runs["per linear"])):
        assert_close(lc, lp, "bf16", f"{arch} decode step {s}: chain vs launch per Linear")
        assert np.array_equal(tc, np.argmax(lc, -1).astype(np.uint32))
    # the chain's first step against the oracle on three sequences (the later steps were fed the device's own tokens)
    rows = [0, B // 2, B - 1]
    ref = qwen2.Model(cfg, params, "bf16")
    exact = qwen2.Model(cfg, params, "f32")       # the same stored weights and rotary tables, f32 arithmetic
    exact.sin, exact.cos = ref.sin, ref.cos
    ref.fwd(ids[rows])
    exact.fwd(ids[rows])
    dec, _ = build(cfg, B, CTX + 2, request)
    _, tok0 = dec.forward(ids)
    logits, tok = dec.forward(tok0.reshape(B, 1))
    nxt = tok0[rows].reshape(-1, 1)
    want = ref.fwd(nxt)
    assert_logits_close(logits[rows], want, exact.fwd(nxt), "bf16", f"{arch} decode step through the chain vs the oracle")
    check_tokens(tok[rows], want, "bf16")
    dec.close()


@pytest.mark.parametrize("arch", ["qwen2", "gemma"])
def test_every_sequence_through_a_second_device_path(hip, request, monkeypatch, arch):
    """The oracle follows three sequences of these batches (a size it covers in minutes); the other 13 / 29 are held
    here to a second, independent device path: the same prefill and two decode steps once through the default kernels
    (DMA tile GEMMs with stream-K, streaming MFMA Linears over fragment-order weights with fused norms, MFMA decode
    attention, captured graph) and once through the register-staged 128 x 128 tile kernel on whole tiles, the
    LDS-staged small-M Linears over row-major weights, stand-alone norms, the context-split VALU decode attention and
    plain launches.  Every sequence's logits agree within the dtype's tolerance; tokens are each path's own argmax."""
    if arch == "qwen2":
        cfg = qwen2.Config("qwen2", 151936, 1536, 8960, 2, 12, 2, "silu", max_position_embeddings=2048, rope_theta=1e6,
                           head_dim=128)
        B, CTX = 16, 1024
    else:
        cfg = qwen2.Config("gemma", 256000, 2048, 16384, 2, 8, 1, "gelu", max_position_embeddings=4096, head_dim=256)
        B, CTX = 32, 2048
    ids = np.random.Generator(np.random.PCG64(61)).integers(0, cfg.vocab_size, (B, CTX)).astype(np.uint32)
    second = {"RAI_HIP_GEMM_TILE": "classic", "RAI_HIP_NO_STREAMK": "1", "RAI_HIP_NO_MFMA_STREAM": "1", "RAI_HIP_NO_MFMA_DECODE": "1",
              "RAI_HIP_NO_FRAG": "1", "RAI_HIP_NO_FUSED_NORM": "1", "RAI_HIP_NO_POST_NORM": "1", "RAI_HIP_NO_GRAPH": "1",
              "RAI_HIP_NO_SPLIT_CHOICE": "1", "RAI_HIP_NO_FUSED_SPLITK": "1"}
    runs = {}
    for label in ("default", "second"):
        for k, v in second.items():
            if label == "second":
                monkeypatch.setenv(k, v)
            else:
                monkeypatch.delenv(k, raising=False)
        dec, _ = build(cfg, B, CTX + 8, request)
        progress(request, f"{label} path: prefill {B} x {CTX} and two decode steps")
        logits, tok = dec.forward(ids)
        steps = [(logits.copy(), tok.copy())]
        feed = tok if label == "default" else runs["default"][0][1]     # both paths decode the same tokens
        for s in range(2):
            logits, tok = dec.forward(feed.reshape(B, 1))
            steps.append((logits.copy(), tok.copy()))
            feed = tok if label == "default" else runs["default"][s + 1][1]
        runs[label] = steps
        dec.close()
    for k in second:
        monkeypatch.delenv(k, raising=False)
    for s, ((la, ta), (lb, tb)) in enumerate(zip(runs["default"], runs["second"])):
        assert la.shape == (B, cfg.vocab_size)
        for b in range(B):
            assert_close(la[b], lb[b], "bf16", f"{arch} sequence {b}, step {s}: default vs second device path")
        assert np.array_equal(ta, np.argmax(la, -1).astype(np.uint32))
        assert np.array_equal(tb, np.argmax(lb, -1).astype(np.uint32))



def test_decode_chain_barrier_timeout_is_reported(hip, request, monkeypatch):
    """A barrier wait of the chain kernel that expires (forced from the host with a spin limit of one poll): the kernel
    flags the fault, later waits fall through so every wave exits, the call returns an error instead of wrong logits,
    and after clearing the cache the decoder works again."""
    from rai_amd._lib import RaiHipError
    cfg = qwen2.Config("gemma", 1024, 2048, 16384, 2, 8, 1, "gelu", max_position_embeddings=128, head_dim=256)
    B = 16
    monkeypatch.setenv("RAI_HIP_CHAIN", "1")
    dec, _ = build(cfg, B, 32, request)
    ids = np.random.Generator(np.random.PCG64(52)).integers(0, cfg.vocab_size, (B, 8)).astype(np.uint32)
    _, tok = dec.forward(ids)
    good, good_tok = dec.forward(tok.reshape(B, 1))
    dec.clear_kv_cache()
    _, tok = dec.forward(ids)
    monkeypatch.setenv("RAI_HIP_CHAIN_SPIN_LIMIT", "1")
    with pytest.raises(RaiHipError, match="barrier of the decode chain"):
        dec.forward(tok.reshape(B, 1))
    monkeypatch.delenv("RAI_HIP_CHAIN_SPIN_LIMIT")
    dec.clear_kv_cache()
    _, tok = dec.forward(ids)
    again, again_tok = dec.forward(tok.reshape(B, 1))
    np.testing.assert_array_equal(again, good)
    np.testing.assert_array_equal(again_tok, good_tok)
    dec.close()
