"""Qwen2 and Gemma decoders on the device vs the CPU oracle, through the C ABI."""
import numpy as np
import pytest

from oracle import qwen2
from oracle.dtypes import to_storage
from tests.test_gpu_phi2 import check_tokens
from tests.util import assert_close

pytestmark = pytest.mark.gpu


def make(cfg, dt, max_batch=2, max_context=64, seed=0):
    from rai_amd.models import Decoder
    params = qwen2.random_params(cfg, dt, seed=seed)
    g = np.random.Generator(np.random.PCG64(seed + 100))
    for k in params:   # exercise biases and norm weights
        if k.endswith(".bias"):
            params[k] = qwen2.rnd(0.02 * g.standard_normal(params[k].shape).astype(np.float32), dt)
        elif k.endswith("norm.weight"):
            params[k] = qwen2.rnd(params[k] + 0.1 * g.standard_normal(params[k].shape).astype(np.float32), dt)
    dec = Decoder(cfg.arch, dt, vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size,
                  intermediate_size=cfg.intermediate_size, num_hidden_layers=cfg.num_hidden_layers,
                  num_attention_heads=cfg.num_attention_heads, num_key_value_heads=cfg.num_key_value_heads,
                  head_dim=cfg.head_dim, rotary_dim=cfg.head_dim, max_position_embeddings=cfg.max_position_embeddings,
                  hidden_act=cfg.hidden_act, tie_word_embeddings=cfg.arch == "gemma", rope_theta=cfg.rope_theta,
                  norm_eps=cfg.rms_norm_eps, max_batch=max_batch, max_context=max_context)
    names = dec.param_names()
    assert set(names) == set(params)
    for n in names:
        assert names[n] == params[n].size
        dec.load_param(n, to_storage(params[n], dt))
    return dec, qwen2.Model(cfg, params, dt)


CFGS = {
    "qwen2": lambda: qwen2.Config("qwen2", 1000, 256, 640, 2, 4, 2, "silu", max_position_embeddings=64, rope_theta=1e6,
                                  head_dim=64),
    "gemma": lambda: qwen2.Config("gemma", 1000, 512, 1024, 2, 2, 1, "gelu", max_position_embeddings=64, head_dim=256),
}


@pytest.mark.parametrize("arch", ["qwen2", "gemma"])
@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_prefill_then_decode_logits(hip, arch, dt):
    cfg = CFGS[arch]()
    dec, ref = make(cfg, dt)
    ids = np.random.Generator(np.random.PCG64(1)).integers(0, cfg.vocab_size, (2, 21)).astype(np.uint32)
    logits, tok = dec.forward(ids)
    want = ref.fwd(ids)
    assert_close(logits, want, dt, f"{arch} prefill logits")
    check_tokens(tok, want, dt)
    nxt = np.argmax(want, -1).astype(np.uint32).reshape(2, 1)
    for step in range(4):
        logits, tok = dec.forward(nxt)
        want = ref.fwd(nxt)
        assert_close(logits, want, dt, f"{arch} decode step {step}")
        check_tokens(tok, want, dt)
        nxt = np.argmax(want, -1).astype(np.uint32).reshape(2, 1)
    dec.close()


@pytest.mark.parametrize("arch", ["qwen2", "gemma"])
def test_batched_prefill_many_rows_bf16(hip, arch):
    # enough rows for the MFMA tile path (gated-MLP epilogue, q/k/v bias, GQA flash attention)
    cfg = CFGS[arch]()
    dec, ref = make(cfg, "bf16", max_batch=4, max_context=64)
    ids = np.random.Generator(np.random.PCG64(2)).integers(0, cfg.vocab_size, (4, 40)).astype(np.uint32)
    logits, tok = dec.forward(ids)
    want = ref.fwd(ids)
    assert_close(logits, want, "bf16", f"{arch} batched prefill")
    check_tokens(tok, want, "bf16")
    dec.close()


@pytest.mark.parametrize("arch", ["qwen2", "gemma"])
def test_greedy_generate_matches_oracle(hip, arch):
    cfg = CFGS[arch]()
    dec, ref = make(cfg, "bf16")
    prompt = np.random.Generator(np.random.PCG64(3)).integers(0, cfg.vocab_size, (2, 12)).astype(np.uint32)
    toks, _, _ = dec.generate(prompt, 10)
    want, logits_all = qwen2.greedy_decode(ref, prompt, 10)
    for b in range(2):
        for s in range(10):
            if toks[b, s] != want[b, s]:
                check_tokens(toks[:, s], logits_all[s], "bf16")
                break
    toks2, _, _ = dec.generate(prompt, 10)
    assert np.array_equal(toks, toks2)
    dec.close()


@pytest.mark.parametrize("arch", ["qwen2", "gemma"])
def test_batched_decode_many_sequences_bf16(hip, arch):
    # 24 sequences decoded together: 9..64 activation rows take the weight-streaming MFMA path
    # (gated-MLP epilogue, q/k/v bias, output split, residual) and the split decode attention
    cfg = CFGS[arch]()
    dec, ref = make(cfg, "bf16", max_batch=24, max_context=64)
    ids = np.random.Generator(np.random.PCG64(4)).integers(0, cfg.vocab_size, (24, 5)).astype(np.uint32)
    logits, tok = dec.forward(ids)
    want = ref.fwd(ids)
    assert_close(logits, want, "bf16", f"{arch} prefill 24x5")
    nxt = np.argmax(want, -1).astype(np.uint32).reshape(24, 1)
    for step in range(3):
        logits, tok = dec.forward(nxt)
        want = ref.fwd(nxt)
        assert_close(logits, want, "bf16", f"{arch} batched decode step {step}")
        check_tokens(tok, want, "bf16")
        nxt = np.argmax(want, -1).astype(np.uint32).reshape(24, 1)
    dec.close()


GQA_CFGS = {
    # all query heads of a KV head share one block of the MFMA decode-attention kernel
    "gemma-mqa-8x256": lambda: qwen2.Config("gemma", 500, 256, 512, 1, 8, 1, "gelu", max_position_embeddings=320,
                                            head_dim=256),
    "qwen2-gqa-12/2x128": lambda: qwen2.Config("qwen2", 500, 256, 512, 1, 12, 2, "silu", max_position_embeddings=320,
                                               rope_theta=1e6, head_dim=128),
    "qwen2-gqa-16/4x64": lambda: qwen2.Config("qwen2", 500, 256, 512, 1, 16, 4, "silu", max_position_embeddings=320,
                                              rope_theta=1e6, head_dim=64),
}


@pytest.mark.parametrize("splits,keys", [(None, None), ("2", None), ("2", "128"), ("5", "128"), ("2", "96"), ("4", "96")])
@pytest.mark.parametrize("name", list(GQA_CFGS))
def test_grouped_query_decode_attention_long_context(hip, name, splits, keys, monkeypatch):
    # context long enough that one block holds several 16-key tiles (few splits) or a handful of keys
    # (default: as many splits as fill the GPU); the new token lands in different tiles and lanes
    if splits is None:
        monkeypatch.delenv("RAI_HIP_ATTN_SPLITS", raising=False)
    else:
        monkeypatch.setenv("RAI_HIP_ATTN_SPLITS", splits)
    if keys is None:
        monkeypatch.delenv("RAI_HIP_ATTN_KEYS", raising=False)
    else:
        monkeypatch.setenv("RAI_HIP_ATTN_KEYS", keys)     # keys per block of the MFMA kernel
    cfg = GQA_CFGS[name]()
    dec, ref = make(cfg, "bf16", max_batch=3, max_context=320)
    ids = np.random.Generator(np.random.PCG64(5)).integers(0, cfg.vocab_size, (3, 171)).astype(np.uint32)
    logits, tok = dec.forward(ids)
    want = ref.fwd(ids)
    assert_close(logits, want, "bf16", f"{name} prefill")
    nxt = np.argmax(want, -1).astype(np.uint32).reshape(3, 1)
    for step in range(6):
        logits, tok = dec.forward(nxt)
        want = ref.fwd(nxt)
        assert_close(logits, want, "bf16", f"{name} decode step {step} splits {splits}")
        check_tokens(tok, want, "bf16")
        nxt = np.argmax(want, -1).astype(np.uint32).reshape(3, 1)
    dec.close()
