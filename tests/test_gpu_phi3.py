"""Phi-3 decoder on the device (the Qwen2 block with fused qkv_proj / gate_up_proj parameters,
rai-models/src/llm/phi3.rs) against the CPU oracle, through the C ABI."""
import numpy as np
import pytest

from oracle import phi3
from oracle.dtypes import to_storage
from tests.test_gpu_phi2 import check_tokens
from tests.util import assert_close

pytestmark = pytest.mark.gpu


def make(cfg, dt, max_batch=2, max_context=64, seed=0):
    from rai_amd.models import Decoder
    params = phi3.random_params(cfg, dt, seed=seed)
    g = np.random.Generator(np.random.PCG64(seed + 100))
    for k in params:
        if k.endswith("norm.weight"):
            params[k] = phi3.rnd(params[k] + 0.1 * g.standard_normal(params[k].shape).astype(np.float32), dt)
    dec = Decoder("phi3", dt, vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size,
                  intermediate_size=cfg.intermediate_size, num_hidden_layers=cfg.num_hidden_layers,
                  num_attention_heads=cfg.num_attention_heads, num_key_value_heads=cfg.num_key_value_heads,
                  head_dim=cfg.head_dim, rotary_dim=cfg.head_dim, max_position_embeddings=cfg.max_position_embeddings,
                  hidden_act=cfg.hidden_act, tie_word_embeddings=False, rope_theta=cfg.rope_theta,
                  norm_eps=cfg.rms_norm_eps, max_batch=max_batch, max_context=max_context)
    names = dec.param_names()
    assert set(names) == set(params)            # the fused names of phi3.rs, nothing else
    for n in names:
        assert names[n] == params[n].size
        dec.load_param(n, to_storage(params[n], dt))
    return dec, phi3.Model(cfg, params, dt)


def small_cfg(**kw):
    base = dict(vocab_size=1000, hidden_size=384, intermediate_size=640, num_hidden_layers=2, num_attention_heads=4,
                num_key_value_heads=2, hidden_act="silu", max_position_embeddings=64)   # head_dim 96 as Phi-3-mini
    base.update(kw)
    return phi3.Config(**base)


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_prefill_then_decode_logits(hip, dt):
    cfg = small_cfg()
    dec, ref = make(cfg, dt)
    ids = np.random.Generator(np.random.PCG64(1)).integers(0, cfg.vocab_size, (2, 21)).astype(np.uint32)
    logits, tok = dec.forward(ids)
    want = ref.fwd(ids)
    assert_close(logits, want, dt, "prefill logits")
    check_tokens(tok, want, dt)
    nxt = np.argmax(want, -1).astype(np.uint32).reshape(2, 1)
    for step in range(5):
        logits, tok = dec.forward(nxt)
        want = ref.fwd(nxt)
        assert_close(logits, want, dt, f"decode step {step}")
        check_tokens(tok, want, dt)
        nxt = np.argmax(want, -1).astype(np.uint32).reshape(2, 1)
    assert dec.context_len() == 26
    dec.close()


def test_greedy_generate_matches_oracle(hip):
    cfg = small_cfg(num_key_value_heads=4)      # multi-head variant (Phi-3-mini has kv heads == heads)
    dec, ref = make(cfg, "bf16")
    prompt = np.random.Generator(np.random.PCG64(3)).integers(0, cfg.vocab_size, (2, 12)).astype(np.uint32)
    toks, _, _ = dec.generate(prompt, 10)
    want, logits_all = phi3.greedy_decode(ref, prompt, 10)
    for b in range(2):
        for s in range(10):
            if toks[b, s] != want[b, s]:
                check_tokens(toks[:, s], logits_all[s], "bf16")
                break
    toks2, _, _ = dec.generate(prompt, 10)
    assert np.array_equal(toks, toks2)
    dec.close()


def test_batched_decode_many_sequences_bf16(hip):
    cfg = small_cfg()
    dec, ref = make(cfg, "bf16", max_batch=24, max_context=48)
    ids = np.random.Generator(np.random.PCG64(4)).integers(0, cfg.vocab_size, (24, 7)).astype(np.uint32)
    logits, _ = dec.forward(ids)
    want = ref.fwd(ids)
    assert_close(logits, want, "bf16", "prefill logits")
    nxt = np.argmax(want, -1).astype(np.uint32).reshape(24, 1)
    for step in range(3):
        logits, tok = dec.forward(nxt)
        want = ref.fwd(nxt)
        assert_close(logits, want, "bf16", f"decode step {step}")
        nxt = np.argmax(want, -1).astype(np.uint32).reshape(24, 1)
    dec.close()


def test_rotary_inverse_frequencies_round_once_from_f64(hip):
    # phi3.rs:45-51 casts an f64 tensor to the model dtype; the decoder's single-token logits on a long context depend
    # on those tables, so a bf16 run over many positions against the oracle (which rounds once) covers it
    cfg = small_cfg(num_hidden_layers=1, max_position_embeddings=128)
    dec, ref = make(cfg, "bf16", max_batch=1, max_context=128)
    ids = np.random.Generator(np.random.PCG64(5)).integers(0, cfg.vocab_size, (1, 120)).astype(np.uint32)
    logits, _ = dec.forward(ids)
    assert_close(logits, ref.fwd(ids), "bf16", "long prefill")
    dec.close()


def test_safetensors_with_fused_names(hip, tmp_path):
    from tests.test_gpu_safetensors import write_safetensors
    cfg = small_cfg(num_hidden_layers=1)
    dec, ref = make(cfg, "f32", max_batch=1)
    fresh_params = phi3.random_params(cfg, "f32", seed=11)
    path = tmp_path / "phi3.safetensors"
    write_safetensors(path, fresh_params, "F32")
    dec.load_safetensors([str(path)])
    ids = np.array([[5, 9, 700, 31]], np.uint32)
    logits, _ = dec.forward(ids)
    assert_close(logits, phi3.Model(cfg, fresh_params, "f32").fwd(ids), "f32", "after load_safetensors")
    dec.close()
