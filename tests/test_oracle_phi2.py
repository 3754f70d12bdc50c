"""Pins the Phi-2 restatement (oracle/phi2.py) against an independent
implementation: Hugging Face transformers' PhiForCausalLM built locally from an
in-memory config (no download) and loaded with the oracle's seeded weights --
rai's parameter names coincide with the HF ones (phi2.rs:307-313)."""
import numpy as np
import pytest
import torch

from oracle import phi2


def hf_model(cfg, params, qk_layernorm=False):
    from transformers import PhiConfig, PhiForCausalLM
    hc = PhiConfig(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size, intermediate_size=cfg.intermediate_size,
                   num_hidden_layers=cfg.num_hidden_layers, num_attention_heads=cfg.num_attention_heads,
                   num_key_value_heads=cfg.num_key_value_heads, max_position_embeddings=cfg.max_position_embeddings,
                   partial_rotary_factor=cfg.partial_rotary_factor, hidden_act="gelu_new",
                   layer_norm_eps=cfg.layer_norm_eps, rope_theta=cfg.rope_theta, tie_word_embeddings=False,
                   resid_pdrop=0.0, embd_pdrop=0.0, attention_dropout=0.0, qk_layernorm=qk_layernorm)
    hc._attn_implementation = "eager"
    m = PhiForCausalLM(hc).eval()
    sd = {k: torch.from_numpy(np.asarray(v, np.float32)) for k, v in params.items()}
    missing, unexpected = m.load_state_dict(sd, strict=False)
    assert not unexpected and all("rotary" in k or "inv_freq" in k for k in missing), (missing, unexpected)
    return m


@pytest.mark.parametrize("kv_heads", [None, 2])
def test_phi2_oracle_matches_hf_transformers(kv_heads):
    cfg = phi2.Config(vocab_size=500, hidden_size=320, intermediate_size=640, num_hidden_layers=2,
                      num_attention_heads=4, num_key_value_heads=kv_heads, max_position_embeddings=64)
    params = phi2.random_params(cfg, "f32", seed=3, std=0.05)
    # non-trivial biases / LayerNorm parameters so every term is exercised
    g = np.random.Generator(np.random.PCG64(9))
    for k in params:
        if k.endswith(".bias"):
            params[k] = (0.05 * g.standard_normal(params[k].shape)).astype(np.float32)
        elif k.endswith("layernorm.weight"):
            params[k] = (1 + 0.1 * g.standard_normal(params[k].shape)).astype(np.float32)
    ref = phi2.Model(cfg, params, "f32")
    hf = hf_model(cfg, params)
    ids = g.integers(0, cfg.vocab_size, (2, 19)).astype(np.uint32)
    with torch.no_grad():
        out = hf(torch.from_numpy(ids.astype(np.int64)), use_cache=True)
    want = out.logits[:, -1, :].numpy()
    got = ref.fwd(ids)
    assert np.max(np.abs(got - want)) <= 1e-4 * np.max(np.abs(want))
    # one cached decode step
    nxt = np.argmax(want, -1).astype(np.uint32).reshape(2, 1)
    with torch.no_grad():
        out2 = hf(torch.from_numpy(nxt.astype(np.int64)), past_key_values=out.past_key_values, use_cache=True)
    got2 = ref.fwd(nxt)
    assert np.max(np.abs(got2 - out2.logits[:, -1, :].numpy())) <= 1e-4 * np.max(np.abs(want))


def test_kv_cache_equals_recompute_and_greedy_loop():
    cfg = phi2.Config(vocab_size=300, hidden_size=160, intermediate_size=320, num_hidden_layers=2,
                      num_attention_heads=2, max_position_embeddings=48)
    params = phi2.random_params(cfg, "f32", seed=1, std=0.1)
    m = phi2.Model(cfg, params, "f32")
    ids = np.random.Generator(np.random.PCG64(2)).integers(0, 300, (1, 12)).astype(np.uint32)
    toks, _ = phi2.greedy_decode(m, ids, 5)
    # recomputing the whole sequence without a cache gives the same next tokens
    seq = ids
    for s in range(5):
        m.clear_kv_cache()
        nxt = np.argmax(m.fwd(seq), -1).astype(np.uint32)
        assert nxt[0] == toks[0, s]
        seq = np.concatenate([seq, nxt.reshape(1, 1)], 1)


def test_bf16_model_close_to_f32_model_and_param_names():
    cfg = phi2.Config(vocab_size=300, hidden_size=160, intermediate_size=320, num_hidden_layers=2,
                      num_attention_heads=2, max_position_embeddings=48)
    names = phi2.param_shapes(cfg)
    assert "model.layers.1.self_attn.dense.bias" in names and "model.final_layernorm.weight" in names
    assert names["lm_head.weight"] == (300, 160) and names["model.layers.0.mlp.fc1.weight"] == (320, 160)
    pb = phi2.random_params(cfg, "bf16", seed=1)
    ids = np.random.Generator(np.random.PCG64(2)).integers(0, 300, (2, 10)).astype(np.uint32)
    lb = phi2.Model(cfg, pb, "bf16").fwd(ids)
    lf = phi2.Model(cfg, pb, "f32").fwd(ids)      # same (bf16-representable) weights, f32 arithmetic
    assert np.max(np.abs(lb - lf)) <= 2e-2 * np.max(np.abs(lf))


def test_qk_layernorm_single_head_matches_hf_and_many_heads_is_the_references_shape_error():
    # phi2.rs:207-216 normalises the un-split projections with head_dim-sized parameters: well-formed for one head
    # only, where it coincides with transformers' per-head q/k LayerNorm
    cfg = phi2.Config(vocab_size=300, hidden_size=80, intermediate_size=160, num_hidden_layers=2, num_attention_heads=1,
                      max_position_embeddings=48, qk_layernorm=True)
    params = phi2.random_params(cfg, "f32", seed=4, std=0.1)
    g = np.random.Generator(np.random.PCG64(10))
    for k in params:
        if k.endswith(".bias"):
            params[k] = (0.05 * g.standard_normal(params[k].shape)).astype(np.float32)
        elif k.endswith("layernorm.weight"):
            params[k] = (1 + 0.1 * g.standard_normal(params[k].shape)).astype(np.float32)
    assert params["model.layers.0.self_attn.q_layernorm.weight"].shape == (80,)
    ids = g.integers(0, cfg.vocab_size, (2, 11)).astype(np.uint32)
    hf = hf_model(cfg, params, qk_layernorm=True)
    with torch.no_grad():
        want = hf(torch.from_numpy(ids.astype(np.int64))).logits[:, -1, :].numpy()
    got = phi2.Model(cfg, params, "f32").fwd(ids)
    assert np.max(np.abs(got - want)) <= 1e-4 * np.max(np.abs(want))
    many = phi2.Config(vocab_size=300, hidden_size=160, intermediate_size=160, num_hidden_layers=1,
                       num_attention_heads=2, max_position_embeddings=48, qk_layernorm=True)
    with pytest.raises(ValueError, match="IncompatibleShape"):
        phi2.Model(many, phi2.random_params(many, "f32", seed=4), "f32").fwd(ids)
