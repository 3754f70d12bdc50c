"""Pins oracle/qwen2.py (Qwen2 and Gemma restatements) against Hugging Face
transformers models built locally from in-memory configs and loaded with the
oracle's seeded weights (parameter names coincide with rai's, qwen2.rs:276-282,
gemma.rs:309-319)."""
import numpy as np
import pytest
import torch

from oracle import qwen2


def hf_model(cfg, params):
    import transformers
    common = dict(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size, intermediate_size=cfg.intermediate_size,
                  num_hidden_layers=cfg.num_hidden_layers, num_attention_heads=cfg.num_attention_heads,
                  num_key_value_heads=cfg.num_key_value_heads, max_position_embeddings=cfg.max_position_embeddings,
                  rms_norm_eps=cfg.rms_norm_eps, rope_theta=cfg.rope_theta, attention_dropout=0.0)
    if cfg.arch == "qwen2":
        hc = transformers.Qwen2Config(hidden_act="silu", tie_word_embeddings=False, use_sliding_window=False, **common)
        cls = transformers.Qwen2ForCausalLM
    else:
        hc = transformers.GemmaConfig(head_dim=cfg.head_dim, hidden_act="gelu", hidden_activation="gelu",
                                      attention_bias=False, tie_word_embeddings=True, **common)
        cls = transformers.GemmaForCausalLM
    hc._attn_implementation = "eager"
    m = cls(hc).eval()
    sd = {k: torch.from_numpy(np.asarray(v, np.float32)) for k, v in params.items()}
    if cfg.arch == "gemma":
        sd["lm_head.weight"] = sd["model.embed_tokens.weight"]
    missing, unexpected = m.load_state_dict(sd, strict=False)
    assert not unexpected and all("rotary" in k or "inv_freq" in k for k in missing), (missing, unexpected)
    return m


@pytest.mark.parametrize("arch,act,heads,kv,hd", [("qwen2", "silu", 4, 2, 32), ("qwen2", "silu", 4, 4, 32),
                                                 ("gemma", "gelu", 4, 1, 64), ("gemma", "gelu", 2, 2, 64)])
def test_oracle_matches_hf_transformers(arch, act, heads, kv, hd):
    hidden = heads * hd
    cfg = qwen2.Config(arch, 400, hidden, 256, 2, heads, kv, act, max_position_embeddings=64,
                       rope_theta=1e6 if arch == "qwen2" else 1e4, head_dim=hd)
    params = qwen2.random_params(cfg, "f32", seed=5, std=0.05)
    g = np.random.Generator(np.random.PCG64(6))
    for k in params:  # non-trivial biases and norm weights
        if k.endswith(".bias"):
            params[k] = (0.05 * g.standard_normal(params[k].shape)).astype(np.float32)
        elif k.endswith("norm.weight"):
            params[k] = (params[k] + 0.1 * g.standard_normal(params[k].shape)).astype(np.float32)
    ref = qwen2.Model(cfg, params, "f32")
    hf = hf_model(cfg, params)
    ids = g.integers(0, cfg.vocab_size, (2, 17)).astype(np.uint32)
    with torch.no_grad():
        out = hf(torch.from_numpy(ids.astype(np.int64)), use_cache=True)
    want = out.logits[:, -1, :].numpy()
    got = ref.fwd(ids)
    assert np.max(np.abs(got - want)) <= 1e-4 * np.max(np.abs(want))
    nxt = np.argmax(want, -1).astype(np.uint32).reshape(2, 1)
    with torch.no_grad():
        out2 = hf(torch.from_numpy(nxt.astype(np.int64)), past_key_values=out.past_key_values, use_cache=True)
    assert np.max(np.abs(ref.fwd(nxt) - out2.logits[:, -1, :].numpy())) <= 1e-4 * np.max(np.abs(want))


def test_bf16_close_to_f32_and_names():
    cfg = qwen2.Config("gemma", 300, 128, 256, 2, 2, 1, "gelu", max_position_embeddings=48, head_dim=64)
    names = qwen2.param_shapes(cfg)
    assert "lm_head.weight" not in names and names["model.layers.0.self_attn.k_proj.weight"] == (64, 128)
    assert "model.layers.0.self_attn.q_proj.bias" in qwen2.param_shapes(
        qwen2.Config("qwen2", 300, 128, 256, 1, 2, 1, "silu", head_dim=64))
    pb = qwen2.random_params(cfg, "bf16", seed=1)
    ids = np.random.Generator(np.random.PCG64(2)).integers(0, 300, (2, 10)).astype(np.uint32)
    lb = qwen2.Model(cfg, pb, "bf16").fwd(ids)
    lf = qwen2.Model(cfg, pb, "f32").fwd(ids)
    assert np.max(np.abs(lb - lf)) <= 2e-2 * np.max(np.abs(lf))
