"""Pins oracle/phi3.py (rai-models/src/llm/phi3.rs restated) against Hugging Face transformers'
Phi3ForCausalLM built locally from an in-memory config and loaded with the oracle's seeded weights
(the parameter names coincide with rai's, phi3.rs:262-270)."""
import numpy as np
import pytest
import torch

from oracle import phi3


def hf_model(cfg, params):
    import transformers
    hc = transformers.Phi3Config(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size,
                                 intermediate_size=cfg.intermediate_size, num_hidden_layers=cfg.num_hidden_layers,
                                 num_attention_heads=cfg.num_attention_heads, num_key_value_heads=cfg.num_key_value_heads,
                                 max_position_embeddings=cfg.max_position_embeddings,
                                 original_max_position_embeddings=cfg.max_position_embeddings, rms_norm_eps=cfg.rms_norm_eps,
                                 rope_theta=cfg.rope_theta, hidden_act="silu", attention_dropout=0.0, resid_pdrop=0.0,
                                 embd_pdrop=0.0, tie_word_embeddings=False, pad_token_id=0, sliding_window=None)
    hc._attn_implementation = "eager"
    m = transformers.Phi3ForCausalLM(hc).eval()
    sd = {k: torch.from_numpy(np.asarray(v, np.float32)) for k, v in params.items()}
    missing, unexpected = m.load_state_dict(sd, strict=False)
    assert not unexpected and all("rotary" in k or "inv_freq" in k for k in missing), (missing, unexpected)
    return m


@pytest.mark.parametrize("heads,kv,hd", [(4, 4, 32), (4, 2, 24), (6, 1, 16)])
def test_oracle_matches_hf_transformers(heads, kv, hd):
    cfg = phi3.Config(400, heads * hd, 256, 2, heads, kv, "silu", max_position_embeddings=64, rope_theta=1e4)
    params = phi3.random_params(cfg, "f32", seed=7, std=0.05)
    g = np.random.Generator(np.random.PCG64(8))
    for k in params:
        if k.endswith("norm.weight"):
            params[k] = (params[k] + 0.1 * g.standard_normal(params[k].shape)).astype(np.float32)
    ref = phi3.Model(cfg, params, "f32")
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


def test_fused_projections_equal_their_split_form():
    # the fused qkv_proj / gate_up_proj are row-wise concatenations: the same model written with Qwen2's split
    # projections (no biases) gives the same logits bit for bit, up to the rotary table's inv_freq rounding
    from oracle import qwen2
    cfg = phi3.Config(300, 96, 128, 2, 4, 2, "silu", max_position_embeddings=32)
    p3 = phi3.random_params(cfg, "f32", seed=9)
    qd, kd, i = 96, 48, 128
    pq = {}
    for k, v in p3.items():
        if k.endswith("qkv_proj.weight"):
            pre = k[: -len("qkv_proj.weight")]
            pq[pre + "q_proj.weight"], pq[pre + "k_proj.weight"], pq[pre + "v_proj.weight"] = v[:qd], v[qd:qd + kd], v[qd + kd:]
        elif k.endswith("gate_up_proj.weight"):
            pre = k[: -len("gate_up_proj.weight")]
            pq[pre + "gate_proj.weight"], pq[pre + "up_proj.weight"] = v[:i], v[i:]
        else:
            pq[k] = v
    qcfg = qwen2.Config("qwen2", 300, 96, 128, 2, 4, 2, "silu", max_position_embeddings=32, rms_norm_eps=cfg.rms_norm_eps,
                        head_dim=24)
    a = phi3.Model(cfg, p3, "f32")
    b = qwen2.Model(qcfg, pq, "f32")
    ids = np.random.Generator(np.random.PCG64(10)).integers(0, 300, (1, 9)).astype(np.uint32)
    assert np.allclose(a.fwd(ids), b.fwd(ids), rtol=0, atol=2e-5)


def test_parameter_names_and_bf16():
    cfg = phi3.Config(200, 64, 96, 1, 2, 1)
    names = phi3.param_shapes(cfg)
    assert names["model.layers.0.self_attn.qkv_proj.weight"] == (64 + 2 * 32, 64)
    assert names["model.layers.0.mlp.gate_up_proj.weight"] == (192, 64)
    assert "lm_head.weight" in names and not any(k.endswith(".bias") for k in names)
    ids = np.array([[3, 5, 7, 11]], np.uint32)
    f = phi3.Model(cfg, phi3.random_params(cfg, "f32", 1), "f32").fwd(ids)
    b = phi3.Model(cfg, phi3.random_params(cfg, "bf16", 1), "bf16").fwd(ids)
    assert np.max(np.abs(f - b)) <= 3e-2 * np.max(np.abs(f))
