"""Phi-2 decoder on the device vs the CPU oracle (rai-models/src/llm/phi2.rs restated),
through the C ABI: logits of prefill and decode steps, KV-cache behaviour and
greedy token identity."""
import numpy as np
import pytest

from oracle import phi2
from oracle.dtypes import to_storage
from tests.util import assert_close

pytestmark = pytest.mark.gpu


def make(cfg, dt, hip, max_batch=2, max_context=64, seed=0):
    from rai_amd.models import Decoder
    params = phi2.random_params(cfg, dt, seed=seed)
    dec = Decoder("phi2", dt, vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size,
                  intermediate_size=cfg.intermediate_size, num_hidden_layers=cfg.num_hidden_layers,
                  num_attention_heads=cfg.num_attention_heads, num_key_value_heads=cfg.num_key_value_heads,
                  rotary_dim=cfg.rotary_dim, max_position_embeddings=cfg.max_position_embeddings,
                  hidden_act=cfg.hidden_act, tie_word_embeddings=cfg.tie_word_embeddings, rope_theta=cfg.rope_theta,
                  norm_eps=cfg.layer_norm_eps, max_batch=max_batch, max_context=max_context)
    names = dec.param_names()
    assert set(names) == {n for n in params if not (cfg.tie_word_embeddings and n.startswith("lm_head"))}
    for n in names:
        assert names[n] == params[n].size
        dec.load_param(n, to_storage(params[n], dt))
    return dec, phi2.Model(cfg, params, dt)


def small_cfg(**kw):
    base = dict(vocab_size=1000, hidden_size=320, intermediate_size=1280, num_hidden_layers=2, num_attention_heads=4,
                max_position_embeddings=64)
    base.update(kw)
    return phi2.Config(**base)


def check_tokens(dev_tok, logits_oracle, dt):
    """Greedy ids must equal the oracle's; a mismatch is tolerated only where the
    oracle's own top-2 gap is inside the dtype's resolution (a near tie)."""
    want = np.argmax(logits_oracle, -1)
    for b in range(len(want)):
        if dev_tok[b] != want[b]:
            row = logits_oracle[b].astype(np.float64)
            gap = row[want[b]] - row[dev_tok[b]]
            tol = {"f32": 1e-4, "bf16": 2e-2}[dt] * np.max(np.abs(row))
            assert gap <= tol, f"token {dev_tok[b]} vs oracle {want[b]}, logit gap {gap:.3e} > {tol:.3e}"


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_prefill_then_decode_logits(hip, dt):
    cfg = small_cfg()
    dec, ref = make(cfg, dt, hip)
    ids = np.random.Generator(np.random.PCG64(1)).integers(0, cfg.vocab_size, (2, 24)).astype(np.uint32)
    logits, tok = dec.forward(ids)
    want = ref.fwd(ids)
    assert_close(logits, want, dt, "prefill logits")
    check_tokens(tok, want, dt)
    assert dec.context_len() == 24
    # six single-token steps on the cached context, feeding the oracle's tokens to both
    nxt = np.argmax(want, -1).astype(np.uint32).reshape(2, 1)
    for step in range(6):
        logits, tok = dec.forward(nxt)
        want = ref.fwd(nxt)
        assert_close(logits, want, dt, f"decode step {step}")
        check_tokens(tok, want, dt)
        nxt = np.argmax(want, -1).astype(np.uint32).reshape(2, 1)
    assert dec.context_len() == 30
    # clear_kv_cache restarts from position 0 and reproduces the first result
    dec.clear_kv_cache()
    ref.clear_kv_cache()
    again, _ = dec.forward(ids)
    assert_close(again, ref.fwd(ids), dt, "after clear_kv_cache")
    dec.close()


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_chunked_prefill_equals_whole(hip, dt):
    # appending 10 tokens to a 14-token cache must equal prefilling all 24 (causal offset mask)
    cfg = small_cfg()
    dec, ref = make(cfg, dt, hip)
    ids = np.random.Generator(np.random.PCG64(2)).integers(0, cfg.vocab_size, (1, 24)).astype(np.uint32)
    whole, _ = dec.forward(ids)
    dec.clear_kv_cache()
    dec.forward(ids[:, :14])
    part, _ = dec.forward(ids[:, 14:])
    assert_close(part, whole, dt, "chunked prefill")
    dec.close()


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_greedy_generate_matches_oracle(hip, dt):
    cfg = small_cfg(num_hidden_layers=3)
    dec, ref = make(cfg, dt, hip)
    prompt = np.random.Generator(np.random.PCG64(3)).integers(0, cfg.vocab_size, (2, 16)).astype(np.uint32)
    toks, pre_ms, dec_ms = dec.generate(prompt, 12)
    want, logits_all = phi2.greedy_decode(ref, prompt, 12)
    assert toks.dtype == np.uint32 and toks.shape == (2, 12) and pre_ms > 0 and dec_ms > 0
    for b in range(2):
        for s in range(12):
            if toks[b, s] != want[b, s]:
                # sequences legitimately diverge after a near tie; it must be one
                check_tokens(toks[:, s], logits_all[s], dt)
                break
    # generate is repeatable (cache is cleared on entry)
    toks2, _, _ = dec.generate(prompt, 12)
    assert np.array_equal(toks, toks2)
    dec.close()


def test_graph_replay_equals_eager_steps(hip, monkeypatch):
    # the captured single-token step must reproduce the eager launches on every replay,
    # also when eager work and synchronisations happen between replays
    cfg = small_cfg(num_hidden_layers=2)
    dec, _ = make(cfg, "bf16", hip)
    prompt = np.random.Generator(np.random.PCG64(5)).integers(0, cfg.vocab_size, (2, 11)).astype(np.uint32)
    monkeypatch.setenv("RAI_HIP_NO_GRAPH", "1")
    eager, _, _ = dec.generate(prompt, 20)
    monkeypatch.delenv("RAI_HIP_NO_GRAPH")
    for n in (20, 7, 20):
        graph, _, _ = dec.generate(prompt, n)
        assert np.array_equal(graph, eager[:, :n]), f"graph replay differs from eager at n={n}"
        # eager forward + sync between graph uses
        dec.clear_kv_cache()
        _, tok = dec.forward(prompt)
        assert np.array_equal(tok, eager[:, 0])
    dec.close()


def test_prefill_norm_fused_into_split_k_pass_changes_no_bit(hip, monkeypatch):
    """A 96-token prefill goes through the tile GEMM; its dense|fc2 product splits K and the pass over the
    partial sums also writes the next layer's LayerNorm.  Same logits, bit for bit, as with the norm as its own
    launch, and both match the oracle."""
    cfg = small_cfg(num_hidden_layers=3, max_position_embeddings=128)
    ids = np.random.Generator(np.random.PCG64(5)).integers(0, cfg.vocab_size, (1, 96)).astype(np.uint32)
    dec, ref = make(cfg, "bf16", hip, max_batch=1, max_context=128)
    fused, tok = dec.forward(ids)
    monkeypatch.setenv("RAI_HIP_NO_POST_NORM", "1")
    dec2, _ = make(cfg, "bf16", hip, max_batch=1, max_context=128)
    plain, tok2 = dec2.forward(ids)
    monkeypatch.delenv("RAI_HIP_NO_POST_NORM")
    np.testing.assert_array_equal(np.asarray(fused), np.asarray(plain))
    np.testing.assert_array_equal(tok, tok2)
    want = ref.fwd(ids)
    assert_close(fused, want, "bf16", "prefill logits, fused norm")
    check_tokens(tok, want, "bf16")


@pytest.mark.parametrize("hidden,heads,inter", [(2560, 32, 10240), (4096, 32, 4096)])
def test_prefill_norm_fused_at_wide_rows(hip, monkeypatch, hidden, heads, inter):
    """The fused summation + LayerNorm pass at 5 and 8 column groups per lane (rows of 2560 and 4096): bit-identical
    logits to the path with the stand-alone norm."""
    cfg = small_cfg(hidden_size=hidden, num_attention_heads=heads, intermediate_size=inter, num_hidden_layers=2,
                    max_position_embeddings=128, vocab_size=512, partial_rotary_factor=0.25)   # an even rotary_dim
    ids = np.random.Generator(np.random.PCG64(6)).integers(0, cfg.vocab_size, (1, 80)).astype(np.uint32)

    def with_random_vectors(dec):
        # biases and norm parameters away from the 0 / 1 of random_params, so that a dropped one would show
        rng = np.random.Generator(np.random.PCG64(7))
        for name, size in sorted(dec.param_names().items()):
            if name.endswith(".bias") or name.endswith("layernorm.weight"):
                dec.load_param(name, to_storage((0.5 + rng.random(size, dtype=np.float32)) * np.float32(0.1), "bf16"))
        return dec

    dec = with_random_vectors(make(cfg, "bf16", hip, max_batch=1, max_context=128)[0])
    fused, tok = dec.forward(ids)
    del dec
    monkeypatch.setenv("RAI_HIP_NO_POST_NORM", "1")
    dec2 = with_random_vectors(make(cfg, "bf16", hip, max_batch=1, max_context=128)[0])
    plain, tok2 = dec2.forward(ids)
    np.testing.assert_array_equal(np.asarray(fused), np.asarray(plain))
    np.testing.assert_array_equal(tok, tok2)
    assert np.isfinite(np.asarray(fused, dtype=np.float32)).all()


def test_gqa_and_tied_head(hip):
    # num_key_value_heads < heads (repeat_kv phi2.rs:190-200) and tie_word_embeddings
    cfg = small_cfg(num_key_value_heads=2, tie_word_embeddings=True)
    dec, ref = make(cfg, "f32", hip)
    ids = np.random.Generator(np.random.PCG64(4)).integers(0, cfg.vocab_size, (2, 9)).astype(np.uint32)
    logits, _ = dec.forward(ids)
    assert_close(logits, ref.fwd(ids), "f32", "gqa prefill")
    nxt = np.array([[5], [7]], np.uint32)
    logits, _ = dec.forward(nxt)
    assert_close(logits, ref.fwd(nxt), "f32", "gqa decode")
    dec.close()


def test_full_width_single_layer_f32(hip):
    # single Phi-2-width layer: hidden 2560, 32 heads x 80, rotary 32, MLP 10240, 128 tokens,
    # vocab 51200 with a tied head, f32
    cfg = phi2.Config(num_hidden_layers=1, tie_word_embeddings=True, max_position_embeddings=256)
    dec, ref = make(cfg, "f32", hip, max_batch=1, max_context=160, seed=0)
    ids = np.random.Generator(np.random.PCG64(1)).integers(0, cfg.vocab_size, (1, 128)).astype(np.uint32)
    # the hidden state after the layer, [1, 128, 2560] (what DecoderLayer::fwd returns, phi2.rs:293-299), then the
    # argmax over the tied 51200-way head
    hidden, logits, tok = dec.forward_hidden(ids=ids, want_logits=True)
    assert hidden.shape == (1, 128, cfg.hidden_size)
    assert_close(hidden, ref.hidden(ids), "f32", "C0 hidden state after the layer")
    ref.clear_kv_cache()
    want = ref.fwd(ids)
    assert_close(logits, want, "f32", "C0 logits")
    assert tok[0] == np.argmax(want[0])
    # the same through the ordinary entry point
    dec.clear_kv_cache()
    logits2, tok2 = dec.forward(ids)
    np.testing.assert_array_equal(logits2, logits)
    assert tok2[0] == tok[0]
    dec.close()


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_forward_hidden_rows_in_place_of_the_embedding(hip, dt):
    # rows handed in directly give what the same rows give when they come out of the embedding table
    cfg = small_cfg()
    dec, ref = make(cfg, dt, hip)
    ids = np.random.Generator(np.random.PCG64(8)).integers(0, cfg.vocab_size, (2, 11)).astype(np.uint32)
    from oracle import nn as onn
    rows = onn.embedding(ids, ref.p["model.embed_tokens.weight"])
    h_ids, l_ids, t_ids = dec.forward_hidden(ids=ids, want_logits=True)
    dec.clear_kv_cache()
    h_rows, l_rows, t_rows = dec.forward_hidden(hidden_in=to_storage(rows, dt), want_logits=True)
    np.testing.assert_array_equal(h_ids, h_rows)
    np.testing.assert_array_equal(l_ids, l_rows)
    np.testing.assert_array_equal(t_ids, t_rows)
    assert_close(h_ids, ref.hidden(ids), dt, "hidden state of the small model")
    import ctypes as C
    from rai_amd._lib import RaiHipError, call
    st = to_storage(rows, dt)
    dec.clear_kv_cache()
    with pytest.raises(RaiHipError):      # ids and rows at once
        call("rai_hip_decoder_forward_hidden", dec._h, ids.ctypes.data_as(C.POINTER(C.c_uint32)),
             st.ctypes.data_as(C.c_void_p), 2, 11, None, None, None)
    dec.close()


def test_decoder_errors(hip):
    from rai_amd._lib import RaiHipError
    cfg = small_cfg()
    dec, _ = make(cfg, "f32", hip, max_batch=1, max_context=16)
    with pytest.raises(RaiHipError):
        dec.forward(np.zeros((2, 4), np.uint32))            # batch > max_batch
    with pytest.raises(RaiHipError):
        dec.forward(np.zeros((1, 17), np.uint32))           # beyond max_context
    with pytest.raises(RaiHipError):
        dec.forward(np.full((1, 4), cfg.vocab_size, np.uint32))  # id outside the vocabulary
    with pytest.raises(RaiHipError):
        dec.load_param("model.layers.0.nope", np.zeros(4, np.float32))
    dec.close()
