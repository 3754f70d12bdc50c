"""The persistent per-token decode kernel (Phi-2 width, bf16, batch 1): every layer of
a single-token step in one launch, blocks exchanging vectors as tagged packets.  Checked against the CPU oracle
(rai-models/src/llm/phi2.rs restated) and against the launch-per-primitive path of the
same library."""
import numpy as np
import pytest

from oracle import phi2
from tests.test_gpu_phi2 import check_tokens, make
from rai_amd._lib import RaiHipError
from tests.util import assert_close

pytestmark = pytest.mark.gpu


def wide_cfg(**kw):
    # the kernel is specialised for Phi-2's hidden width 2560 = 32 heads x 80; the MLP and the
    # vocabulary are shrunk so that the oracle stays fast
    base = dict(vocab_size=512, hidden_size=2560, intermediate_size=1024, num_hidden_layers=2, num_attention_heads=32,
                max_position_embeddings=128)
    base.update(kw)
    return phi2.Config(**base)


@pytest.mark.parametrize("width", [dict(), dict(hidden_size=2048, partial_rotary_factor=0.5),
                                   dict(num_key_value_heads=8), dict(hidden_size=2048, partial_rotary_factor=0.5,
                                                                     num_key_value_heads=4)])
def test_persistent_step_logits_match_oracle(hip, width):
    # the two widths the kernel is built for: 2560 = 32 x 80 (Phi-2) and 2048 = 32 x 64 (Phi-1 / Phi-1.5), each also
    # with grouped-query attention (repeat_kv, rai-models/src/llm/phi2.rs:190-200)
    cfg = wide_cfg(**width)
    dec, ref = make(cfg, "bf16", hip, max_batch=1, max_context=96)
    ids = np.random.Generator(np.random.PCG64(11)).integers(0, cfg.vocab_size, (1, 21)).astype(np.uint32)
    logits, tok = dec.forward(ids)          # prefill: tile kernels
    want = ref.fwd(ids)
    assert_close(logits, want, "bf16", "prefill logits")
    nxt = np.argmax(want, -1).astype(np.uint32).reshape(1, 1)
    for step in range(8):                   # single-token steps: the persistent kernel
        logits, tok = dec.forward(nxt)
        want = ref.fwd(nxt)
        assert_close(logits, want, "bf16", f"decode step {step}")
        check_tokens(tok, want, "bf16")
        nxt = np.argmax(want, -1).astype(np.uint32).reshape(1, 1)
    assert dec.context_len() == 29
    us, nbytes = dec.time_decode_step(2)     # refused unless the persistent kernel serves this model
    assert us > 0 and nbytes > 0
    dec.close()


def test_persistent_generate_equals_per_primitive_path(hip, monkeypatch):
    cfg = wide_cfg(num_hidden_layers=3)
    prompt = np.random.Generator(np.random.PCG64(12)).integers(0, cfg.vocab_size, (1, 37)).astype(np.uint32)
    monkeypatch.setenv("RAI_HIP_NO_MEGA", "1")
    plain, ref = make(cfg, "bf16", hip, max_batch=1, max_context=96)
    monkeypatch.delenv("RAI_HIP_NO_MEGA")
    mega, _ = make(cfg, "bf16", hip, max_batch=1, max_context=96)
    a, _, _ = plain.generate(prompt, 24)
    b, _, _ = mega.generate(prompt, 24)
    want, logits_all = phi2.greedy_decode(ref, prompt, 24)
    for s in range(24):
        if b[0, s] != want[0, s]:
            check_tokens(b[:, s], logits_all[s], "bf16")  # a near tie in the oracle's own logits
            break
    # graph replays of the persistent step are repeatable
    b2, _, _ = mega.generate(prompt, 24)
    assert np.array_equal(b, b2)
    # and agree with the launch-per-primitive path up to a near tie
    for s in range(24):
        if a[0, s] != b[0, s]:
            check_tokens(b[:, s], logits_all[s], "bf16")
            break
    plain.close()
    mega.close()


def test_lost_packet_times_out_and_reports(hip, monkeypatch):
    """A block whose phase-A packets never arrive: the waves waiting for them give up after the spin
    limit, every wave of the launch still runs to its end, the call returns an error, and the decoder
    works again afterwards.  The condition is forced from the host (a test hook drops the packets and
    the spin limit is made tiny); nothing faults on the device."""
    cfg = wide_cfg()
    monkeypatch.setenv("RAI_HIP_MEGA_PROF", "1")    # the instrumented build of the kernel honours the two hooks
    dec, ref = make(cfg, "bf16", hip, max_batch=1, max_context=96)
    monkeypatch.delenv("RAI_HIP_MEGA_PROF")
    ids = np.random.Generator(np.random.PCG64(13)).integers(0, cfg.vocab_size, (1, 9)).astype(np.uint32)
    one = np.array([[7]], np.uint32)
    dec.forward(ids)
    monkeypatch.setenv("RAI_HIP_MEGA_SPIN_LIMIT", "400")
    monkeypatch.setenv("RAI_HIP_MEGA_TEST_MUTE_BLOCK", "40")
    with pytest.raises(RaiHipError) as e:
        dec.forward(one)
    assert e.value.status == -5 and "timed out" in str(e.value)   # RAI_ERR_HIP
    monkeypatch.delenv("RAI_HIP_MEGA_SPIN_LIMIT")
    monkeypatch.delenv("RAI_HIP_MEGA_TEST_MUTE_BLOCK")
    dec.clear_kv_cache()
    logits, _ = dec.forward(ids)
    assert_close(logits, ref.fwd(ids), "bf16", "prefill after the fault")
    logits, tok = dec.forward(one)
    want = ref.fwd(one)
    assert_close(logits, want, "bf16", "persistent step after the fault")
    check_tokens(tok, want, "bf16")
    dec.close()


def test_persistent_step_long_context_takes_several_prefetch_passes(hip):
    """Beyond ~612 cached positions one head's values, and beyond ~665 its keys, no longer fit the registers the
    attention blocks prefetch them into, so the kernel fetches them in several passes; the benchmark's last
    tokens run there."""
    cfg = wide_cfg(max_position_embeddings=768)
    dec, ref = make(cfg, "bf16", hip, max_batch=1, max_context=704)
    ids = np.random.Generator(np.random.PCG64(14)).integers(0, cfg.vocab_size, (1, 660)).astype(np.uint32)
    logits, _ = dec.forward(ids)
    want = ref.fwd(ids)
    assert_close(logits, want, "bf16", "prefill logits")
    nxt = np.argmax(want, -1).astype(np.uint32).reshape(1, 1)
    for step in range(10):                   # context 660..669: two passes over the values, from 666 on also over the keys
        logits, tok = dec.forward(nxt)
        want = ref.fwd(nxt)
        assert_close(logits, want, "bf16", f"decode step at context {660 + step}")
        check_tokens(tok, want, "bf16")
        nxt = np.argmax(want, -1).astype(np.uint32).reshape(1, 1)
    assert dec.context_len() == 670
    dec.close()


def test_persistent_step_with_and_without_lds_staged_weights(hip, monkeypatch):
    """At Phi-2's real MLP width every stream wave keeps the eight weight tiles behind its register ring in LDS
    (fetched while it waits for its inputs).  The tiles are consumed in the same order either way, so the logits
    are the same bits with the staging switched off, and both match the oracle."""
    cfg = wide_cfg(intermediate_size=10240)
    ids = np.random.Generator(np.random.PCG64(15)).integers(0, cfg.vocab_size, (1, 19)).astype(np.uint32)
    dec, ref = make(cfg, "bf16", hip, max_batch=1, max_context=96)
    want = ref.fwd(ids)
    first = np.argmax(want, -1).astype(np.uint32).reshape(1, 1)
    runs = []
    for off in ("0", "1"):
        monkeypatch.setenv("RAI_HIP_MEGA_NO_STAGE", off)     # read per launch
        dec.clear_kv_cache()
        dec.forward(ids)
        nxt, out = first, []
        for step in range(6):
            logits, tok = dec.forward(nxt)
            out.append(logits.copy())
            nxt = tok.reshape(1, 1).astype(np.uint32)
        runs.append(out)
    monkeypatch.delenv("RAI_HIP_MEGA_NO_STAGE")
    nxt = first
    for step in range(6):
        assert np.array_equal(runs[0][step], runs[1][step]), f"step {step}: staged and unstaged logits differ"
        want = ref.fwd(nxt)
        assert_close(runs[0][step], want, "bf16", f"decode step {step}")
        check_tokens(np.argmax(runs[0][step], -1), want, "bf16")
        nxt = np.argmax(runs[0][step], -1).astype(np.uint32).reshape(1, 1)
    dec.close()


@pytest.mark.parametrize("vocab", [16384, 32768])
def test_greedy_choice_takes_the_first_maximum_and_passes_over_nans(hip, vocab):
    # The token choice behind the head product (rai-models/examples/phi2/src/main.rs:76-87 takes the argmax of the
    # last logits row), at both of its forms: one block scanning the row, and, from 32768 logits on, shares of the row
    # scanned by many blocks and merged.  Ties and NaNs are planted through the head's bias: rows 100 and 200 (different
    # shares) and 301, 302 (neighbours) share the largest logit; a NaN at row 7 is passed over; a NaN at row 0 wins
    # (a scan that starts from element 0 and replaces on a strict comparison never leaves it).
    from tests.test_gpu_phi2 import to_storage
    cfg = wide_cfg(vocab_size=vocab, intermediate_size=512)
    prompt = np.random.Generator(np.random.PCG64(31)).integers(0, cfg.vocab_size, (1, 19)).astype(np.uint32)
    dec, ref = make(cfg, "bf16", hip, max_batch=1, max_context=96)
    logits, tok = dec.forward(prompt)
    assert tok[0] == int(np.argmax(logits[0]))
    for _ in range(3):   # single-token steps: the persistent kernel, then the same head and choice
        logits, tok = dec.forward(np.array([[tok[0]]], np.uint32))
        assert tok[0] == int(np.argmax(logits[0]))
    params = phi2.random_params(cfg, "bf16", seed=0)
    w, b = params["lm_head.weight"].copy(), params["lm_head.bias"].copy()
    for r in (100, 200, 301, 302):
        w[r] = 0
        b[r] = 64.0
    b[7] = np.nan
    dec.load_param("lm_head.weight", to_storage(w, "bf16"))
    dec.load_param("lm_head.bias", to_storage(b, "bf16"))
    dec.clear_kv_cache()
    logits, tok = dec.forward(prompt)
    assert np.isnan(logits[0, 7]) and logits[0, 100] == logits[0, 200] == logits[0, 301] == 64.0
    assert np.nanmax(logits[0]) == 64.0
    assert tok[0] == 100
    b[100] = 0.0
    b[200] = 0.0
    dec.load_param("lm_head.bias", to_storage(b, "bf16"))
    dec.clear_kv_cache()
    assert dec.forward(prompt)[1][0] == 301
    b[0] = np.nan
    dec.load_param("lm_head.bias", to_storage(b, "bf16"))
    dec.clear_kv_cache()
    assert dec.forward(prompt)[1][0] == 0
    dec.close()


@pytest.mark.parametrize("width", [dict(), dict(hidden_size=2048, partial_rotary_factor=0.5, vocab_size=8192),
                                   dict(tie_word_embeddings=True, vocab_size=4096)])
def test_head_kernel_against_norm_head_and_choice_as_three_launches(hip, monkeypatch, width):
    # One sequence, greedy: the final LayerNorm, the head product and the token choice run as one launch (every block
    # normalises once, streams its rows of the head like the step kernel does, and the block that finishes last picks
    # among the blocks' best rows).  Against the three launches it replaces: logits to the bf16 bar (the rows are summed
    # in a different order), the same tokens up to a near tie, the same device-side counters; graph replays repeat.
    # (both widths the kernel is built for; a head tied to the embedding matrix has no bias)
    cfg = wide_cfg(**{**dict(vocab_size=16384, intermediate_size=512, num_hidden_layers=3), **width})
    prompt = np.random.Generator(np.random.PCG64(41)).integers(0, cfg.vocab_size, (1, 23)).astype(np.uint32)
    monkeypatch.setenv("RAI_HIP_NO_HEAD_KERNEL", "1")
    apart, ref = make(cfg, "bf16", hip, max_batch=1, max_context=96)
    la, ta = apart.forward(prompt)
    ctx_forward = apart.context_len()
    ga, _, _ = apart.generate(prompt, 20)
    ctx_generate = apart.context_len()
    monkeypatch.delenv("RAI_HIP_NO_HEAD_KERNEL")
    one, _ = make(cfg, "bf16", hip, max_batch=1, max_context=96)
    lo, to = one.forward(prompt)          # prefill, then the head kernel on the last row
    want = ref.fwd(prompt)
    assert_close(lo, want, "bf16", "prefill logits through the head kernel")
    assert_close(lo, la, "bf16", "head kernel vs three launches")
    assert to[0] == int(np.argmax(lo[0]))
    assert one.context_len() == ctx_forward
    nxt = np.argmax(want, -1).astype(np.uint32).reshape(1, 1)
    for step in range(4):                 # single-token steps: step kernel + head kernel
        lo, to = one.forward(nxt)
        want = ref.fwd(nxt)
        assert_close(lo, want, "bf16", f"decode step {step}")
        assert to[0] == int(np.argmax(lo[0]))
        check_tokens(to, want, "bf16")
        nxt = np.argmax(want, -1).astype(np.uint32).reshape(1, 1)
    go, _, _ = one.generate(prompt, 20)
    assert one.context_len() == ctx_generate
    assert np.array_equal(go, one.generate(prompt, 20)[0])   # graph replays
    wanted, logits_all = phi2.greedy_decode(ref, prompt, 20)
    for s in range(20):
        if go[0, s] != ga[0, s] or go[0, s] != wanted[0, s]:
            check_tokens(go[:, s], logits_all[s], "bf16")   # a near tie in the oracle's own logits
            break
    apart.close()
    one.close()
