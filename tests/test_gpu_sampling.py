"""The example loop's token choice on the device (repeat penalty over the last tokens, last maximum
under f32 total order; examples/phi2/src/main.rs:29-50,72-95) against oracle/sampling.py, through the
C ABI: the primitive bit-exactly, the generate loop token by token."""
import numpy as np
import pytest

from oracle import phi2, sampling
from oracle.dtypes import rnd, to_storage
from rai_amd.hip import HipTensor
from tests import test_gpu_phi2 as tp
from tests import test_gpu_qwen2_gemma as tq

pytestmark = pytest.mark.gpu


def f32_bits(b):
    return np.array([b], np.uint32).view(np.float32)[0]


def device_choice(hip, rows_f32, dt, context, penalty):
    from rai_amd import ops
    lg = HipTensor.from_storage(to_storage(rows_f32, dt), dt)
    ctx = None if context is None else HipTensor.from_storage(np.ascontiguousarray(context, np.uint32), "u32")
    return ops.sample_argmax(lg, ctx, penalty).to_storage()


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("vocab", [1, 7, 33, 1000, 4099, 51200])
def test_sample_argmax_bit_exact(hip, dt, vocab):
    rng = np.random.Generator(np.random.PCG64(vocab))
    rows = 5
    x = rnd(rng.standard_normal((rows, vocab)).astype(np.float32) * np.float32(3), dt)
    x[1] = np.round(x[1])                                  # many exact ties
    x[2, rng.integers(0, vocab, 3)] = np.float32(x[2].max())   # the maximum several times: the last one wins
    if vocab >= 7:
        x[3, :6] = [0.0, -0.0, np.inf, np.inf, -np.inf, 0.0]
        x[4, 2] = np.nan
        x[4, 5] = f32_bits(0xFFC00000)                     # a negative NaN is the smallest value
    for penalty, n_ctx in [(1.1, 64), (2.0, 5), (1.0, 9), (0.9, 64), (1.1, 0)]:
        ctx = rng.integers(0, vocab + 3, (rows, n_ctx)).astype(np.uint32)   # duplicates and ids outside the vocabulary
        if n_ctx:
            ctx[2, 0] = int(np.argmax(x[2]))               # penalise a current maximum
        got = device_choice(hip, x, dt, ctx if n_ctx else None, penalty)
        for r in range(rows):
            want, _ = sampling.choose(x[r], list(ctx[r]), penalty, n_ctx)
            assert got[r] == want, f"row {r} penalty {penalty} ctx {n_ctx}: {got[r]} vs {want}"


def test_sample_argmax_rejects_bad_arguments(hip):
    from rai_amd import ops
    from rai_amd._lib import RaiHipError
    lg = HipTensor.from_storage(np.zeros((2, 8), np.float32), "f32")
    with pytest.raises(RaiHipError):
        ops.sample_argmax(lg, HipTensor.from_storage(np.zeros((3, 4), np.uint32), "u32"), 1.1)   # rows differ
    with pytest.raises(RaiHipError):
        ops.sample_argmax(lg, None, float("nan"))
    with pytest.raises(RaiHipError):
        ops.sample_argmax(HipTensor.from_storage(np.zeros((2, 8), np.uint32), "u32"), None, 1.1)


def compare_rows(toks, n_gen, want, want_gen, rows_all, dt):
    """Token by token per sequence; at the first difference the oracle's own penalised logits must hold a
    near tie between the two tokens (then the rest of that sequence is not comparable)."""
    tol_rel = {"f32": 1e-4, "bf16": 2e-2}[dt]
    exact = 0
    for b in range(toks.shape[0]):
        for s in range(toks.shape[1]):
            if toks[b, s] != want[b, s]:
                row = rows_all[s][b].astype(np.float64)
                gap = row[want[b, s]] - row[toks[b, s]]
                tol = tol_rel * np.max(np.abs(row[np.isfinite(row)]))
                assert 0 <= gap <= tol, f"seq {b} step {s}: token {toks[b, s]} vs {want[b, s]}, gap {gap:.3e} > {tol:.3e}"
                break
        else:
            exact += 1
            assert n_gen[b] == want_gen[b]
    return exact


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_phi2_generate_sampled_matches_oracle(hip, dt):
    cfg = tp.small_cfg()
    dec, ref = tp.make(cfg, dt, hip)
    prompt = np.random.Generator(np.random.PCG64(21)).integers(0, cfg.vocab_size, (2, 9)).astype(np.uint32)
    n_new = 20
    want, want_gen, rows_all = sampling.sampled_decode(ref, prompt, n_new, 1.5, 4)
    greedy, _ = phi2.greedy_decode(ref, prompt, n_new)
    assert not np.array_equal(want, greedy)                # the penalty changes the sequence in this case
    eos = int(want[0, 7])
    _, want_gen, _ = sampling.sampled_decode(ref, prompt, n_new, 1.5, 4, eos_token=eos)
    toks, n_gen, _, _ = dec.generate_sampled(prompt, n_new, 1.5, 4, eos_token=eos)
    assert compare_rows(toks, n_gen, want, want_gen, rows_all, dt) >= 1
    # replays (captured graphs for bf16) repeat themselves, and the greedy entry point is unaffected afterwards
    toks2, _, _, _ = dec.generate_sampled(prompt, n_new, 1.5, 4)
    assert np.array_equal(toks, toks2)
    g, _, _ = dec.generate(prompt, n_new)
    g2, _, _ = dec.generate(prompt, n_new)
    assert np.array_equal(g, g2) and not np.array_equal(g, toks)
    # other parameters recapture the step graphs
    want3, gen3, rows3 = sampling.sampled_decode(ref, prompt, n_new, 1.1, 64)
    toks3, n3, _, _ = dec.generate_sampled(prompt, n_new)   # the example's defaults: 1.10 over 64 tokens
    compare_rows(toks3, n3, want3, gen3, rows3, dt)
    want4, gen4, rows4 = sampling.sampled_decode(ref, prompt, n_new, 0.5, 64)   # below 1: no penalty, last maximum
    toks4, n4, _, _ = dec.generate_sampled(prompt, n_new, 0.5, 64)
    compare_rows(toks4, n4, want4, gen4, rows4, dt)
    dec.close()


@pytest.mark.parametrize("arch", ["qwen2", "gemma"])
def test_qwen2_gemma_generate_sampled_matches_oracle(hip, arch):
    cfg = tq.CFGS[arch]()
    dec, ref = tq.make(cfg, "bf16")
    prompt = np.random.Generator(np.random.PCG64(22)).integers(0, cfg.vocab_size, (2, 12)).astype(np.uint32)
    want, want_gen, rows_all = sampling.sampled_decode(ref, prompt, 16, 1.3, 8)
    toks, n_gen, _, _ = dec.generate_sampled(prompt, 16, 1.3, 8)
    compare_rows(toks, n_gen, want, want_gen, rows_all, "bf16")
    dec.close()


def test_persistent_kernel_with_sampled_choice(hip):
    from tests.test_gpu_phi2_persistent import wide_cfg
    cfg = wide_cfg()
    dec, ref = tp.make(cfg, "bf16", hip, max_batch=1, max_context=96)
    prompt = np.random.Generator(np.random.PCG64(23)).integers(0, cfg.vocab_size, (1, 30)).astype(np.uint32)
    want, want_gen, rows_all = sampling.sampled_decode(ref, prompt, 24, 1.1, 64)
    toks, n_gen, _, _ = dec.generate_sampled(prompt, 24)
    compare_rows(toks, n_gen, want, want_gen, rows_all, "bf16")
    dec.close()
