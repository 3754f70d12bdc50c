"""Pins oracle/sampling.py (the example loop's token choice, examples/phi2/src/main.rs:29-50)
without the oracle's own formulas: sample_argmax against a pure-Python `max_by` over Rust's
documented f32::total_cmp (compare the bit patterns as i32 after `bits ^= ((bits >> 31) as u32 >> 1)`),
apply_repeat_penalty against hand-computed rows and an element loop."""
import struct

import numpy as np

from oracle import sampling


def rust_total_cmp_key(x):
    """f32::total_cmp as the standard library documents it: reinterpret as i32, flip the low 31 bits of
    negative patterns (`bits ^= ((bits >> 31) as u32 >> 1) as i32`), compare as signed integers."""
    bits = struct.unpack("<i", struct.pack("<f", x))[0]
    return bits ^ 0x7FFFFFFF if bits < 0 else bits


def rust_max_by_last(row):
    best = None
    for i, v in enumerate(row):
        k = rust_total_cmp_key(float(v))
        if best is None or k >= best[0]:         # max_by keeps the later of two equal elements
            best = (k, i)
    return best[1]


def f32_from_bits(b):
    return np.array([b], np.uint32).view(np.float32)[0]


def test_total_cmp_key_orders_the_special_values():
    neg_nan, pos_nan = f32_from_bits(0xFFC00000), f32_from_bits(0x7FC00000)
    ladder = [neg_nan, -np.inf, -3.0e38, -1.0, -1e-45, -0.0, 0.0, 1e-45, 1.0, 3.0e38, np.inf, pos_nan]
    keys = sampling.total_order_key(np.array(ladder, np.float32)).astype(np.int64)
    assert np.all(np.diff(keys) > 0)
    rk = [rust_total_cmp_key(float(np.float32(v))) for v in ladder]
    assert all(a < b for a, b in zip(rk, rk[1:]))


def test_sample_argmax_known_answers():
    assert sampling.sample_argmax(np.array([1.0, 3.0, 2.0], np.float32)) == 1
    assert sampling.sample_argmax(np.array([3.0, 1.0, 3.0, 2.0, 3.0, 0.0], np.float32)) == 4      # last maximum
    assert sampling.sample_argmax(np.array([0.0, -0.0, 0.0, -0.0], np.float32)) == 2              # +0 above -0
    assert sampling.sample_argmax(np.array([-0.0, -0.0], np.float32)) == 1
    assert sampling.sample_argmax(np.array([np.inf, np.nan, 1.0], np.float32)) == 1               # +NaN is the top
    assert sampling.sample_argmax(np.array([f32_from_bits(0xFFC00000), -np.inf], np.float32)) == 1  # -NaN is the bottom
    assert sampling.sample_argmax(np.array([7.0], np.float32)) == 0


def test_sample_argmax_matches_rust_max_by_on_random_rows():
    rng = np.random.Generator(np.random.PCG64(5))
    specials = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1.0, 1.0, -1.0], np.float32)
    for trial in range(200):
        n = int(rng.integers(1, 40))
        row = rng.integers(-3, 4, n).astype(np.float32)          # many ties
        k = int(rng.integers(0, min(n, 4) + 1))
        row[rng.integers(0, n, k)] = rng.choice(specials, k)
        if trial % 7 == 0:
            row[int(rng.integers(0, n))] = f32_from_bits(0xFFC00001)
        assert int(sampling.sample_argmax(row)) == rust_max_by_last(row), row


def test_apply_repeat_penalty_known_answers():
    row = np.array([2.2, -1.0, 0.0, -0.0, 5.5, -3.0], np.float32)
    out = sampling.apply_repeat_penalty(row, 1.1, np.array([0, 1, 1, 3, 5, 0, 99], np.uint32))   # repeats and an id outside the row
    p = np.float32(1.1)
    want = np.array([np.float32(2.2) / p, np.float32(-1.0) * p, 0.0, np.float32(-0.0) / p, 5.5, np.float32(-3.0) * p], np.float32)
    assert np.array_equal(out.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(row, np.array([2.2, -1.0, 0.0, -0.0, 5.5, -3.0], np.float32))          # input untouched
    # NaN is "not >= 0": multiplied, stays NaN; +inf / p stays +inf
    out = sampling.apply_repeat_penalty(np.array([np.nan, np.inf, -np.inf], np.float32), 1.1, [0, 1, 2])
    assert np.isnan(out[0]) and out[1] == np.inf and out[2] == -np.inf


def test_apply_repeat_penalty_matches_element_loop():
    rng = np.random.Generator(np.random.PCG64(6))
    for _ in range(50):
        n = int(rng.integers(1, 64))
        row = rng.standard_normal(n).astype(np.float32) * np.float32(4)
        ctx = rng.integers(0, n + 5, int(rng.integers(0, 80))).astype(np.uint32)
        want = row.copy()
        seen = set(int(t) for t in ctx)
        for i in range(n):                                       # main.rs:41-49 as written
            if i in seen:
                want[i] = want[i] / np.float32(1.3) if want[i] >= 0 else want[i] * np.float32(1.3)
        got = sampling.apply_repeat_penalty(row, 1.3, ctx)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_choose_window_and_skip_rule():
    row = np.array([1.0, 1.05, 0.5], np.float32)
    tok, pen = sampling.choose(row, [2, 2, 1, 0], 1.1, 2)
    assert tok == 1 and pen[0] < pen[1] and pen[2] == np.float32(0.5)   # window [1, 0]: both penalised, 1.05/1.1 > 1/1.1
    tok, _ = sampling.choose(row, [1, 2, 2], 1.1, 2)
    assert tok == 1                              # token 1 fell out of the window [2, 2]
    tok, _ = sampling.choose(row, [0, 1], 1.1, 2)
    assert tok == 1
    tok, _ = sampling.choose(row, [1], 1.1, 64)
    assert tok == 0                              # 1.05 / 1.1 = 0.954 < 1.0
    tok, _ = sampling.choose(row, [1], 0.5, 64)
    assert tok == 1                              # penalty below 1 is skipped (main.rs:79)


def test_sampled_decode_stops_where_the_example_would():
    class Fixed:
        def __init__(self): self.t = 0
        def clear_kv_cache(self): self.t = 0
        def fwd(self, ids):
            self.t += 1
            row = np.zeros((ids.shape[0], 6), np.float32)
            row[:, self.t % 6] = 5.0
            return row
    toks, n_gen, rows = sampling.sampled_decode(Fixed(), np.array([[0, 1]], np.uint32), 5, 1.1, 64, eos_token=3)
    assert toks.tolist() == [[1, 2, 3, 4, 5]] and n_gen.tolist() == [3] and len(rows) == 5
    _, n_gen, _ = sampling.sampled_decode(Fixed(), np.array([[0, 1]], np.uint32), 5, 1.1, 64, eos_token=None)
    assert n_gen.tolist() == [5]
