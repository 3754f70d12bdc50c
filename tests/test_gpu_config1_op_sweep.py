"""The primitive sweep at its stated shapes, bf16 and f32, HIP path against the CPU oracle through the C ABI:
matmul [4096,2560] x [2560,10240] (N(0,1) operands; the row-major right operand of rai's MatMul and the
transposed-weight form rai-nn's Linear produces), softmax over the last dim of [32,128,2048] (N(0,3) logits),
LayerNorm and RMSNorm over [4096,2560], RoPE on [1,32,2048,80] with rotary dim 32 and theta 10000,
index_select of 4096 uniform ids from a [51200,2560] table, argmax over [64,51200].

The second half pins every tile shape of the bf16 MFMA GEMM (selected per call through RAI_HIP_GEMM_TILE) on ragged
shapes with every epilogue the decoders use: two biases, activation from a column on, residual, two outputs,
gated MLP, K split over blocks.
"""
import numpy as np
import pytest

from oracle import nn as onn
from oracle import ops as oo
from oracle import phi2
from oracle.dtypes import rnd
from tests.util import assert_close, assert_close_elem, down, rand, up

pytestmark = pytest.mark.gpu

DTS = ["bf16", "f32"]


@pytest.fixture(scope="module")
def R(hip):
    from rai_amd import ops
    return ops


def rng(seed):
    return np.random.Generator(np.random.PCG64(seed))


def gemm_elem_check(got, want, dt, k, what):
    """Beyond the tensor-relative bar: every element within two roundings of the storage dtype of the oracle's value,
    plus the noise a different f32 summation order may add (~sqrt(K) * eps_f32 * the typical product)."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    ulp = {"bf16": 2.0 ** -8, "f32": 2.0 ** -23}[dt]
    noise = 8.0 * np.sqrt(k) * 2.0 ** -24 * float(np.sqrt(np.mean(want * want)) + 1e-30)
    err = np.abs(got - want)
    bound = 2.0 * ulp * np.abs(want) + noise
    bad = err > bound
    assert not bad.any(), f"{what}: {bad.sum()} of {err.size} elements beyond two {dt} roundings (worst {err.max():.3e})"


# ------------------------------------------------------------------ the sweep at its stated shapes
@pytest.mark.parametrize("dt", DTS)
def test_matmul_4096x2560_by_2560x10240(R, dt):
    g = rng(101)
    a, b = rand(g, (4096, 2560), dt), rand(g, (2560, 10240), dt)
    want = oo.matmul(a, b, dt)
    xa, xb = up(a, dt), up(b, dt)
    got = down(R.matmul(xa, xb))                                   # MatMul with a row-major [K, N] right operand
    assert_close(got, want, dt, "matmul NN")
    gemm_elem_check(got, want, dt, 2560, "matmul NN")
    # rai-nn Linear: x @ W.broadcast_left().t() with W [N, K]  (rai-nn/src/linear.rs:59-69)
    w = up(np.ascontiguousarray(b.T), dt)
    got = down(R.matmul(xa.reshape((1, 4096, 2560)), w.broadcast_to((1, 10240, 2560)).transpose(1, 2)))[0]
    assert_close(got, want, dt, "matmul NT (Linear layout)")
    gemm_elem_check(got, want, dt, 2560, "matmul NT")
    got = down(R.linear(xa, w))
    assert_close(got, want, dt, "linear")
    gemm_elem_check(got, want, dt, 2560, "linear")


@pytest.mark.parametrize("dt", DTS)
def test_softmax_32x128x2048(R, dt):
    a = rand(rng(102), (32, 128, 2048), dt, 3.0)
    got = down(R.softmax(up(a, dt), -1))
    want = oo.softmax(a, -1, dt)
    assert_close(got, want, dt, "softmax", scale=1.0 if dt == "f32" else None)
    if dt == "f32":
        # probabilities span many decades: each one must also be right relative to itself.  (Not for bf16: the
        # reference chain rounds x - max to bf16 before the exponential, which alone moves small probabilities by
        # several per cent; the kernel rounds once, at the end.)
        assert_close_elem(got, want, dt, "softmax per element", atol=1e-30)
    assert_close(got.astype(np.float64).sum(-1), np.ones((32, 128)), dt, "rows sum to 1", scale=2.0)


@pytest.mark.parametrize("dt", DTS)
def test_layer_norm_rms_norm_4096x2560(R, dt):
    g = rng(103)
    x = rand(g, (4096, 2560), dt, 1.5)
    w = rnd(1.0 + 0.1 * g.standard_normal(2560).astype(np.float32), dt)
    b = rand(g, (2560,), dt, 0.1)
    xd, wd, bd = up(x, dt), up(w, dt), up(b, dt)
    assert_close(down(R.layer_norm(xd, wd, bd, 1e-5)), onn.layer_norm(x, w, b, 1e-5, dt), dt, "LayerNorm")
    assert_close(down(R.rms_norm(xd, wd, 1e-6)), onn.rms_norm(x, w, 1e-6, dt), dt, "RMSNorm")
    w0 = rnd(w - 1.0, dt)
    assert_close(down(R.rms_norm(xd, up(w0, dt), 1e-6, True)), onn.gemma_rms_norm(x, w0, 1e-6, dt), dt, "RMSNorm (1+w)")
    if dt == "f32":   # textbook properties at this size: unit weight, zero bias -> zero mean, unit variance rows
        y = down(R.layer_norm(xd, None, None, 1e-5)).astype(np.float64)
        assert np.abs(y.mean(-1)).max() < 1e-5 and np.abs(y.var(-1) - 1).max() < 1e-3


@pytest.mark.parametrize("dt", DTS)
def test_rope_1x32x2048x80_rot32(R, dt):
    cfg = phi2.Config(max_position_embeddings=2048)          # rotary dim 32 of 80, theta 10000
    sin, cos = phi2.rotary_tables(cfg, dt)
    x = rand(rng(104), (1, 32, 2048, 80), dt)
    want = phi2.rotary(x, sin, cos, cfg.rotary_dim, 0, dt)
    got = down(R.rope(up(x, dt), up(cos, dt), up(sin, dt), cfg.rotary_dim, 0))
    assert_close_elem(got, want, dt, "rope", atol=1e-6 if dt == "f32" else 1e-3)
    assert np.array_equal(got[..., 32:], x[..., 32:]), "pass-through dims must be copied bit for bit"
    assert np.array_equal(got[:, :, 0, :], x[:, :, 0, :]), "position 0 is the identity"
    # the layout the models hand over: [B,S,H,D] storage viewed as [B,H,S,D]
    xt = up(np.ascontiguousarray(np.swapaxes(x, 1, 2)), dt).transpose(1, 2)
    assert np.array_equal(down(R.rope(xt, up(cos, dt), up(sin, dt), cfg.rotary_dim, 0)), got)
    if dt == "f32":   # device-built tables against the reference chain, and the rotation preserves pair norms
        c32, s32 = R.rope_tables(2048, 32, 10000.0, "f32")
        assert_close(down(c32), cos, "f32", "cos table")
        assert_close(down(s32), sin, "f32", "sin table")
        n_in = x[..., :16] ** 2 + x[..., 16:32] ** 2
        n_out = got[..., :16].astype(np.float64) ** 2 + got[..., 16:32].astype(np.float64) ** 2
        assert np.allclose(n_in, n_out, rtol=1e-4, atol=1e-6)


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("idt", ["u32", "i64"])
def test_index_select_4096_of_51200x2560(R, dt, idt):
    g = rng(105)
    table = rand(g, (51200, 2560), dt)
    ids = g.integers(0, 51200, 4096).astype({"u32": np.uint32, "i64": np.int64}[idt])
    ids[:3] = [0, 51199, 51199]
    t = up(table, dt)
    got = R.index_select(t, 0, up(ids, idt)).to_storage()
    assert np.array_equal(got, t.to_storage()[ids.astype(np.int64)])           # bit-exact rows
    assert np.array_equal(down(R.index_select(t, 0, up(ids, idt))), oo.index_select(table, 0, ids))
    assert R.index_errors() == 0


@pytest.mark.parametrize("dt", DTS)
def test_argmax_64x51200(R, dt):
    g = rng(106)
    a = rand(g, (64, 51200), dt)                      # N(0,1) logits: bf16 rounding alone produces exact ties
    a[1, 51199] = 9.0                                  # maximum in the last element
    a[2, 0] = 9.0                                      # in the first
    a[3, 777] = a[3, 40000] = 9.0                      # an exact tie: the first index wins
    got = down(R.argmax(up(a, dt), -1))
    want = oo.argmax(a, -1)
    assert got.dtype == np.uint32 and np.array_equal(got, want)
    assert list(got[1:4]) == [51199, 0, 777]
    assert np.array_equal(down(R.argmax(up(a, dt), 1, True)), oo.argmax(a, 1, True))
    assert np.array_equal(down(R.argmin(up(a, dt), -1)), oo.argmin(a, -1))


# ------------------------------------------------------------------ every tile of the bf16 MFMA GEMM
TILES = ["128x128", "128x128k64", "256x192", "256x128", "256x256", "256x256x8w", "classic"]
K64_TILES = ("128x128k64", "256x192")      # two LDS stages of K 64: refused unless K % 64 == 0


def packed_case(g, m, n, k, scale=0.05):
    x, w = rand(g, (m, k), "bf16"), rand(g, (n, k), "bf16", scale)
    b1, b2, r = rand(g, (n,), "bf16"), rand(g, (n,), "bf16"), rand(g, (m, n), "bf16")
    return x, w, b1, b2, r


@pytest.mark.parametrize("tile", TILES)
@pytest.mark.parametrize("m,n,k", [(1000, 1111, 2560), (300, 520, 64), (260, 264, 32), (513, 2568, 1024)])
def test_gemm_tile_plain_and_fused_epilogue(R, monkeypatch, tile, m, n, k):
    if tile in K64_TILES and k % 64:
        pytest.skip("K tiles of 64 need K % 64 == 0")
    monkeypatch.setenv("RAI_HIP_GEMM_TILE", tile)      # read per call by the tile dispatcher
    dt = "bf16"
    x, w, b1, _, r = packed_case(rng(110), m, n, k)
    xd, wd = up(x, dt), up(w, dt)
    lin = onn.linear(x, w, None, dt)
    got = down(R.linear(xd, wd))
    assert_close(got, lin, dt, f"{tile} linear {m}x{n}x{k}")
    gemm_elem_check(got, lin, dt, k, f"{tile} linear {m}x{n}x{k}")
    want = oo.add(onn.new_gelu(onn.linear(x, w, b1, dt), dt), r, dt)
    got = down(R.linear(xd, wd, up(b1, dt), "new_gelu", up(r, dt)))
    assert_close(got, want, dt, f"{tile} linear + bias + new_gelu + residual {m}x{n}x{k}")


@pytest.mark.parametrize("tile", TILES)
@pytest.mark.parametrize("k_splits,n1", [(0, 312), (3, 312), (5, 312), (0, 301), (2, 301)])
def test_gemm_tile_partial_activation_two_outputs(R, monkeypatch, tile, k_splits, n1):
    # the q|k|v|fc1 product of the Phi-2 block: one weight matrix, columns [0, n1) are q|k|v (no activation), the
    # rest is fc1 with gelu_new, written to a second tensor (rai-models/src/llm/phi2.rs:99-101,202-206)
    monkeypatch.setenv("RAI_HIP_GEMM_TILE", tile)
    dt, m, n, k = "bf16", 700, 1336, 640     # n1 = 301: outputs whose rows are not 16-byte aligned
    x, w, b1, _, _ = packed_case(rng(111), m, n, k)
    o1, o2 = R.linear_packed(up(x, dt), up(w, dt), bias=up(b1, dt), act="new_gelu", act_from=n1, n1=n1,
                             k_splits=k_splits)
    y = onn.linear(x, w, b1, dt)
    assert_close(down(o1), y[:, :n1], dt, f"{tile} splits {k_splits}: q|k|v columns")
    assert_close(down(o2), onn.new_gelu(y[:, n1:], dt), dt, f"{tile} splits {k_splits}: fc1 columns")


@pytest.mark.parametrize("tile", TILES)
@pytest.mark.parametrize("k_splits", [0, 4])
def test_gemm_tile_sum_of_two_linears_plus_residual(R, monkeypatch, tile, k_splits):
    # dense(attn) + fc2(act) + x of the Phi-2 block as one contraction over the concatenated inputs, both biases
    # added (rai-models/src/llm/phi2.rs:293-299)
    monkeypatch.setenv("RAI_HIP_GEMM_TILE", tile)
    dt, m, n, k1, k2 = "bf16", 515, 776, 256, 1024
    x, w, b1, b2, r = packed_case(rng(112), m, n, k1 + k2)
    got = down(R.linear_packed(up(x, dt), up(w, dt), bias=up(b1, dt), bias2=up(b2, dt), residual=up(r, dt),
                               k_splits=k_splits))
    attn = onn.linear(x[:, :k1], w[:, :k1], b1, dt)
    mlp = onn.linear(x[:, k1:], w[:, k1:], b2, dt)
    want = oo.add(oo.add(attn, mlp, dt), r, dt)
    assert_close(got, want, dt, f"{tile} splits {k_splits}: dense + fc2 + residual")


@pytest.mark.parametrize("tile", TILES)
@pytest.mark.parametrize("act", ["silu", "gelu"])
@pytest.mark.parametrize("k_splits", [0, 3])
def test_gemm_tile_gated_mlp(R, monkeypatch, tile, act, k_splits):
    # act(gate(x)) * up(x) with the gate and up rows interleaved (rai-models/src/llm/qwen2.rs:100-104)
    monkeypatch.setenv("RAI_HIP_GEMM_TILE", tile)
    dt, m, i, k = "bf16", 530, 552, 512
    g = rng(113)
    x, wg, wu = rand(g, (m, k), dt), rand(g, (i, k), dt, 0.05), rand(g, (i, k), dt, 0.05)
    w = np.empty((2 * i, k), np.float32)
    w[0::2], w[1::2] = wg, wu
    got = down(R.linear_packed(up(x, dt), up(w, dt), act=act, glu=True, k_splits=k_splits))
    want = oo.mul(onn.activation(act)(onn.linear(x, wg, None, dt), dt), onn.linear(x, wu, None, dt), dt)
    assert_close(got, want, dt, f"{tile} splits {k_splits}: {act}(gate) * up")


# Stream-K form of the eight-wave 256 x 256 tile: the K tiles of the last, partial round of tiles are dealt out evenly
# over the CUs and the shares of a tile are summed by whichever block finishes last.  Shapes: 156 tiles (no whole
# round; two or three shares per tile), 180 tiles at K = 512, 324 tiles (one whole round joins the shared part), 720
# tiles (two whole rounds follow the shared part); all ragged in M and N.
STREAMK_SHAPES = [(3000, 3100, 2560), (2100, 5000, 512), (4400, 4600, 320), (5000, 9000, 256)]


# "streamk64" / "256x256x8wk64": the same with K tiles of 64 (two LDS stages, 128-byte rows), K % 64 == 0
@pytest.mark.parametrize("form,whole_tile", [("streamk", "256x256x8w"), ("streamk64", "256x256x8wk64")])
@pytest.mark.parametrize("m,n,k", STREAMK_SHAPES)
def test_gemm_streamk_plain_and_fused_epilogue(R, monkeypatch, m, n, k, form, whole_tile):
    monkeypatch.setenv("RAI_HIP_GEMM_TILE", form)   # refuses (RAI_ERR_UNSUPPORTED) where the form does not apply
    dt = "bf16"
    x, w, b1, _, r = packed_case(rng(120), m, n, k)
    xd, wd = up(x, dt), up(w, dt)
    lin = onn.linear(x, w, None, dt)
    first = down(R.linear(xd, wd))
    assert_close(first, lin, dt, f"{form} linear {m}x{n}x{k}")
    gemm_elem_check(first, lin, dt, k, f"{form} linear {m}x{n}x{k}")
    # the shares are summed in slot order whoever arrives last: every run gives the same bits
    for _ in range(3):
        assert np.array_equal(down(R.linear(xd, wd)), first)
    want = oo.add(onn.new_gelu(onn.linear(x, w, b1, dt), dt), r, dt)
    got = down(R.linear(xd, wd, up(b1, dt), "new_gelu", up(r, dt)))
    assert_close(got, want, dt, f"stream-K linear + bias + new_gelu + residual {m}x{n}x{k}")
    # against the same tile without sharing: same products, another grouping of the f32 sums
    monkeypatch.setenv("RAI_HIP_GEMM_TILE", whole_tile)
    whole = down(R.linear(xd, wd))
    assert_close(whole, lin, dt, f"{whole_tile} linear {m}x{n}x{k}")
    gemm_elem_check(whole, lin, dt, k, f"{whole_tile} linear {m}x{n}x{k}")
    gemm_elem_check(first, whole, dt, k, f"stream-K against whole tiles {m}x{n}x{k}")


@pytest.mark.parametrize("form", ["streamk", "streamk64", "256x256x8wk64"])
def test_gemm_streamk_packed_epilogues(R, monkeypatch, form):
    monkeypatch.setenv("RAI_HIP_GEMM_TILE", form)
    dt, m, n, k, n1 = "bf16", 2100, 4936, 640, 2421      # 180 tiles; n1 odd: second output rows not 16-byte aligned
    x, w, b1, b2, r = packed_case(rng(121), m, n, k)
    xd, wd = up(x, dt), up(w, dt)
    o1, o2 = R.linear_packed(xd, wd, bias=up(b1, dt), act="new_gelu", act_from=n1, n1=n1)
    y = onn.linear(x, w, b1, dt)
    assert_close(down(o1), y[:, :n1], dt, "stream-K: q|k|v columns")
    assert_close(down(o2), onn.new_gelu(y[:, n1:], dt), dt, "stream-K: fc1 columns")
    k1 = 256
    got = down(R.linear_packed(xd, wd, bias=up(b1, dt), bias2=up(b2, dt), residual=up(r, dt)))
    want = oo.add(oo.add(onn.linear(x[:, :k1], w[:, :k1], b1, dt), onn.linear(x[:, k1:], w[:, k1:], b2, dt), dt), r, dt)
    assert_close(got, want, dt, "stream-K: dense + fc2 + residual")
    wg, wu = w[0::2], w[1::2]
    got = down(R.linear_packed(xd, wd, act="silu", glu=True))
    want = oo.mul(onn.silu(onn.linear(x, wg, None, dt), dt), onn.linear(x, wu, None, dt), dt)
    assert_close(got, want, dt, "stream-K: silu(gate) * up")


def test_gemm_streamk_lost_share_is_reported_and_recovers(R, monkeypatch):
    """A share that never arrives: the block that sums a tile gives up its bounded wait, writes nothing for that tile
    and flags the fault; the host's next synchronisation returns an error instead of wrong numbers, and the launch
    after that works from clean counters.  Forced from the host (a tiny spin limit, one tile whose stored shares are
    never counted): every wave exits normally."""
    from rai_amd._lib import RaiHipError
    from rai_amd.hip import sync
    monkeypatch.setenv("RAI_HIP_GEMM_TILE", "streamk64")
    dt, (m, n, k) = "bf16", STREAMK_SHAPES[0]
    x, w, _, _, _ = packed_case(rng(122), m, n, k)
    xd, wd = up(x, dt), up(w, dt)
    want = down(R.linear(xd, wd))
    monkeypatch.setenv("RAI_HIP_STREAMK_TEST", "64,0")
    with pytest.raises(RaiHipError, match="stream-K share never arrived"):
        R.linear(xd, wd)
        sync()
    monkeypatch.delenv("RAI_HIP_STREAMK_TEST")
    for _ in range(2):
        assert np.array_equal(down(R.linear(xd, wd)), want)


def test_gemm_streamk_refuses_where_it_does_not_apply(R, monkeypatch):
    from rai_amd._lib import RaiHipError
    monkeypatch.setenv("RAI_HIP_GEMM_TILE", "streamk")
    x, w = up(np.zeros((512, 64), np.float32), "bf16"), up(np.zeros((512, 64), np.float32), "bf16")
    with pytest.raises(RaiHipError):
        R.linear(x, w)      # four tiles


def test_gemm_dispatcher_picks_each_tile_by_itself(R, monkeypatch):
    # no override: 3072 x 3072 gives 144 tiles of 256 x 256 (the eight-wave tile), 4096 x 2048 gives 512 of 256 x 128,
    # 600 x 520 stays on 128 x 128; K = 64 is shorter than the prefetch depth of every one of them
    monkeypatch.delenv("RAI_HIP_GEMM_TILE", raising=False)
    dt = "bf16"
    for m, n, k in [(3072, 3072, 64), (4096, 2048, 96), (600, 520, 64), (3000, 3100, 2560)]:
        g = rng(114)
        x, w = rand(g, (m, k), dt), rand(g, (n, k), dt, 0.05)
        want = onn.linear(x, w, None, dt)
        got = down(R.linear(up(x, dt), up(w, dt)))
        assert_close(got, want, dt, f"linear {m}x{n}x{k}")
        gemm_elem_check(got, want, dt, k, f"linear {m}x{n}x{k}")
