"""The lazy-graph evaluator on the device against the CPU oracle: rai's own
decompositions (LayerNorm, RMSNorm, new_gelu / gelu / silu, Linear, Embedding, a
softmax attention block) built node by node and evaluated through the dispatcher;
the elementwise-fusion pass must give bit-identical results with fewer launches."""
import numpy as np
import pytest

from oracle import nn as onn, ops as oo
from oracle.dtypes import from_storage, rnd, to_storage
from rai_amd import graph as g
from rai_amd.graph import Tensor
from tests.util import assert_close

pytestmark = pytest.mark.gpu


def dev(arr, dt):
    return Tensor.from_array(to_storage(arr, dt), dt)


def rand(rng, shape, dt, scale=1.0):
    return rnd(rng.standard_normal(shape).astype(np.float32) * scale, dt)


def run(build, fusion, compose=False):
    """Builds and evaluates with the elementwise pass on/off; the composition pass is off unless asked for, so that
    the bit-identity checks of the elementwise pass compare like with like."""
    g.set_fusion(fusion)
    g.set_compose(compose)
    g.stats(reset=True)
    out = build()
    storage = out.as_storage()
    st = g.stats()
    g.set_fusion(True)
    g.set_compose(True)
    return storage, st, out


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_layer_norm_chain_matches_oracle_and_fuses(hip, dt):
    rng = np.random.default_rng(0)
    x, w, b = rand(rng, (6, 37, 96), dt), rand(rng, (96,), dt), rand(rng, (96,), dt)
    build = lambda: g.layer_norm(dev(x, dt), dev(w, dt), dev(b, dt), 1e-5)
    fused, st_f, _ = run(build, True)
    plain, st_p, _ = run(build, False)
    assert np.array_equal(fused, plain), "fusion changed the result"
    assert st_f["fused_regions"] >= 2 and st_f["kernel_launches"] < st_p["kernel_launches"]
    assert st_p["fused_regions"] == 0
    want = onn.layer_norm(x, w, b, 1e-5, dt)
    assert_close(from_storage(fused, dt), want, dt, "layer_norm")


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("act", ["new_gelu", "gelu", "silu", "relu"])
def test_activations_fuse_into_one_launch(hip, dt, act):
    rng = np.random.default_rng(1)
    x = rand(rng, (5, 1000), dt, 2.0)
    build = lambda: getattr(dev(x, dt), act)()
    fused, st_f, _ = run(build, True)
    plain, st_p, _ = run(build, False)
    assert np.array_equal(fused, plain), "fusion changed the result"
    assert st_f["kernel_launches"] == 1 and st_f["fused_regions"] == 1     # the whole chain is one region
    assert st_p["kernel_launches"] >= (5 if act != "relu" else 2)
    want = getattr(onn, act)(x, dt)
    assert_close(from_storage(fused, dt), want, dt, act)


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_rms_norm_linear_embedding(hip, dt):
    rng = np.random.default_rng(2)
    table = rand(rng, (50, 64), dt)
    ids = rng.integers(0, 50, (2, 7)).astype(np.uint32)
    w, wl, bl = rand(rng, (64,), dt), rand(rng, (48, 64), dt, 0.2), rand(rng, (48,), dt)

    def build():
        h = g.embedding(Tensor.from_array(ids, "u32"), dev(table, dt))
        h = g.rms_norm(h, dev(w, dt), 1e-6)
        return g.linear(h, dev(wl, dt), dev(bl, dt))

    fused, st_f, out = run(build, True)
    plain, _, _ = run(build, False)
    assert out.shape == (2, 7, 48)
    assert np.array_equal(fused, plain)
    h = onn.embedding(ids, table)
    h = onn.rms_norm(h, w, 1e-6, dt)
    want = onn.linear(h, wl, bl, dt)
    assert_close(from_storage(fused, dt), want, dt, "embedding -> rms_norm -> linear")


def test_attention_block_through_the_graph(hip):
    # q k^T * scale, causal mask by where, softmax, p v: the node sequence of phi2.rs:244-262 (f32)
    rng = np.random.default_rng(3)
    B, H, S, D = 2, 3, 9, 16
    q, k, v = (rand(rng, (B, H, S, D), "f32") for _ in range(3))
    mask = np.triu(np.ones((S, S), np.uint8), 1)

    def build():
        scores = dev(q, "f32").matmul(dev(k, "f32").transpose(-2, -1) * (1.0 / np.sqrt(D)))
        m = Tensor.from_array(mask, "u8").broadcast_to((B, H, S, S))
        scores = m.where_cond(scores.full_like(float("-inf")), scores)
        return scores.softmax(-1).matmul(dev(v, "f32")).transpose(1, 2).reshape((B, S, H * D))

    got, _, _ = run(build, True)
    s = np.einsum("bhsd,bhtd->bhst", q, k * np.float32(1.0 / np.sqrt(D)))
    s = np.where(mask.astype(bool), -np.inf, s)
    p = np.exp(s - s.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    want = np.einsum("bhst,bhtd->bhsd", p, v).transpose(0, 2, 1, 3).reshape(B, S, H * D)
    assert_close(got, want, "f32", "attention through the graph")


def test_views_share_storage_and_detach_drops_inputs(hip):
    x = dev(np.arange(24, dtype=np.float32).reshape(2, 3, 4), "f32")
    y = x.transpose(0, 2).narrow(1, 1, 2)          # views only
    g.stats(reset=True)
    y.eval(retain_graph=True)
    assert g.stats()["kernel_launches"] == 0 and y.num_inputs() == 1     # retain_graph keeps the inputs
    assert x.is_evaluated() and y.storage().data == x.storage().data      # zero-copy views
    np.testing.assert_array_equal(y.as_storage(), np.arange(24, dtype=np.float32).reshape(2, 3, 4).transpose(2, 1, 0)[:, 1:3])
    z = (y + 1.0).sum(0)
    z.eval()
    assert z.num_inputs() == 0                      # eval.rs:47-49 detach
    np.testing.assert_array_equal(z.as_storage(), (np.arange(24, dtype=np.float32).reshape(2, 3, 4).transpose(2, 1, 0)[:, 1:3] + 1).sum(0))


def test_shared_intermediates_are_materialised_not_inlined(hip):
    rng = np.random.default_rng(4)
    x = rand(rng, (64, 33), "f32")

    def build():
        y = dev(x, "f32").exp()                      # three consumers: must receive data
        return (y + y.tanh()) * y

    fused, st, _ = run(build, True)
    plain, _, _ = run(build, False)
    assert np.array_equal(fused, plain)
    y = np.exp(x)
    assert_close(fused, (y + np.tanh(y)) * y, "f32", "shared intermediate")


def test_held_intermediate_is_not_folded_away(hip):
    x = dev(np.linspace(-2, 2, 40, dtype=np.float32), "f32")
    mid = x.tanh()                                   # a handle stays alive: it must be evaluated
    out = (mid * 2.0).exp()
    out.eval(retain_graph=True)
    assert mid.is_evaluated()
    np.testing.assert_allclose(mid.as_storage(), np.tanh(np.linspace(-2, 2, 40, dtype=np.float32)), rtol=1e-6)


def test_unimplemented_rule_and_err_node_fail_eval(hip):
    x = dev(np.ones((3, 5), np.float32), "f32")
    g.dispatch_unregister("Softmax")
    try:
        with pytest.raises(g.RaiHipError) as e:
            x.softmax(-1).eval()
        assert e.value.status == -7 and "Unimplemented" in str(e.value) and "Softmax" in str(e.value)
        # fusion never hides a missing rule of a node it would fold
        g.dispatch_unregister("Unary")
        with pytest.raises(g.RaiHipError):
            ((x.tanh() + 1.0) * 2.0).eval()
    finally:
        g.dispatch_register_builtin("Softmax")
        g.dispatch_register_builtin("Unary")
    np.testing.assert_allclose(x.softmax(-1).as_storage(), np.full((3, 5), 0.2, np.float32), rtol=1e-6)
    with pytest.raises(g.RaiHipError) as e:
        (x.matmul(x) + 1.0).eval()
    assert e.value.status == -2


def test_large_region_falls_back_to_node_by_node(hip):
    x0 = np.linspace(0.1, 1.0, 128, dtype=np.float32)

    def build():
        t = dev(x0, "f32")
        for _ in range(40):                          # longer than one fused program
            t = (t * 1.01).tanh()
        return t

    fused, _, _ = run(build, True)
    plain, _, _ = run(build, False)
    assert np.array_equal(fused, plain)
    want = x0.astype(np.float64)
    for _ in range(40):
        want = np.tanh(want * np.float64(np.float32(1.01)))
    assert_close(fused, want, "f32", "long chain")


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_phi2_through_the_graph_matches_oracle(hip, dt):
    # the model code of phi2.rs recorded as a lazy graph and evaluated node by node on the
    # device (the reference's own execution scheme), prefill then two cached decode steps
    from oracle import phi2
    from tests.graph_models import Phi2Graph
    cfg = phi2.Config(vocab_size=300, hidden_size=128, intermediate_size=256, num_hidden_layers=2,
                      num_attention_heads=4, max_position_embeddings=64)
    params = phi2.random_params(cfg, dt, seed=0)
    ref = phi2.Model(cfg, params, dt)
    model = Phi2Graph(cfg, {k: dev(v, dt) for k, v in params.items()}, dt)
    ids = np.random.Generator(np.random.PCG64(1)).integers(0, cfg.vocab_size, (2, 10)).astype(np.uint32)
    for step in range(3):
        g.stats(reset=True)
        logits = model.fwd(Tensor.from_array(ids, "u32"))
        got = from_storage(logits.as_storage(), dt)[:, 0, :]
        want = ref.fwd(ids)
        assert_close(got, want, dt, f"graph phi2 step {step}")
        st = g.stats()
        assert st["kernel_launches"] < st["nodes_evaluated"]
        # the composition pass (on by default) takes every module of the two layers and the head: per layer one
        # LayerNorm, six Linears (fc1 with its activation, fc2 with the layer input added, dense with that sum added),
        # two rotary embeddings and one attention block; in the cached steps the rotary embeddings, both cache
        # concatenations and the attention block are one launch
        assert st["composed_regions"] == 2 * (10, 8, 8)[step] + 2, st
        # launches: those, two copies in the first cached step (the prefill's caches move into buffers with room to
        # grow), the embedding and, in the first evaluation, the rotary tables
        assert st["kernel_launches"] <= 2 * ((10, 8, 8)[step] + (0, 2, 0)[step]) + (14, 4, 4)[step], st
        ids = np.argmax(want, -1).astype(np.uint32).reshape(2, 1)
    # greedy ids through the graph: argmax node, u32, bit-exact against the oracle on the same logits
    tok = logits.argmax(-1).as_storage()[:, 0]
    assert tok.dtype == np.uint32 and np.array_equal(tok, np.argmax(got, -1))


def test_gather_index_add_scatter_add_nodes(hip):
    # the primitives the vjp rules of index_select and gather evaluate, on strided (transposed) inputs too
    rng = np.random.default_rng(5)
    x = rand(rng, (6, 9), "f32")
    ix = rng.integers(0, 6, (4, 9)).astype(np.uint32)
    got = dev(x, "f32").gather(0, Tensor.from_array(ix, "u32")).as_storage()
    assert np.array_equal(got, oo.gather(x, 0, ix))
    got = dev(x.T.copy(), "f32").t().gather(0, Tensor.from_array(ix, "u32")).as_storage()   # non-contiguous x
    assert np.array_equal(got, oo.gather(x, 0, ix))
    ids = rng.integers(0, 6, 13).astype(np.uint32)
    src = rand(rng, (13, 9), "f32")
    got = dev(x, "f32").index_add(0, Tensor.from_array(ids, "u32"), dev(src, "f32")).as_storage()
    assert np.array_equal(got, oo.index_add(x, 0, ids, src, "f32"))
    # adjoint pair as the reference's vjp builds it (ops/index_select.rs:40-48): zeros_like(x).index_add(dim, index, cotangent)
    zero = Tensor.full(0.0, (6, 9), "f32")
    got = zero.index_add(0, Tensor.from_array(ids, "u32"), dev(src.T.copy(), "f32").t()).as_storage()
    assert np.array_equal(got, oo.index_add(np.zeros_like(x), 0, ids, src, "f32"))
    upd = rand(rng, (4, 9), "f32")
    got = dev(x, "f32").scatter_add(0, Tensor.from_array(ix, "u32"), dev(upd, "f32")).as_storage()
    assert np.array_equal(got, oo.scatter_add(x, 0, ix, upd, "f32"))
    with pytest.raises(Exception):
        dev(x, "f32").gather(1, Tensor.from_array(ix, "u32")).as_storage()   # Err node surfaces at eval


# ------------------------------------------------------------------ composition pass
@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_compositions_are_taken_by_one_launch_each(hip, dt):
    rng = np.random.default_rng(7)
    x, w, b = rand(rng, (4, 21, 96), dt), rand(rng, (96,), dt), rand(rng, (96,), dt)
    wl, bl = rand(rng, (40, 96), dt, 0.2), rand(rng, (40,), dt)
    cases = {
        "layer_norm": (lambda: g.layer_norm(dev(x, dt), dev(w, dt), dev(b, dt), 1e-5), onn.layer_norm(x, w, b, 1e-5, dt)),
        "rms_norm": (lambda: g.rms_norm(dev(x, dt), dev(w, dt), 1e-6), onn.rms_norm(x, w, 1e-6, dt)),
        "linear": (lambda: g.linear(dev(x, dt), dev(wl, dt), dev(bl, dt)), onn.linear(x, wl, bl, dt)),
    }

    def rms_norm_by_division():     # the same value recorded as x / sqrt(n): also taken
        xt, wt = dev(x, dt), dev(w, dt)
        return wt * xt * ((xt / float(np.sqrt(96))).square().sum(-1, True) + 1e-6).rsqrt()
    cases["rms_norm recorded as a division"] = (rms_norm_by_division, onn.rms_norm(x, w, 1e-6, dt))
    for name, (build, want) in cases.items():
        composed, st_c, _ = run(build, True, compose=True)
        plain, st_p, _ = run(build, True, compose=False)
        assert st_c["composed_regions"] == 1 and st_c["kernel_launches"] == 1, (name, st_c)
        assert st_p["composed_regions"] == 0 and st_p["kernel_launches"] > 1, (name, st_p)
        assert_close(from_storage(composed, dt), want, dt, f"{name} composed")
        assert_close(from_storage(plain, dt), want, dt, f"{name} node by node")


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_rotary_and_attention_compositions(hip, dt):
    from oracle import phi2
    from tests.graph_models import Phi2Graph
    cfg = phi2.Config(vocab_size=50, hidden_size=160, intermediate_size=64, num_hidden_layers=1, num_attention_heads=2,
                      max_position_embeddings=64)
    model = Phi2Graph(cfg, {}, dt)
    rng = np.random.default_rng(8)
    xs = rand(rng, (2, 2, 9, 80), dt)
    sin, cos = phi2.rotary_tables(cfg, dt)
    g.eval_all([model.sin, model.cos])          # the tables are shared state of the model, built once
    for offset in (0, 13):
        build = lambda: model._rotary(dev(xs, dt), offset)
        composed, st_c, _ = run(build, True, compose=True)
        plain, st_p, _ = run(build, True, compose=False)
        assert st_c["composed_regions"] == 1 and st_p["composed_regions"] == 0
        assert st_c["kernel_launches"] < st_p["kernel_launches"]
        want = phi2.rotary(xs, sin, cos, cfg.rotary_dim, offset, dt)
        assert_close(from_storage(composed, dt), want, dt, "rotary composed")
        assert np.array_equal(composed, plain), "the rotary launcher rounds where the node chain rounds"
    # the attention block of phi2.rs:244-262 with the causal mask, and without one on a longer key range (decode)
    B, H, D = 2, 3, 80
    for S, T, causal in ((9, 9, True), (1, 30, False)):
        q, k, v = rand(rng, (B, H, S, D), dt), rand(rng, (B, H, T, D), dt), rand(rng, (B, H, T, D), dt)

        def build():
            w = dev(q, dt).to_dtype("f32").matmul(dev(k, dt).to_dtype("f32").t() * (1.0 / np.sqrt(D)))
            if causal:
                m = Tensor.from_array(np.triu(np.ones((S, T), np.uint8), 1), "u8").broadcast_to(w.shape)
                w = m.where_cond(w.full_like(float("-inf")), w)
            return w.softmax(-1).to_dtype(dt).matmul(dev(v, dt)).transpose(1, 2).reshape((B, S, H * D))

        composed, st_c, _ = run(build, True, compose=True)
        plain, st_p, _ = run(build, True, compose=False)
        assert st_c["composed_regions"] == 1 and st_c["kernel_launches"] == 1, st_c
        assert st_p["kernel_launches"] >= 4
        assert_close(from_storage(composed, dt), from_storage(plain, dt), dt, "attention composed vs node by node")
    # a mask that is not the causal one must not be taken for it
    S = T = 9
    q, k, v = (rand(rng, (B, H, S, D), dt) for _ in range(3))
    odd = np.triu(np.ones((S, T), np.uint8), 2)

    def build_odd():
        w = dev(q, dt).to_dtype("f32").matmul(dev(k, dt).to_dtype("f32").t() * 0.1)
        w = Tensor.from_array(odd, "u8").broadcast_to(w.shape).where_cond(w.full_like(float("-inf")), w)
        return w.softmax(-1).to_dtype(dt).matmul(dev(v, dt)).transpose(1, 2).reshape((B, S, H * D))

    _, st, _ = run(build_odd, True, compose=True)
    assert st["composed_regions"] == 0


def test_composition_is_not_taken_when_an_interior_node_is_observable(hip):
    rng = np.random.default_rng(9)
    x, w, b = rand(rng, (5, 64), "f32"), rand(rng, (64,), "f32"), rand(rng, (64,), "f32")
    xd = dev(x, "f32")
    mean = xd.mean(-1, True)                       # the caller keeps the mean: LayerNorm below recomputes its own,
    var = xd.var(-1, True)                         # but this variance node is the one the norm uses
    xs = (xd - mean) * (var + 1e-5).rsqrt()
    y = dev(w, "f32") * xs + dev(b, "f32")
    g.set_compose(True)
    g.stats(reset=True)
    got = y.as_storage()
    st = g.stats()
    assert st["composed_regions"] == 0             # `mean`, `var`, `xs` are held outside the graph
    assert_close(got, onn.layer_norm(x, w, b, 1e-5, "f32"), "f32")
    assert_close(var.as_storage(), onn.var(x, -1, True, "f32"), "f32", "the held node is still evaluated")


def test_phi2_qk_layernorm_through_the_graph(hip):
    # phi2.rs:207-216: one head is the only well-formed case (the parameters have head_dim elements, the projection
    # heads * head_dim); with more heads the recorded graph holds the reference's IncompatibleShape error node
    from oracle import phi2
    from rai_amd._lib import RaiHipError
    from rai_amd.models import Decoder
    from tests.graph_models import Phi2Graph
    dt = "f32"
    cfg = phi2.Config(vocab_size=200, hidden_size=80, intermediate_size=160, num_hidden_layers=2, num_attention_heads=1,
                      max_position_embeddings=48, qk_layernorm=True)
    params = phi2.random_params(cfg, dt, seed=2, std=0.1)
    rng = np.random.default_rng(12)
    for k in params:
        if "layernorm" in k:
            params[k] = rnd(params[k] + 0.1 * rng.standard_normal(params[k].shape).astype(np.float32), dt)
    ref = phi2.Model(cfg, params, dt)
    model = Phi2Graph(cfg, {k: dev(v, dt) for k, v in params.items()}, dt)
    ids = rng.integers(0, cfg.vocab_size, (2, 9)).astype(np.uint32)
    for _ in range(2):
        got = from_storage(model.fwd(Tensor.from_array(ids, "u32")).as_storage(), dt)[:, 0, :]
        want = ref.fwd(ids)
        assert_close(got, want, dt, "phi2 with qk_layernorm through the graph")
        ids = np.argmax(want, -1).astype(np.uint32).reshape(2, 1)
    many = phi2.Config(vocab_size=200, hidden_size=160, intermediate_size=160, num_hidden_layers=1,
                       num_attention_heads=2, max_position_embeddings=48, qk_layernorm=True)
    pm = phi2.random_params(many, dt, seed=2)
    bad = Phi2Graph(many, {k: dev(v, dt) for k, v in pm.items()}, dt).fwd(Tensor.from_array(ids[:, :1], "u32"))
    with pytest.raises(RaiHipError, match="IncompatibleShape"):
        bad.as_storage()
    with pytest.raises(RaiHipError) as e:          # the decoder drivers decline the option
        Decoder("phi2", dt, vocab_size=200, hidden_size=80, intermediate_size=160, num_hidden_layers=1,
                num_attention_heads=1, rotary_dim=32, qk_layernorm=True)
    assert e.value.status == -7


# ------------------------------------------------------------------ wider compositions, cache append, Qwen2 / Gemma
@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_linear_takes_its_activation_and_one_residual(hip, dt):
    rng = np.random.default_rng(21)
    x, wl, bl = rand(rng, (3, 17, 96), dt), rand(rng, (40, 96), dt, 0.2), rand(rng, (40,), dt)
    r = rand(rng, (3, 17, 40), dt)
    lin = lambda bias: g.linear(dev(x, dt), dev(wl, dt), dev(bl, dt) if bias else None)
    cases = {}
    for act in ("new_gelu", "gelu", "silu", "relu"):
        cases[f"{act}(linear + b)"] = (lambda act=act: getattr(lin(True), act)(), getattr(onn, act)(onn.linear(x, wl, bl, dt), dt))
    cases["silu(linear)"] = (lambda: lin(False).silu(), onn.silu(onn.linear(x, wl, None, dt), dt))
    cases["linear + b + r"] = (lambda: lin(True) + dev(r, dt), oo.add(onn.linear(x, wl, bl, dt), r, dt))
    cases["r + linear"] = (lambda: dev(r, dt) + lin(False), oo.add(r, onn.linear(x, wl, None, dt), dt))
    cases["gelu(linear + b) + r"] = (lambda: lin(True).gelu() + dev(r, dt), oo.add(onn.gelu(onn.linear(x, wl, bl, dt), dt), r, dt))
    for name, (build, want) in cases.items():
        composed, st_c, _ = run(build, True, compose=True)
        plain, st_p, _ = run(build, True, compose=False)
        assert st_c["composed_regions"] == 1 and st_c["kernel_launches"] == 1, (name, st_c)
        assert st_p["composed_regions"] == 0 and st_p["kernel_launches"] >= 2, (name, st_p)
        assert_close(from_storage(composed, dt), want, dt, f"{name} composed")
        assert_close(from_storage(plain, dt), want, dt, f"{name} node by node")
    # an activation whose argument is used elsewhere too is not folded away: both results must be right
    def shared():
        y = lin(True)
        return y.silu() + y
    composed, st_c, _ = run(shared, True, compose=True)
    y = onn.linear(x, wl, bl, dt)
    assert_close(from_storage(composed, dt), oo.add(onn.silu(y, dt), y, dt), dt, "silu(y) + y")


def test_linears_of_one_row_share_a_launch(hip, monkeypatch):
    """A decode step's q, k, v projections and first MLP Linear (phi2.rs:293-297) read one normalised row: at one row
    they run as one launch, the LayerNorm in its prologue when nothing else reads it.  Against the oracle, against the
    same graph with the grouping off (RAI_HIP_GRAPH_NO_LINEAR_GROUPS=1; same bits when no norm is folded in), and with a
    fifth Linear on the same row (a second launch; the norm is then materialised)."""
    dt, K = "bf16", 256
    rng = np.random.default_rng(31)
    x = rand(rng, (1, 1, K), dt)
    lw, lb = rnd(1.0 + 0.1 * rng.standard_normal(K).astype(np.float32), dt), rand(rng, (K,), dt, 0.1)
    shapes = [64, 32, 48, 512, 40]
    ws = [rand(rng, (n, K), dt, 0.1) for n in shapes]
    bs = [rand(rng, (n,), dt) for n in shapes]
    params = [dev(a, dt) for a in ws + bs + [lw, lb]]
    g.eval_all(params)
    wd, bd, lwd, lbd = params[:5], params[5:10], params[10], params[11]

    def build(norm, count):
        xt = dev(x, dt)
        h = g.layer_norm(xt, lwd, lbd, 1e-5) if norm else xt
        outs = [g.linear(h, wd[i], bd[i]) for i in range(count)]
        if count > 3:
            outs[3] = outs[3].new_gelu()
        return outs

    def want(norm, count):
        h = onn.layer_norm(x, lw, lb, 1e-5, dt) if norm else x
        outs = [onn.linear(h, ws[i], bs[i], dt) for i in range(count)]
        if count > 3:
            outs[3] = onn.new_gelu(outs[3], dt)
        return outs

    def evaluate(norm, count):
        g.stats(reset=True)
        outs = build(norm, count)
        g.eval_all(outs)
        return [o.as_storage() for o in outs], g.stats()

    for norm, count, launches in ((True, 4, 1), (False, 4, 1), (True, 5, 3), (False, 2, 1)):
        got, st = evaluate(norm, count)
        assert st["kernel_launches"] == launches, (norm, count, st)
        for i, (a, b) in enumerate(zip(got, want(norm, count))):
            assert_close(from_storage(a, dt), b, dt, f"grouped linear {i} norm={norm} count={count}")
        monkeypatch.setenv("RAI_HIP_GRAPH_NO_LINEAR_GROUPS", "1")
        plain, st_p = evaluate(norm, count)
        monkeypatch.delenv("RAI_HIP_GRAPH_NO_LINEAR_GROUPS")
        assert st_p["kernel_launches"] == count + (1 if norm else 0), st_p
        for i, (a, b) in enumerate(zip(got, plain)):
            if norm and count <= 4:
                assert_close(from_storage(a, dt), from_storage(b, dt), dt, f"grouped vs single linear {i}")
            else:
                np.testing.assert_array_equal(a, b)


def test_head_takes_the_final_norm_through_the_last_position_view(hip, monkeypatch):
    """Model::fwd of phi2.rs ends with final_layernorm, narrow to the last position, lm_head.  At one row the narrow
    keeps every element, and norm + view + Linear are one launch; with more rows the norm stays a launch of its own."""
    dt, K, N = "bf16", 256, 1000
    rng = np.random.default_rng(41)
    lw, lb = rnd(1.0 + 0.1 * rng.standard_normal(K).astype(np.float32), dt), rand(rng, (K,), dt, 0.1)
    w, b = rand(rng, (N, K), dt, 0.1), rand(rng, (N,), dt)
    params = [dev(a, dt) for a in (lw, lb, w, b)]
    g.eval_all(params)
    for rows, launches in ((1, 1), (5, 2)):
        x = rand(rng, (1, rows, K), dt)
        g.stats(reset=True)
        def head():   # the handles of the norm and of the view end with the function, as in Model::fwd
            h = g.layer_norm(dev(x, dt), params[0], params[1], 1e-5).narrow(1, rows - 1, 1)
            return g.linear(h, params[2], params[3])
        got = from_storage(head().as_storage(), dt)
        st = g.stats()
        want = onn.linear(onn.layer_norm(x, lw, lb, 1e-5, dt)[:, rows - 1:, :], w, b, dt)
        assert_close(got, want, dt, f"head behind the final norm, {rows} rows")
        assert st["kernel_launches"] == launches, (rows, st)


@pytest.mark.parametrize("arch", ["qwen2", "gemma"])
def test_bias_free_linears_of_one_row_are_grouped_too(hip, monkeypatch, arch):
    """A decode step of gemma.rs / qwen2.rs at batch 1: q, k, v (no bias in Gemma) behind one RMSNorm, gate and up behind
    the other.  Each norm and its Linears are one launch; the whole model agrees with the oracle step for step, with
    the grouping on and off."""
    from oracle import qwen2
    from tests.graph_models import SeqGraph
    dt = "bf16"
    if arch == "qwen2":
        cfg = qwen2.Config("qwen2", 300, 128, 256, 2, 4, 2, "silu", max_position_embeddings=64, rope_theta=1e6, head_dim=32)
    else:
        cfg = qwen2.Config("gemma", 300, 128, 256, 2, 4, 1, "gelu", max_position_embeddings=64, head_dim=32)
    params = qwen2.random_params(cfg, dt, seed=0)
    rng = np.random.default_rng(29)
    for k in params:
        if k.endswith("norm.weight") or k.endswith(".bias"):
            params[k] = rnd(params[k] + 0.1 * rng.standard_normal(params[k].shape).astype(np.float32), dt)
    launches = {}
    for grouped in (True, False):
        if not grouped:
            monkeypatch.setenv("RAI_HIP_GRAPH_NO_LINEAR_GROUPS", "1")
        ref = qwen2.Model(cfg, params, dt)
        model = SeqGraph(cfg, {k: dev(v, dt) for k, v in params.items()}, dt)
        ids = np.random.Generator(np.random.PCG64(3)).integers(0, cfg.vocab_size, (1, 9)).astype(np.uint32)
        for step in range(4):
            g.stats(reset=True)
            got = from_storage(model.fwd(Tensor.from_array(ids, "u32")).as_storage(), dt)[:, 0, :]
            want = ref.fwd(ids)
            assert_close(got, want, dt, f"{arch} one-row graph step {step} grouped={grouped}")
            launches[grouped] = g.stats()["kernel_launches"]
            ids = np.argmax(want, -1).astype(np.uint32).reshape(1, 1)
    monkeypatch.delenv("RAI_HIP_GRAPH_NO_LINEAR_GROUPS", raising=False)
    # per layer: norm + q|k|v, rotary + append + attention, o + x, norm + gate|up, act(gate) * up, down + x1
    assert launches[True] <= 2 * 6 + 5, launches
    assert launches[False] >= launches[True] + 2 * 5, launches


@pytest.mark.parametrize("k1,k2,n", [(64, 1024, 96), (2560, 10240, 2560), (512, 256, 40)])
def test_two_linears_and_the_layer_input_of_one_row_share_a_launch(hip, monkeypatch, k1, k2, n):
    """(dense(attn) + fc2(act)) + x of DecoderLayer::fwd (phi2.rs:298) at one row: one launch that streams both weight
    matrices; two launches with the grouping off; both against the oracle's node-by-node sums."""
    dt = "bf16"
    rng = np.random.default_rng(37)
    x1, x2, r = rand(rng, (1, 1, k1), dt), rand(rng, (1, 1, k2), dt), rand(rng, (1, 1, n), dt)
    w1, w2 = rand(rng, (n, k1), dt, 0.05), rand(rng, (n, k2), dt, 0.02)
    b1, b2 = rand(rng, (n,), dt), rand(rng, (n,), dt)
    params = [dev(a, dt) for a in (w1, w2, b1, b2)]
    g.eval_all(params)
    want = oo.add(oo.add(onn.linear(x1, w1, b1, dt), onn.linear(x2, w2, b2, dt), dt), r, dt)

    def evaluate():
        g.stats(reset=True)
        out = (g.linear(dev(x1, dt), params[0], params[2]) + g.linear(dev(x2, dt), params[1], params[3])) + dev(r, dt)
        got = from_storage(out.as_storage(), dt)
        return got, g.stats()

    got, st = evaluate()
    assert st["kernel_launches"] == 1 and st["composed_regions"] == 2, st
    assert_close(got, want, dt, "two linears + x, one launch")
    monkeypatch.setenv("RAI_HIP_GRAPH_NO_LINEAR_GROUPS", "1")
    plain, st_p = evaluate()
    assert st_p["kernel_launches"] == 2 and st_p["composed_regions"] == 2, st_p
    assert_close(plain, want, dt, "two linears + x, two launches")


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_cache_concatenation_appends_in_place(hip, dt):
    # cat([cache, new], 2) step after step, as the models' key / value caches grow: after the first growth only the
    # new rows are written (one small launch), every result is what a plain concatenation gives, earlier results stay
    # intact, and a second concatenation onto the same tensor does not see the first one's rows
    rng = np.random.default_rng(22)
    from rai_amd.graph import cat
    base = rand(rng, (2, 3, 10, 16), dt)
    want = base
    cache = dev(base, dt)
    cache.eval()
    held = []
    for step in range(5):
        new = rand(rng, (2, 3, 1, 16), dt)
        want = np.concatenate([want, new], axis=2)
        g.stats(reset=True)
        cache = cat([cache, dev(new, dt)], 2)
        got = cache.as_storage()
        st = g.stats()
        assert np.array_equal(got, to_storage(want, dt)), f"step {step}"
        assert st["kernel_launches"] == (2 if step == 0 else 1), (step, st)   # the upload of `new` launches nothing
        held.append((cache, want))
    for c, w in held:                      # the earlier tensors still read as they did
        assert np.array_equal(c.as_storage(), to_storage(w, dt))
    # branching: two different appends onto the same tensor
    c3, w3 = held[2]
    a, b = rand(rng, (2, 3, 1, 16), dt), rand(rng, (2, 3, 2, 16), dt)
    ca, cb = cat([c3, dev(a, dt)], 2), cat([c3, dev(b, dt)], 2)
    assert np.array_equal(cb.as_storage(), to_storage(np.concatenate([w3, b], axis=2), dt))
    assert np.array_equal(ca.as_storage(), to_storage(np.concatenate([w3, a], axis=2), dt))
    assert np.array_equal(held[3][0].as_storage(), to_storage(held[3][1], dt))
    # consumers see the strided result like any other tensor
    t = held[4][0]
    assert np.array_equal(t.transpose(1, 2).reshape((2, 15, 48)).as_storage(),
                          to_storage(held[4][1].transpose(0, 2, 1, 3).reshape(2, 15, 48), dt))
    assert np.array_equal(t.unsqueeze(2).as_storage(), to_storage(held[4][1][:, :, None], dt))


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("arch", ["qwen2", "gemma"])
def test_qwen2_and_gemma_through_the_graph(hip, arch, dt):
    # qwen2.rs / gemma.rs recorded as lazy graphs: prefill then two cached decode steps, node by node (the reference's
    # execution scheme) and with the composition pass, against the oracle's restatement of the same files
    from oracle import qwen2
    from tests.graph_models import SeqGraph
    if arch == "qwen2":
        cfg = qwen2.Config("qwen2", 300, 128, 256, 2, 4, 2, "silu", max_position_embeddings=64, rope_theta=1e6, head_dim=32)
    else:
        cfg = qwen2.Config("gemma", 300, 128, 256, 2, 4, 1, "gelu", max_position_embeddings=64, head_dim=32)
    params = qwen2.random_params(cfg, dt, seed=0)
    rng = np.random.default_rng(23)
    for k in params:   # norm weights and biases away from their trivial values
        if k.endswith("norm.weight") or k.endswith(".bias"):
            params[k] = rnd(params[k] + 0.1 * rng.standard_normal(params[k].shape).astype(np.float32), dt)
    for compose in (False, True):
        g.set_compose(compose)
        ref = qwen2.Model(cfg, params, dt)
        model = SeqGraph(cfg, {k: dev(v, dt) for k, v in params.items()}, dt)
        ids = np.random.Generator(np.random.PCG64(2)).integers(0, cfg.vocab_size, (2, 10)).astype(np.uint32)
        for step in range(3):
            g.stats(reset=True)
            got = from_storage(model.fwd(Tensor.from_array(ids, "u32")).as_storage(), dt)[:, 0, :]
            want = ref.fwd(ids)
            assert_close(got, want, dt, f"graph {arch} step {step} compose={compose}")
            st = g.stats()
            if compose:
                # per layer: two norms, rotary embedding of q and k, the attention block, and the Linears that carry a
                # bias (Qwen2: q, k, v), an activation (gate) or a residual (o, down); plus the final norm
                # (in the cached steps rotary embeddings, cache appends and attention are one launch)
                per_layer = 2 + 2 + 1 + 3 + (3 if arch == "qwen2" else 0) - (2 if step >= 1 else 0)
                assert st["composed_regions"] == 2 * per_layer + 1, st
            else:
                assert st["composed_regions"] == 0
            ids = np.argmax(want, -1).astype(np.uint32).reshape(2, 1)
    g.set_compose(True)


def test_storage_crosses_the_boundary_both_ways(hip):
    # what the Rust bridge does per tape: operands that have data come in as views of their allocations, results go
    # back out as (view, allocation) pairs that outlive the nodes
    rng = np.random.default_rng(24)
    x, w = rand(rng, (4, 6), "f32"), rand(rng, (5, 6), "f32")
    a = dev(x, "f32").eval()
    leaf = Tensor.from_storage(a.storage(), a.buffer())
    assert leaf.is_evaluated() and leaf.shape == (4, 6) and leaf.num_inputs() == 0
    view = Tensor.from_storage(a.t().eval().storage(), a.buffer())        # a strided view of the same allocation
    assert view.shape == (6, 4)
    out = (g.linear(leaf, dev(w, "f32")) * 2.0).eval()
    desc, buf = out.storage(), out.buffer()
    assert buf and desc.rank == 2
    from rai_amd import _lib
    _lib.call("rai_hip_retain", buf)          # the front end's handle on the result
    del out, leaf
    again = Tensor.from_storage(desc, buf)    # still valid after the nodes are gone
    assert_close(from_storage(again.as_storage(), "f32"), oo.mul(onn.linear(x, w, None, "f32"), np.float32(2.0), "f32"), "f32", "round trip")
    assert np.array_equal(view.as_storage(), to_storage(x.T.copy(), "f32"))
    del again
    _lib.call("rai_hip_release", buf)
