"""Safetensors loading through the C ABI (Module::update_by_safetensors, rai-core/src/nn.rs:39-55):
parameters found by the reference's names, converted to the model dtype, missing ones named in the error."""
import json
import struct

import numpy as np
import pytest

from oracle import phi2
from oracle.dtypes import to_storage
from tests.test_gpu_phi2 import small_cfg
from tests.util import assert_close

pytestmark = pytest.mark.gpu

ST_NAME = {"f32": "F32", "bf16": "BF16", "f16": "F16", "f64": "F64"}


def raw_bytes(a, st_dtype):
    a = np.asarray(a, np.float32)
    if st_dtype == "F32":
        return a.astype("<f4").tobytes()
    if st_dtype == "F64":
        return a.astype("<f8").tobytes()
    if st_dtype == "F16":
        return a.astype("<f2").tobytes()
    if st_dtype == "BF16":
        return to_storage(phi2.rnd(a, "bf16"), "bf16").astype("<u2").tobytes()
    raise ValueError(st_dtype)


def write_safetensors(path, tensors, st_dtype, metadata=None):
    """Writes the format by hand (8-byte little-endian header length, JSON header, raw bytes), so the
    parser is pinned against the format itself and not against a writer library."""
    header, blobs, off = {}, [], 0
    if metadata is not None:
        header["__metadata__"] = metadata
    for name, a in tensors.items():
        dt = st_dtype[name] if isinstance(st_dtype, dict) else st_dtype
        if dt == "I64":
            b = np.asarray(a).astype("<i8").tobytes()
        else:
            b = raw_bytes(a, dt)
        header[name] = {"dtype": dt, "shape": list(np.shape(a)), "data_offsets": [off, off + len(b)]}
        blobs.append(b)
        off += len(b)
    hj = json.dumps(header).encode()
    hj += b" " * (-len(hj) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(hj)))
        f.write(hj)
        for b in blobs:
            f.write(b)


def new_decoder(cfg, dt):
    from rai_amd.models import Decoder
    return Decoder("phi2", dt, vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size,
                   intermediate_size=cfg.intermediate_size, num_hidden_layers=cfg.num_hidden_layers,
                   num_attention_heads=cfg.num_attention_heads, num_key_value_heads=cfg.num_key_value_heads,
                   rotary_dim=cfg.rotary_dim, max_position_embeddings=cfg.max_position_embeddings,
                   hidden_act=cfg.hidden_act, tie_word_embeddings=cfg.tie_word_embeddings, rope_theta=cfg.rope_theta,
                   norm_eps=cfg.layer_norm_eps, max_batch=2, max_context=64)


def nonzero_params(cfg, seed=0):
    """f32 master weights with non-trivial biases and norm parameters."""
    params = phi2.random_params(cfg, "f32", seed=seed)
    g = np.random.Generator(np.random.PCG64(seed + 7))
    for k in params:
        if k.endswith(".bias"):
            params[k] = (0.02 * g.standard_normal(params[k].shape)).astype(np.float32)
    return params


@pytest.mark.parametrize("model_dt", ["f32", "bf16"])
@pytest.mark.parametrize("file_dt", ["f32", "bf16", "f16", "f64"])
def test_load_safetensors_converts_to_model_dtype(hip, tmp_path, model_dt, file_dt):
    cfg = small_cfg()
    master = nonzero_params(cfg)
    path = tmp_path / "model.safetensors"
    extra = {"model.rotary_emb.inv_freq": np.arange(16, dtype=np.float32)}   # not a parameter of the model: ignored
    write_safetensors(path, {**master, **extra}, ST_NAME[file_dt], metadata={"format": "pt", "note": "café \"q\""})
    dec = new_decoder(cfg, model_dt)
    dec.load_safetensors(path)
    # what update_by_name does: stored value -> (file dtype) -> to_dtype(model dtype)
    stored = {k: phi2.rnd(v, file_dt) if file_dt in ("bf16", "f16") else v for k, v in master.items()}
    want_params = {k: phi2.rnd(np.asarray(v, np.float32), model_dt) for k, v in stored.items()}
    ref = phi2.Model(cfg, want_params, model_dt)
    ids = np.random.Generator(np.random.PCG64(1)).integers(0, cfg.vocab_size, (2, 9)).astype(np.uint32)
    logits, _ = dec.forward(ids)
    assert_close(logits, ref.fwd(ids), model_dt, f"logits after loading {file_dt} file into {model_dt} model")
    # the same weights through load_param give bit-identical logits
    dec2 = new_decoder(cfg, model_dt)
    for n in dec2.param_names():
        dec2.load_param(n, to_storage(want_params[n], model_dt))
    logits2, _ = dec2.forward(ids)
    assert np.array_equal(logits, logits2)
    dec.close()
    dec2.close()


def test_sharded_checkpoint_and_index(hip, tmp_path):
    from rai_amd.models import safetensors_index_files
    cfg = small_cfg()
    master = nonzero_params(cfg, seed=3)
    names = sorted(master)
    shard_a = {n: master[n] for n in names[::2]}
    shard_b = {n: master[n] for n in names[1::2]}
    write_safetensors(tmp_path / "model-00001-of-00002.safetensors", shard_a, "F32")
    write_safetensors(tmp_path / "model-00002-of-00002.safetensors", shard_b, "F32")
    weight_map = {n: "model-00001-of-00002.safetensors" for n in shard_a}
    weight_map.update({n: "model-00002-of-00002.safetensors" for n in shard_b})
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps({"metadata": {"total_size": 1}, "weight_map": weight_map}))
    files = safetensors_index_files(tmp_path / "model.safetensors.index.json")
    assert files == [str(tmp_path / "model-00001-of-00002.safetensors"), str(tmp_path / "model-00002-of-00002.safetensors")]
    dec = new_decoder(cfg, "f32")
    dec.load_safetensors(files)
    ref = phi2.Model(cfg, master, "f32")
    ids = np.random.Generator(np.random.PCG64(2)).integers(0, cfg.vocab_size, (1, 7)).astype(np.uint32)
    logits, _ = dec.forward(ids)
    assert_close(logits, ref.fwd(ids), "f32", "sharded load")
    dec.close()


def test_load_safetensors_errors(hip, tmp_path):
    from rai_amd._lib import RaiHipError
    cfg = small_cfg()
    master = nonzero_params(cfg)
    dec = new_decoder(cfg, "f32")
    # a parameter missing from every file: Error::ParamNotFound(name)
    missing = "model.layers.1.mlp.fc2.bias"
    write_safetensors(tmp_path / "a.safetensors", {k: v for k, v in master.items() if k != missing}, "F32")
    with pytest.raises(RaiHipError) as e:
        dec.load_safetensors(tmp_path / "a.safetensors")
    assert e.value.status == -9 and missing in str(e.value)
    # wrong element count
    bad = dict(master)
    bad["model.final_layernorm.weight"] = np.ones(cfg.hidden_size + 1, np.float32)
    write_safetensors(tmp_path / "b.safetensors", bad, "F32")
    with pytest.raises(RaiHipError) as e:
        dec.load_safetensors(tmp_path / "b.safetensors")
    assert e.value.status == -2 and "model.final_layernorm.weight" in str(e.value)
    # right element count, wrong shape: a transposed matrix must not load
    bad = dict(master)
    name = "model.layers.0.mlp.fc1.weight"
    bad[name] = np.ascontiguousarray(master[name].T)
    write_safetensors(tmp_path / "b2.safetensors", bad, "F32")
    with pytest.raises(RaiHipError) as e:
        dec.load_safetensors(tmp_path / "b2.safetensors")
    assert e.value.status == -2 and name in str(e.value)
    # a header whose shape describes far more elements than the file holds
    blob = (tmp_path / "a.safetensors").read_bytes()
    hlen = struct.unpack("<Q", blob[:8])[0]
    import json as _json
    hdr = _json.loads(blob[8:8 + hlen])
    first = next(k for k in hdr if k != "__metadata__")
    hdr[first]["shape"] = [2 ** 40, 2 ** 40]
    h2 = _json.dumps(hdr).encode()
    (tmp_path / "b3.safetensors").write_bytes(struct.pack("<Q", len(h2)) + h2 + blob[8 + hlen:])
    with pytest.raises(RaiHipError) as e:
        dec.load_safetensors(tmp_path / "b3.safetensors")
    assert e.value.status == -10
    # integer tensor where a floating parameter is expected
    write_safetensors(tmp_path / "c.safetensors", master, {k: ("I64" if k == "model.final_layernorm.bias" else "F32") for k in master})
    with pytest.raises(RaiHipError) as e:
        dec.load_safetensors(tmp_path / "c.safetensors")
    assert e.value.status == -1 and "model.final_layernorm.bias" in str(e.value)
    # truncated file, missing file
    (tmp_path / "d.safetensors").write_bytes(struct.pack("<Q", 1 << 40) + b"{}")
    with pytest.raises(RaiHipError) as e:
        dec.load_safetensors(tmp_path / "d.safetensors")
    assert e.value.status == -10
    with pytest.raises(RaiHipError) as e:
        dec.load_safetensors(tmp_path / "nope.safetensors")
    assert e.value.status == -10
    dec.close()
