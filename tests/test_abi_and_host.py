"""CPU-side checks of the boundary: the shared library loads and exports every
symbol include/rai_hip.h declares (no compute call is made), the ctypes mirror
matches the header, and the host-side view / shape logic behaves like the
reference's metadata rules."""
import ctypes
import re
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parents[1]


def header_functions(header="rai_hip.h"):
    text = (ROOT / "include" / header).read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(rai_hip_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from rai_amd import _lib
    assert _lib.LIB_PATH.exists(), "librai_hip.so is not built (python -m rai_amd.build)"
    so = ctypes.CDLL(str(_lib.LIB_PATH))
    names = header_functions()
    assert len(names) >= 45
    for n in names:
        assert hasattr(so, n), f"{n} declared in rai_hip.h but not exported"
    declared = set(names)
    bound = set(_lib.PROTOTYPES) | {"rai_hip_last_error"}
    assert bound == declared, (sorted(bound - declared), sorted(declared - bound))
    # the measurement aid of include/rai_hip_peaks.h
    peaks = header_functions("rai_hip_peaks.h")
    assert peaks == sorted(_lib.PEAK_PROTOTYPES), peaks
    for n in peaks:
        assert hasattr(so, n), f"{n} declared in rai_hip_peaks.h but not exported"
    text = (ROOT / "include" / "rai_hip_peaks.h").read_text()
    for name, val in re.findall(r"RAI_PEAK_(\w+)\s*=\s*(\d+)", text):
        assert _lib.PEAK_KINDS[name.lower()] == int(val)
    # every header of include/ is covered by one of the checks of this file or of test_graph_host.py
    assert sorted(p.name for p in (ROOT / "include").glob("*.h")) == ["rai_graph.h", "rai_hip.h", "rai_hip_peaks.h"]


def test_ctypes_structs_match_header_layout():
    from rai_amd import _lib
    assert ctypes.sizeof(_lib.TensorDesc) == 8 + 4 + 4 + 8 * 8 + 8 * 8 + 8
    text = (ROOT / "include" / "rai_hip.h").read_text()
    body = text[text.index("typedef struct rai_hip_decoder_config {"):text.index("} rai_hip_decoder_config;")]
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    fields = re.findall(r"(?:int32_t|double)\s+(\w+)\s*;", body)
    assert fields == [f[0] for f in _lib.DecoderConfig._fields_]
    enum = text[text.index("typedef enum rai_hip_unary_op {"):text.index("} rai_hip_unary_op;")]
    for name, val in re.findall(r"RAI_UN_(\w+)\s*=\s*(\d+)", enum):
        assert _lib.UNARY[name.lower()] == int(val)
    enum = text[text.index("typedef enum rai_hip_binary_op {"):text.index("} rai_hip_binary_op;")]
    for name, val in re.findall(r"RAI_BIN_(\w+)\s*=\s*(\d+)", enum):
        assert _lib.BINARY[{"maximum": "maximum", "minimum": "minimum"}.get(name.lower(), name.lower())] == int(val)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from rai_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", tmp_path / "nope.so")
    with pytest.raises(_lib.RaiHipError):
        _lib.load()


def test_broadcast_shape_rules():
    # rai-core/src/shape.rs:88-127 and rai-core/tests/shape.rs
    from rai_amd.ops import broadcast_shapes
    assert broadcast_shapes((2, 3), (3,)) == (2, 3)
    assert broadcast_shapes((4, 1, 5), (3, 1)) == (4, 3, 5)
    assert broadcast_shapes((), (2, 2)) == (2, 2)
    with pytest.raises(ValueError):
        broadcast_shapes((2, 3), (4,))


def test_view_metadata_without_touching_the_device():
    from rai_amd.hip import HipTensor

    class FakeBuf:
        ptr, dev = 0x1000, 0

    t = HipTensor(FakeBuf(), "f32", (2, 3, 4))
    assert t.strides == (12, 4, 1) and t.is_contiguous()
    tr = t.transpose(0, 2)
    assert tr.shape == (4, 3, 2) and tr.strides == (1, 4, 12) and not tr.is_contiguous()
    n = t.narrow(1, 1, 2)
    assert n.shape == (2, 2, 4) and n.offset == 4 and n.strides == (12, 4, 1)
    b = HipTensor(FakeBuf(), "bf16", (3,)).broadcast_to((5, 2, 3))
    assert b.strides == (0, 0, 1)
    d = tr.desc()
    assert d.rank == 3 and list(d.shape)[:3] == [4, 3, 2] and list(d.stride)[:3] == [1, 4, 12] and d.dtype == 5
    with pytest.raises(ValueError):
        t.narrow(1, 2, 2)
    with pytest.raises(ValueError):
        HipTensor(FakeBuf(), "f32", (3,)).broadcast_to((4,))


def test_synthetic_weights_are_seeded_and_shaped():
    from rai_amd import synthetic
    a = synthetic.tensor("model.layers.0.mlp.fc1.weight", 1000, seed=0)
    b = synthetic.tensor("model.layers.0.mlp.fc1.weight", 1000, seed=0)
    c = synthetic.tensor("model.layers.1.mlp.fc1.weight", 1000, seed=0)
    assert np.array_equal(a, b) and not np.array_equal(a, c)
    assert abs(float(a.std()) - 0.02) < 0.003
    assert np.all(synthetic.tensor("model.layers.0.mlp.fc1.bias", 8) == 0)
    assert np.all(synthetic.tensor("model.final_layernorm.weight", 8) == 1)
    import torch
    x = np.random.default_rng(0).standard_normal(1000).astype(np.float32)
    assert np.array_equal(synthetic.f32_to_bf16_bits(x).view(np.int16),
                          torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy())
    p = synthetic.prompt(51200, 1, 512, seed=1)
    assert p.shape == (1, 512) and p.dtype == np.uint32 and p.max() < 51200


def test_bench_refuses_multi_gpu():
    import subprocess
    import sys
    r = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "one GPU" in (r.stderr + r.stdout)


def test_safetensors_index_files_host_only(tmp_path):
    """ext::hf::load_safetensors (rai/src/lib.rs:17-42) minus the download: distinct weight_map values,
    resolved against the index's directory; missing / invalid weight_map is an error.  No GPU involved."""
    import json

    from rai_amd._lib import RaiHipError
    from rai_amd.models import safetensors_index_files
    idx = tmp_path / "model.safetensors.index.json"
    idx.write_text(json.dumps({"metadata": {}, "weight_map": {"a.weight": "s2.safetensors", "b.weight": "s1.safetensors",
                                                               "c.weight": "s2.safetensors", "odd": 3}}))
    assert safetensors_index_files(idx) == [str(tmp_path / "s1.safetensors"), str(tmp_path / "s2.safetensors")]
    idx.write_text(json.dumps({"metadata": {}}))
    with pytest.raises(RaiHipError) as e:
        safetensors_index_files(idx)
    assert e.value.status == -10 and "weight_map" in str(e.value)
    idx.write_text(json.dumps({"weight_map": ["x"]}))
    with pytest.raises(RaiHipError):
        safetensors_index_files(idx)
    idx.write_text("{not json")
    with pytest.raises(RaiHipError):
        safetensors_index_files(idx)


def test_every_environment_knob_of_the_library_is_documented():
    """The library reads a handful of RAI_HIP_* variables (tuning and test aids, most of them read per call).  Each one
    that occurs in the sources has a row in the knob table of the integration notes."""
    knobs = set()
    for src in sorted((ROOT / "rai_amd" / "csrc").iterdir()):
        if src.suffix in (".hip", ".cpp", ".h"):
            knobs |= set(re.findall(r'getenv\("(RAI_HIP_[A-Z0-9_]+)"\)', src.read_text()))
    assert len(knobs) >= 10, knobs
    doc = (ROOT / "INTEGRATION.md").read_text()
    missing = sorted(k for k in knobs if f"`{k}`" not in doc)
    assert not missing, f"not in the knob table: {missing}"
