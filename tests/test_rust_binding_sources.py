"""The Rust side of the boundary (integration/rai-core) cannot be compiled here, so these checks keep its text
honest against what can be checked: the FFI declarations are exactly what the generator derives from
include/rai_hip.h, every entry point of the header has a Rust caller, and every primitive the reference's
register_backend! lists is either given an `impl Eval<Hip, ops::X>` and registered, or named as deliberately
unregistered."""
import re
import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parents[1]
RS = ROOT / "integration" / "rai-core" / "src" / "backend"

# the op types of register_backend! (rai-core/src/dispatch.rs:41-157), generics without their dtype
REFERENCE_OPS = """Full Random Normal Arange FromArray Concatenate Add Sub Mul Div MatMul Equal NotEqual Greater
GreaterEqual Less LessEqual Maximum Minimum Sin Cos Tanh Negative Square Powf Sqrt Rsqrt Sign Abs Exp Log Log2 Log10
ToDType Softmax LogSoftmax Erf ToDevice Gather IndexSelect Narrow Where ScatterAdd IndexAdd Transpose Reshape Permute
Broadcast ToContiguous ReduceSum ReduceMax ReduceMin ArgMax ArgMin Conv1d Conv2d ConvTranspose1d ConvTranspose2d
MaxPool1d MaxPool2d AvgPool1d AvgPool2d UpsampleNearest1d UpsampleNearest2d""".split()
NO_KERNEL = {"Random", "Normal", "Conv1d", "Conv2d", "ConvTranspose1d", "ConvTranspose2d", "MaxPool1d", "MaxPool2d",
             "AvgPool1d", "AvgPool2d", "UpsampleNearest1d", "UpsampleNearest2d"}


def test_hip_sys_is_what_the_generator_writes():
    r = subprocess.run([sys.executable, str(ROOT / "integration" / "gen_hip_sys.py"), "--check"])
    assert r.returncode == 0, "integration/rai-core/src/backend/hip_sys.rs is out of date: run integration/gen_hip_sys.py"


def test_every_header_entry_point_has_a_rust_caller():
    header = re.sub(r"/\*.*?\*/", "", (ROOT / "include" / "rai_hip.h").read_text(), flags=re.S)
    declared = set(re.findall(r"\b(rai_hip_\w+)\s*\(", header))
    callers = (RS / "hip.rs").read_text() + (RS / "hip_fused.rs").read_text() + (RS / "hip_sys.rs").read_text().split('extern "C" {')[1].split("}")[1]
    measurement_only = {"rai_hip_timer_create", "rai_hip_timer_start", "rai_hip_timer_stop", "rai_hip_timer_elapsed_ms",
                        "rai_hip_timer_destroy", "rai_hip_decoder_time_decode_step", "rai_hip_decoder_time_decode_linear",
                        "rai_hip_d2d"}
    missing = sorted(n for n in declared - measurement_only if not re.search(rf"\b{n}\b", callers))
    assert not missing, f"no Rust caller for {missing}"


def test_every_reference_op_is_implemented_or_named_as_unregistered():
    src = (RS / "hip.rs").read_text()
    # expand the two macro invocations that stamp out the binary / unary impls
    stamped = set()
    for body in re.findall(r"hip_(?:binary|unary)!\((.*?)\);", src, flags=re.S):
        stamped |= set(re.findall(r"(\w+)\s*=>", body))
    direct = set(re.findall(r"Eval<Hip, ops::(\w+)", src))
    implemented = stamped | direct
    reg = src[src.index("pub(crate) fn register_hip"):]
    registered = set(re.findall(r"\b([A-Z]\w+)\b", " ".join(re.findall(r"(?:plain|per_dtype)!\((.*?)\);", reg, flags=re.S))))
    registered |= set(re.findall(r"ops::(\w+)", reg))
    registered -= {"U8", "U32", "I64", "F16", "BF16", "F32", "F64"}
    for op in REFERENCE_OPS:
        if op in NO_KERNEL:
            assert op not in implemented and op in src, f"{op} must be named as unregistered in hip.rs"
        else:
            assert op in implemented, f"no impl Eval<Hip, ops::{op}>"
            assert op in registered, f"ops::{op} is implemented but not registered"
    assert implemented - set(REFERENCE_OPS) - {"X"} == set(), implemented - set(REFERENCE_OPS)   # "ops::X" in the prose


def test_graph_bridge_mirrors_every_builder_and_every_registered_op():
    """backend/hip_graph.rs hands a whole tape to the library's evaluator: every node builder of include/rai_graph.h
    has a caller there, every primitive that hip.rs registers is mirrored (ToDevice excepted: a tape that crosses
    devices is left to the per-node loop), and the two storage calls of the bridge are used."""
    header = re.sub(r"/\*.*?\*/", "", (ROOT / "include" / "rai_graph.h").read_text(), flags=re.S)
    builders = set(re.findall(r"^rai_tensor \*\s*(rai_\w+)\s*\(", header, flags=re.M))
    assert len(builders) >= 25
    src = (RS / "hip_graph.rs").read_text()
    missing = sorted(b for b in builders - {"rai_to_device"} if not re.search(rf"\b{b}\b", src))
    assert not missing, f"hip_graph.rs never calls {missing}"
    for call in ("rai_eval", "rai_tensor_storage", "rai_tensor_buffer", "rai_from_storage", "set_data", "strong_count"):
        assert call in src, call
    for op in REFERENCE_OPS:
        if op in NO_KERNEL or op == "ToDevice":
            continue
        assert re.search(rf"\b{op}\b", src), f"hip_graph.rs does not mirror ops::{op}"
    sys_rs = (RS / "hip_graph_sys.rs").read_text()
    for b in builders | {"rai_eval", "rai_tensor_buffer", "rai_from_storage"}:
        assert f"pub fn {b}(" in sys_rs, b
