"""Host-side logic of the lazy graph (no GPU): builders and their shape rules, Err
nodes, the evaluation order, reference counting and the dispatcher table.
Mirrors rai-core/tests/shape.rs and the metadata assertions of rai-core/tests/ops.rs."""
import ctypes
import re
from pathlib import Path

import numpy as np
import pytest

from rai_amd import graph as g
from rai_amd.graph import Tensor

ROOT = Path(__file__).resolve().parents[1]


def test_library_exports_every_graph_symbol():
    from rai_amd import _lib
    text = (ROOT / "include" / "rai_graph.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = sorted(set(re.findall(r"\b(rai_(?!hip_)\w+)\s*\(", text)))
    so = ctypes.CDLL(str(_lib.LIB_PATH))
    assert len(names) >= 40
    for n in names:
        assert hasattr(so, n), f"{n} declared in rai_graph.h but not exported"
    assert set(names) == set(_lib.GRAPH_PROTOTYPES), sorted(set(names) ^ set(_lib.GRAPH_PROTOTYPES))
    enum = text[text.index("typedef enum rai_op_kind {"):text.index("} rai_op_kind;")]
    kinds = [n for n, _ in re.findall(r"RAI_OP_(\w+)\s*=\s*(\d+)", enum)]
    assert [k.replace("_", "").lower() for k in kinds] == [k.lower() for k in g.OP_KINDS]


def test_building_is_lazy_and_metadata_follows_the_reference():
    a = Tensor.ones((2, 3), "f32")
    b = Tensor.full(2.0, (3,), "f32")
    c = a + b                       # rhs is wrapped in a Broadcast node (ops/mod.rs:298-340)
    assert c.shape == (2, 3) and c.dtype == "f32" and c.op == "Binary" and not c.is_evaluated()
    assert c.num_inputs() == 2
    s = c * 2.0                     # scalar -> Full<f32> of c's shape (full.rs:85-92)
    assert s.shape == (2, 3) and s.op == "Binary"
    h = Tensor.ones((4,), "bf16") * 2.0   # Full<f32> then ToDType(bf16)
    order = g.eval_order([h])
    assert len(order) == 4          # ones, Full, ToDType, Binary
    assert a.to_dtype("f32").id == a.id          # to_dtype.rs:45-55 same dtype returns self
    assert a.reshape((2, 3)).id == a.id          # reshape.rs:50-53 equal shape returns self
    assert a.reshape((3, 2)).op == "Reshape"
    assert a.argmax(-1).dtype == "u32" and a.argmax(-1).shape == (2,) and a.argmax(0, True).shape == (1, 3)
    assert a.sum((0, 1)).shape == () and a.sum(1, True).shape == (2, 1)
    assert a.eq(a).dtype == "u8"
    assert a.transpose(0, 1).shape == (3, 2) and a.t().shape == (3, 2)
    assert a.narrow(1, 1, 2).shape == (2, 2)
    assert a.unsqueeze(0).shape == (1, 2, 3) and a.unsqueeze(-1).shape == (2, 3, 1)
    assert g.cat([a, a, a], 0).shape == (6, 3) and g.cat([a, a], -1).shape == (2, 6)
    ids = Tensor.from_array(np.array([[1, 0], [2, 2]], np.uint32), "u32")
    assert a.index_select(1, ids).shape == (2, 4)   # index.elem_count() (index_select.rs:52-61)
    assert Tensor.arange(0, 10, 3).shape == (4,)
    # gather takes the index's shape (gather.rs:47-60); index_add / scatter_add keep x's (index_add.rs:52-62)
    gi = Tensor.from_array(np.zeros((5, 3), np.uint32), "u32")
    assert a.gather(0, gi).shape == (5, 3) and a.gather(0, gi).op == "Gather" and a.gather(0, gi).num_inputs() == 2
    one = Tensor.from_array(np.array([1, 1, 0, 0], np.uint8), "u8")
    ia = a.index_add(0, one, Tensor.ones((4, 3), "f32"))
    assert ia.shape == (2, 3) and ia.op == "IndexAdd" and ia.num_inputs() == 3
    sa = a.scatter_add(0, gi, Tensor.ones((5, 3), "f32"))
    assert sa.shape == (2, 3) and sa.op == "ScatterAdd"
    assert a.gather(1, gi).op == "Err"                                  # extents off the dim differ
    assert a.index_add(0, one, Tensor.ones((3, 3), "f32")).op == "Err"   # source extent != len(index)
    assert a.scatter_add(0, gi, Tensor.ones((4, 3), "f32")).op == "Err"  # index and source shapes differ


@pytest.mark.parametrize("lhs,rhs,out", [((2, 3), (3,), (2, 3)), ((1, 3), (2, 1), (2, 3)), ((4, 1, 5), (7, 1), (4, 7, 5)),
                                          ((), (2, 2), (2, 2))])
def test_broadcast_rule(lhs, rhs, out):
    assert (Tensor.ones(lhs) + Tensor.ones(rhs)).shape == out


def test_matmul_shape_rule():
    # rai-core/src/shape.rs:130-160 and rank-1 promotion of ops/matmul.rs:34-70
    assert Tensor.ones((2, 3)).matmul(Tensor.ones((3, 4))).shape == (2, 4)
    assert Tensor.ones((5, 2, 3)).matmul(Tensor.ones((3, 4))).shape == (5, 2, 4)
    assert Tensor.ones((1, 6, 2, 3)).matmul(Tensor.ones((5, 1, 3, 4))).shape == (5, 6, 2, 4)
    assert Tensor.ones((3,)).matmul(Tensor.ones((3, 4))).shape == (4,)
    assert Tensor.ones((2, 3)).matmul(Tensor.ones((3,))).shape == (2,)
    assert Tensor.ones((3,)).matmul(Tensor.ones((3,))).shape == ()


def test_err_nodes_surface_at_eval():
    # a builder never fails: the node carries the error (ops/err.rs) and eval reports it
    bad = Tensor.ones((2, 3)).matmul(Tensor.ones((4, 5)))
    assert bad.op == "Err" and "IncompatibleShape" in bad.error and "[2, 3]" in bad.error
    assert (Tensor.ones((2, 3)) + Tensor.ones((4,))).op == "Err"
    assert Tensor.ones((2, 3)).reshape((7,)).op == "Err"
    downstream = bad.tanh() + 1.0
    assert downstream.op == "Binary"
    with pytest.raises(g.RaiHipError) as e:
        g.eval_order([downstream])
    assert e.value.status == -2 and "IncompatibleShape" in str(e.value)


def test_eval_order_is_a_topological_order_that_visits_shared_nodes_once():
    x = Tensor.ones((8,))
    y = x.exp()
    z = (y + y.tanh()) * y          # y is shared by three consumers
    order = g.eval_order([z])
    assert len(order) == len(set(order))
    pos = {i: k for k, i in enumerate(order)}
    assert pos[x.id] < pos[y.id] < pos[z.id] and order[-1] == z.id
    # several outputs: nodes reached from the first output are not repeated for the second
    w = y.sin()
    both = g.eval_order([z, w])
    assert both[:len(order)] == order and both[-1] == w.id and len(both) == len(order) + 1


def test_reference_counting_frees_long_chains_without_recursion():
    t = Tensor.ones((4,))
    for _ in range(50000):          # release walks the chain iteratively
        t = t.neg()
    assert t.shape == (4,)
    del t


def test_dispatcher_table():
    assert g.dispatch_has_rule("MatMul") and g.dispatch_has_rule("Softmax") and not g.dispatch_has_rule("Err")
    g.dispatch_unregister("Softmax")
    try:
        assert not g.dispatch_has_rule("Softmax")
    finally:
        g.dispatch_register_builtin("Softmax")
    assert g.dispatch_has_rule("Softmax")


def test_to_device_on_the_same_device_is_the_same_tensor():
    # ops/to_device.rs:49-52: x.to_device(x.device()) returns x itself, no node is added
    x = Tensor.ones((2, 3), "f32", dev=0)
    y = x.to_device(0)
    assert y.id == x.id and y.device == 0
    z = x.neg().to_device(1)        # another device: a ToDevice node on the target device, same shape and dtype
    assert z.device == 1 and z.shape == (2, 3) and z.op == "ToDevice" and z.dtype == "f32"
    assert g.dispatch_has_rule("ToDevice")
