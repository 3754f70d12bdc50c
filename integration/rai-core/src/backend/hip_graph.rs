//! `eval()` for tapes that live on a `Hip` device: the whole tape goes to the evaluator inside librai_hip.so.
//!
//! rai's `eval` (eval.rs:31-51) calls one `Eval::eval` per node, so on its own the `Hip` backend launches one kernel
//! per primitive: ~4 300 launches for a Phi-2 token.  The library's evaluator (`include/rai_graph.h`) takes a whole
//! tape instead and runs two passes over it before launching anything: a composition pass (Linear with bias /
//! activation / residual, LayerNorm, RmsNorm, rotary embedding, the attention block, key / value cache appends in
//! place) and an elementwise-fusion pass.  This file is the bridge: it mirrors the sorted tape node for node through
//! the `rai_*` builders, hands operands that already have data across as they are (`rai_from_storage`), runs
//! `rai_eval`, and puts the results back into the rai tensors with `set_data` (tensor.rs:151-165).  Model code
//! (`rai-models/src/llm/*.rs`), rai-nn modules, `grad` / `vjp` stay unchanged.
//!
//! To add to a rai 0.11 checkout next to `hip.rs` (not compiled in the repository this file ships in):
//!   * `rai-core/src/backend/mod.rs`: `#[cfg(feature = "hip")] mod hip_graph_sys; #[cfg(feature = "hip")] pub(crate) mod hip_graph;`
//!   * `rai-core/src/tensor.rs`: `pub(crate) fn strong_count(&self) -> usize { Rc::strong_count(&self.0) }`
//!   * `rai-core/src/eval.rs`, first lines of `eval` after the tape is built (:32):
//!       `#[cfg(feature = "hip")]`
//!       `if crate::backend::hip_graph::eval_tape(&tape, args.retain_graph()) { return Ok(()); }`
//!     (a tape the bridge declines -- another device, an op without a builder, `retain_graph` -- falls through to the
//!     per-node loop, which on `Hip` dispatches to `backend/hip.rs`).
use super::hip::{dtype_code, Hip, HipData, HipScalar};
use super::hip_graph_sys::*;
use super::hip_sys::*;
use crate::{ops, Op, Tensor, Type, BF16, F16, F32, F64, I64, U32, U8};
use std::collections::HashMap;
use std::ffi::c_void;

/// Owns one reference of a library node for the duration of the call.
struct Node(*mut RaiTensor);
impl Drop for Node {
    fn drop(&mut self) {
        if !self.0.is_null() {
            unsafe { rai_tensor_release(self.0) };
        }
    }
}

fn dims_i64(shape: &[usize]) -> Vec<i64> {
    shape.iter().map(|&d| d as i64).collect()
}

/// The library node for an operand that already has data: a view of its `HipData` allocation.
fn leaf(t: &Tensor, dev: i32) -> Option<Node> {
    let data = t.get_data::<HipData>()?;
    let n = unsafe { rai_from_storage(data.desc(), data.buffer(), dev) };
    (!n.is_null()).then(|| Node(n))
}

macro_rules! per_dtype {
    ($any:expr, $op:ident, |$o:ident, $code:ident| $body:expr) => {{
        let any = $any;
        if let Some($o) = any.downcast_ref::<ops::$op<U8>>() { let $code = RAI_U8; Some($body) }
        else if let Some($o) = any.downcast_ref::<ops::$op<U32>>() { let $code = RAI_U32; Some($body) }
        else if let Some($o) = any.downcast_ref::<ops::$op<I64>>() { let $code = RAI_I64; Some($body) }
        else if let Some($o) = any.downcast_ref::<ops::$op<F16>>() { let $code = RAI_F16; Some($body) }
        else if let Some($o) = any.downcast_ref::<ops::$op<BF16>>() { let $code = RAI_BF16; Some($body) }
        else if let Some($o) = any.downcast_ref::<ops::$op<F32>>() { let $code = RAI_F32; Some($body) }
        else if let Some($o) = any.downcast_ref::<ops::$op<F64>>() { let $code = RAI_F64; Some($body) }
        else { None }
    }};
}

/// One tape node as a library node: the builder that corresponds to its op, applied to the mirrored inputs.
/// `None`: no builder for this op (Random, Normal, convolutions, pooling, upsampling, FlashAttention, ToDevice
/// across devices): the caller leaves the whole tape to the per-node loop.
fn mirror(t: &Tensor, ins: &[*mut RaiTensor], dev: i32) -> Option<*mut RaiTensor> {
    let op: &dyn Op = t.op();
    let any = op.as_any();
    let shape = dims_i64(t.shape());
    let rank = shape.len() as i32;
    macro_rules! unary {
        ($($ty:ident => $code:ident),*) => {$(
            if any.is::<ops::$ty>() { return Some(unsafe { rai_unary($code, ins[0], 0.0) }); }
        )*};
    }
    macro_rules! binary {
        ($($ty:ident => $code:ident),*) => {$(
            if any.is::<ops::$ty>() { return Some(unsafe { rai_binary($code, ins[0], ins[1]) }); }
        )*};
    }
    unary!(Sin => RAI_UN_SIN, Cos => RAI_UN_COS, Tanh => RAI_UN_TANH, Negative => RAI_UN_NEG, Square => RAI_UN_SQUARE,
           Sqrt => RAI_UN_SQRT, Rsqrt => RAI_UN_RSQRT, Sign => RAI_UN_SIGN, Abs => RAI_UN_ABS, Exp => RAI_UN_EXP,
           Log => RAI_UN_LOG, Log2 => RAI_UN_LOG2, Log10 => RAI_UN_LOG10, Erf => RAI_UN_ERF);
    binary!(Add => RAI_BIN_ADD, Sub => RAI_BIN_SUB, Mul => RAI_BIN_MUL, Div => RAI_BIN_DIV, Maximum => RAI_BIN_MAXIMUM,
            Minimum => RAI_BIN_MINIMUM, Equal => RAI_BIN_EQ, NotEqual => RAI_BIN_NE, Greater => RAI_BIN_GT,
            GreaterEqual => RAI_BIN_GE, Less => RAI_BIN_LT, LessEqual => RAI_BIN_LE);
    if any.is::<ops::MatMul>() {
        return Some(unsafe { rai_matmul(ins[0], ins[1]) });
    }
    if let Some(n) = per_dtype!(any, Full, |o, code| unsafe { rai_full(o.val.to_f64_lossless(), code, shape.as_ptr(), rank, dev) }) {
        return Some(n);
    }
    if let Some(n) = per_dtype!(any, Arange, |o, code| unsafe {
        rai_arange(o.start.to_f64_lossless(), o.stop.to_f64_lossless(), o.step.to_f64_lossless(), code, dev)
    }) {
        return Some(n);
    }
    if let Some(n) = per_dtype!(any, FromArray, |o, code| unsafe {
        rai_from_array(o.data.as_ptr() as *const c_void, code, shape.as_ptr(), rank, dev)
    }) {
        return Some(n);
    }
    if let Some(n) = per_dtype!(any, ToDType, |_o, code| unsafe { rai_to_dtype(ins[0], code) }) {
        return Some(n);
    }
    if let Some(o) = any.downcast_ref::<ops::Powf<F32>>() {
        return Some(unsafe { rai_unary(RAI_UN_POWF, ins[0], o.exponent as f64) });
    }
    if let Some(o) = any.downcast_ref::<ops::Powf<F64>>() {
        return Some(unsafe { rai_unary(RAI_UN_POWF, ins[0], o.exponent) });
    }
    if let Some(o) = any.downcast_ref::<ops::Powf<BF16>>() {
        return Some(unsafe { rai_unary(RAI_UN_POWF, ins[0], o.exponent.to_f64_lossless()) });
    }
    if let Some(o) = any.downcast_ref::<ops::Powf<F16>>() {
        return Some(unsafe { rai_unary(RAI_UN_POWF, ins[0], o.exponent.to_f64_lossless()) });
    }
    if let Some(o) = any.downcast_ref::<ops::Softmax>() {
        return Some(unsafe { rai_softmax(ins[0], o.dim as i32) });
    }
    if let Some(o) = any.downcast_ref::<ops::LogSoftmax>() {
        return Some(unsafe { rai_log_softmax(ins[0], o.dim as i32) });
    }
    macro_rules! reduce {
        ($($ty:ident => $code:ident),*) => {$(
            if let Some(o) = any.downcast_ref::<ops::$ty>() {
                let dims: Vec<i32> = o.dims.iter().map(|&d| d as i32).collect();
                return Some(unsafe { rai_reduce($code, ins[0], dims.as_ptr(), dims.len() as i32, o.keep_dim as i32) });
            }
        )*};
    }
    reduce!(ReduceSum => RAI_RED_SUM, ReduceMax => RAI_RED_MAX, ReduceMin => RAI_RED_MIN);
    if let Some(o) = any.downcast_ref::<ops::ArgMax>() {
        return Some(unsafe { rai_argmax(ins[0], o.dim as i32, o.keep_dim as i32) });
    }
    if let Some(o) = any.downcast_ref::<ops::ArgMin>() {
        return Some(unsafe { rai_argmin(ins[0], o.dim as i32, o.keep_dim as i32) });
    }
    if let Some(o) = any.downcast_ref::<ops::IndexSelect>() {
        return Some(unsafe { rai_index_select(ins[0], o.dim as i32, ins[1]) });
    }
    if let Some(o) = any.downcast_ref::<ops::Gather>() {
        return Some(unsafe { rai_gather(ins[0], o.dim as i32, ins[1]) });
    }
    // IndexAdd / ScatterAdd: rai orders the inputs [x, source, index] (ops/index_add.rs:52-62)
    if let Some(o) = any.downcast_ref::<ops::IndexAdd>() {
        return Some(unsafe { rai_index_add(ins[0], o.dim as i32, ins[2], ins[1]) });
    }
    if let Some(o) = any.downcast_ref::<ops::ScatterAdd>() {
        return Some(unsafe { rai_scatter_add(ins[0], o.dim as i32, ins[2], ins[1]) });
    }
    if let Some(o) = any.downcast_ref::<ops::Narrow>() {
        return Some(unsafe { rai_narrow(ins[0], o.dim as i32, o.start as i64, o.len as i64) });
    }
    if let Some(o) = any.downcast_ref::<ops::Concatenate>() {
        return Some(unsafe { rai_concatenate(ins.as_ptr(), ins.len() as i32, o.dim as i32) });
    }
    if any.is::<ops::Where>() {
        // inputs are ordered [on_true, on_false, cond] (ops/where.rs:37-45)
        return Some(unsafe { rai_where(ins[2], ins[0], ins[1]) });
    }
    if let Some(o) = any.downcast_ref::<ops::Transpose>() {
        return Some(unsafe { rai_transpose(ins[0], o.dim0 as i32, o.dim1 as i32) });
    }
    if let Some(o) = any.downcast_ref::<ops::Permute>() {
        let dims: Vec<i32> = o.dims.iter().map(|&d| d as i32).collect();
        return Some(unsafe { rai_permute(ins[0], dims.as_ptr(), dims.len() as i32) });
    }
    if any.is::<ops::Reshape>() {
        return Some(unsafe { rai_reshape(ins[0], shape.as_ptr(), rank) });
    }
    if any.is::<ops::Broadcast>() {
        return Some(unsafe { rai_broadcast_to(ins[0], shape.as_ptr(), rank) });
    }
    if any.is::<ops::ToContiguous>() {
        return Some(unsafe { rai_to_contiguous(ins[0]) });
    }
    None
}

/// Evaluates `tape` (topologically sorted, un-evaluated nodes only: utils.rs:12-66) through the library's evaluator.
/// Returns false, having changed nothing, when the tape is not one it serves; eval.rs then runs its own loop.
pub(crate) fn eval_tape(tape: &[Tensor], retain_graph: bool) -> bool {
    // The passes fold nodes away, so their tensors receive no data: fine for a forward evaluation whose interior
    // nobody holds, not for a graph that is kept for a later transform.
    if retain_graph || tape.is_empty() {
        return false;
    }
    let dev = match tape[0].device().as_any().downcast_ref::<Hip>() {
        Some(h) => h.id() as i32,
        None => return false,
    };
    if tape.iter().any(|t| t.device().as_any().downcast_ref::<Hip>().map(|h| h.id() as i32) != Some(dev)) {
        return false;
    }
    // edges of the tape per node: a tensor referenced from anywhere else (a handle the caller keeps, the model's key /
    // value cache) has a strong count above these edges + the tape's own clone, and must come out with data
    let mut edges: HashMap<usize, usize> = HashMap::new();
    for t in tape {
        for i in t.inputs().iter() {
            *edges.entry(i.id()).or_insert(0) += 1;
        }
    }
    let mut nodes: HashMap<usize, Node> = HashMap::with_capacity(tape.len() * 2);
    let mut held: Vec<*mut RaiTensor> = Vec::new(); // library nodes of tensors observable from outside
    for t in tape {
        let mut ins: Vec<*mut RaiTensor> = Vec::with_capacity(t.inputs().len());
        for i in t.inputs().iter() {
            if !nodes.contains_key(&i.id()) {
                match leaf(i, dev) {
                    Some(n) => { nodes.insert(i.id(), n); }
                    None => return false, // an evaluated input that is not Hip storage
                }
            }
            ins.push(nodes[&i.id()].0);
        }
        let n = match mirror(t, &ins, dev) {
            Some(n) if !n.is_null() => n,
            _ => return false,
        };
        // shape / dtype as rai computed them, or the mirror is not the same graph
        if unsafe { rai_tensor_rank(n) } as usize != t.shape().len() || unsafe { rai_tensor_dtype(n) } != dtype_code(t.dtype()) {
            unsafe { rai_tensor_release(n) };
            return false;
        }
        if t.strong_count() > edges.get(&t.id()).copied().unwrap_or(0) + 1 {
            held.push(n); // the reference kept in `nodes` is the handle "outside the tape" that the planner sees
        }
        nodes.insert(t.id(), Node(n));
    }
    // Every node that must come out with data is requested as an output; the others lose this function's reference
    // first, so the library sees them referenced by graph edges only (its condition for folding a node away).
    let outputs: Vec<*mut RaiTensor> = held;
    let keep: std::collections::HashSet<usize> = outputs.iter().map(|&p| p as usize).collect();
    for t in tape {
        if let Some(n) = nodes.get_mut(&t.id()) {
            if !keep.contains(&(n.0 as usize)) {
                // consumers retain their inputs, so the node stays alive exactly as long as the graph needs it
                unsafe { rai_tensor_release(n.0) };
                n.0 = std::ptr::null_mut();
            }
        }
    }
    check(unsafe { rai_eval(outputs.as_ptr(), outputs.len() as i32, 0) });
    for t in tape {
        let n = match nodes.get(&t.id()) {
            Some(n) if !n.0.is_null() => n.0,
            _ => continue, // folded away or evaluated inside the library only: nobody can ask for it
        };
        let mut view = RaiHipTensor { data: std::ptr::null_mut(), dtype: 0, rank: 0, shape: [1; 8], stride: [0; 8], offset: 0 };
        check(unsafe { rai_tensor_storage(n, &mut view) });
        let buf = unsafe { rai_tensor_buffer(n) };
        t.set_data(HipData::adopt(dev, buf, view)); // retains `buf`; asserts shape and dtype (tensor.rs:151-165)
        t.detach();
    }
    true
}
