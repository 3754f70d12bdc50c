/*
 * rai_graph.h — C ABI of the lazy tensor graph, dispatcher and evaluator that
 * sit on top of the kernels of rai_hip.h (same shared library).
 *
 * It mirrors rai-core's evaluation machinery for the `Hip` device:
 *   rai-core/src/tensor.rs:28-37,229   Tensor = ref-counted node {device, dtype, shape, op, inputs, data}
 *   rai-core/src/ops/                   one builder per primitive (shape inference, Err nodes on bad shapes)
 *   rai-core/src/utils.rs:35-66         iterative DFS topological sort that skips evaluated nodes
 *   rai-core/src/dispatch.rs:159-212    (device, op) -> evaluation rule table, runtime registration
 *   rai-core/src/eval.rs:31-51          eval(): per node look up the rule, run it, detach
 * plus the elementwise-fusion pass: maximal single-consumer chains of
 * elementwise primitives (unary, binary, casts, constants) are evaluated by one
 * kernel that applies the same per-node rounding as node-by-node evaluation, so
 * results are bit-identical with fusion on or off.
 *
 * Every function that returns a tensor returns a new reference (release it with
 * rai_tensor_release).  Builders never fail: a shape error yields an Err node
 * (rai-core/src/ops/err.rs) that surfaces when the node is evaluated.
 */
#ifndef RAI_GRAPH_H
#define RAI_GRAPH_H

#include "rai_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct rai_tensor rai_tensor;

/* Primitive kinds: the op types register_backend! enumerates (dispatch.rs:41-157),
 * restricted to the ones a decoder forward builds. */
typedef enum rai_op_kind {
  RAI_OP_FULL = 0,
  RAI_OP_ARANGE = 1,
  RAI_OP_FROM_ARRAY = 2,
  RAI_OP_TO_DTYPE = 3,
  RAI_OP_UNARY = 4,   /* sub-kind = rai_hip_unary_op */
  RAI_OP_BINARY = 5,  /* sub-kind = rai_hip_binary_op */
  RAI_OP_MATMUL = 6,
  RAI_OP_SOFTMAX = 7,
  RAI_OP_LOG_SOFTMAX = 8,
  RAI_OP_REDUCE = 9,  /* sub-kind = rai_hip_reduce_op */
  RAI_OP_ARGMAX = 10,
  RAI_OP_ARGMIN = 11,
  RAI_OP_INDEX_SELECT = 12,
  RAI_OP_NARROW = 13,
  RAI_OP_CONCATENATE = 14,
  RAI_OP_WHERE = 15,
  RAI_OP_TRANSPOSE = 16,
  RAI_OP_RESHAPE = 17,
  RAI_OP_PERMUTE = 18,
  RAI_OP_BROADCAST = 19,
  RAI_OP_TO_CONTIGUOUS = 20,
  RAI_OP_ERR = 21,
  RAI_OP_GATHER = 22,
  RAI_OP_INDEX_ADD = 23,   /* inputs ordered [x, source, index] (ops/index_add.rs:57-59) */
  RAI_OP_SCATTER_ADD = 24, /* inputs ordered [x, source, index] (ops/scatter_add.rs:57) */
  RAI_OP_TO_DEVICE = 25,   /* ToDevice<Hip>: ops/to_device.rs, registered per device at dispatch.rs:117-121 */
  RAI_OP_COUNT_
} rai_op_kind;

/* ---- creation (Tensor::full / ones / zeros, arange, from_array: ops/full.rs, arange.rs, from_array.rs) */
rai_tensor *rai_full(double value, int32_t dtype, const int64_t *shape, int32_t rank, int32_t dev);
rai_tensor *rai_arange(double start, double stop, double step, int32_t dtype, int32_t dev);
/* The host data is copied into the node at build time (FromArray owns its Vec). */
rai_tensor *rai_from_array(const void *host, int32_t dtype, const int64_t *shape, int32_t rank, int32_t dev);

/* ---- primitives (each returns an unevaluated node) */
rai_tensor *rai_to_dtype(rai_tensor *x, int32_t dtype);                       /* ops/to_dtype.rs:45-55 */
rai_tensor *rai_unary(int32_t op, rai_tensor *x, double param);               /* sin..tanh, powf */
rai_tensor *rai_binary(int32_t op, rai_tensor *lhs, rai_tensor *rhs);         /* ops/mod.rs:298-340 (broadcasts) */
rai_tensor *rai_matmul(rai_tensor *lhs, rai_tensor *rhs);                     /* ops/matmul.rs:34-70 */
rai_tensor *rai_softmax(rai_tensor *x, int32_t dim);
rai_tensor *rai_log_softmax(rai_tensor *x, int32_t dim);
rai_tensor *rai_reduce(int32_t op, rai_tensor *x, const int32_t *dims, int32_t ndims, int32_t keep_dim);
rai_tensor *rai_argmax(rai_tensor *x, int32_t dim, int32_t keep_dim);
rai_tensor *rai_argmin(rai_tensor *x, int32_t dim, int32_t keep_dim);
rai_tensor *rai_index_select(rai_tensor *x, int32_t dim, rai_tensor *index);
/* ops/gather.rs:47-60, ops/index_add.rs:52-62, ops/scatter_add.rs:52-60 (the primitives the vjp rules of
 * index_select and gather evaluate); a shape the reference asserts on gives an error node. */
rai_tensor *rai_gather(rai_tensor *x, int32_t dim, rai_tensor *index);
rai_tensor *rai_index_add(rai_tensor *x, int32_t dim, rai_tensor *index, rai_tensor *source);
rai_tensor *rai_scatter_add(rai_tensor *x, int32_t dim, rai_tensor *index, rai_tensor *source);
rai_tensor *rai_narrow(rai_tensor *x, int32_t dim, int64_t start, int64_t len);
rai_tensor *rai_concatenate(rai_tensor *const *xs, int32_t n, int32_t dim);
rai_tensor *rai_where(rai_tensor *cond, rai_tensor *on_true, rai_tensor *on_false);
rai_tensor *rai_transpose(rai_tensor *x, int32_t dim0, int32_t dim1);
rai_tensor *rai_reshape(rai_tensor *x, const int64_t *shape, int32_t rank);   /* same node if shape is equal */
rai_tensor *rai_permute(rai_tensor *x, const int32_t *dims, int32_t rank);
rai_tensor *rai_broadcast_to(rai_tensor *x, const int64_t *shape, int32_t rank);
rai_tensor *rai_to_contiguous(rai_tensor *x);
/* Tensor::to_device (ops/to_device.rs:48-59): x itself (a new reference) when it already lives on Hip(dev),
 * else a ToDevice node on the target device whose rule copies across devices (rai_hip_to_device). */
rai_tensor *rai_to_device(rai_tensor *x, int32_t dev);

/* ---- handles and metadata (tensor.rs) */
void rai_tensor_retain(rai_tensor *t);
void rai_tensor_release(rai_tensor *t);
int32_t rai_tensor_rank(const rai_tensor *t);
int32_t rai_tensor_dtype(const rai_tensor *t);
int32_t rai_tensor_device(const rai_tensor *t);
int32_t rai_tensor_op(const rai_tensor *t);
int32_t rai_tensor_shape(const rai_tensor *t, int64_t *shape_out); /* returns rank */
int32_t rai_tensor_is_evaluated(const rai_tensor *t);
int32_t rai_tensor_num_inputs(const rai_tensor *t);  /* 0 after detach */
uint64_t rai_tensor_id(const rai_tensor *t);
/* Message of an Err node, or NULL. */
const char *rai_tensor_error(const rai_tensor *t);
/* View of the evaluated storage (fails with RAI_ERR_BAD_ARG if not evaluated). */
int rai_tensor_storage(const rai_tensor *t, rai_hip_tensor *out);
/* The two ends of a bridge from a front end that keeps tensor objects of its own (rai-core's Tensor with HipData in
 * its data slot, tensor.rs:28-37,151-165): rai_from_storage wraps data that already exists as an evaluated node (a
 * view into `buf`, an allocation of rai_hip_alloc, which the node retains and releases with itself), and
 * rai_tensor_buffer hands out the allocation an evaluated node's view points into (NULL if not evaluated; the
 * caller retains it with rai_hip_retain if it keeps it). */
rai_tensor *rai_from_storage(const rai_hip_tensor *view, void *buf, int32_t dev);
void *rai_tensor_buffer(const rai_tensor *t);

/* ---- evaluation (eval.rs:31-51).  Returns RAI_OK, RAI_ERR_UNSUPPORTED for a
 * (device, op) pair without a rule (Error::Unimplemented), RAI_ERR_BAD_SHAPE when
 * the graph contains an Err node (Error::Op), or a kernel failure status. */
int rai_eval(rai_tensor *const *outputs, int32_t n, int32_t retain_graph);
/* The order in which rai_eval would visit the un-evaluated nodes behind `outputs`
 * (utils.rs:35-66): writes up to `capacity` node ids, *count receives the tape length. */
int rai_graph_eval_order(rai_tensor *const *outputs, int32_t n, uint64_t *ids, int32_t capacity, int32_t *count);
/* Tensor::as_vec / as_bytes: evaluates if needed, copies the contiguous contents to the host. */
int rai_tensor_to_host(rai_tensor *t, void *dst, size_t bytes);

/* ---- dispatcher (dispatch.rs:181-212) */
/* Remove / restore the rule of a primitive for the Hip device (restoring installs
 * the built-in rule).  Lets callers exercise the Unimplemented path. */
int rai_dispatch_unregister(int32_t op_kind);
int rai_dispatch_register_builtin(int32_t op_kind);
int32_t rai_dispatch_has_rule(int32_t op_kind);

/* ---- fusion passes: control and counters */
/* Elementwise pass: chains of elementwise primitives as one launch, bit-identical with node-by-node evaluation. */
int rai_graph_set_fusion(int32_t enabled);
/* Composition pass: the compositions rai's modules are made of -- Linear with bias (rai-nn/src/linear.rs:59-69),
 * LayerNorm (layer_norm.rs:32-42), RmsNorm (rms_norm.rs:18-22), the rotary embedding and the attention block of
 * rai-models/src/llm/phi2.rs:66-77,244-262 -- are recognised by structure in the recorded graph and evaluated by
 * their fused launcher (rai_hip_linear / layer_norm / rms_norm / rope / attention).  Taken only when no interior
 * node is observable from outside.  Results agree with node-by-node evaluation within the dtype's tolerance (the
 * fused launchers round less often), not bit for bit. */
int rai_graph_set_compose(int32_t enabled);
typedef struct rai_graph_stats {
  uint64_t nodes_evaluated;   /* nodes that received data */
  uint64_t kernel_launches;   /* device launches issued by eval (views launch nothing) */
  uint64_t fused_regions;     /* multi-node elementwise regions evaluated by one launch */
  uint64_t fused_nodes;       /* nodes folded into those regions */
  uint64_t composed_regions;  /* compositions evaluated by one fused launcher */
  uint64_t composed_nodes;    /* nodes folded into those compositions */
  uint64_t plan_ns;           /* host time of rai_eval spent ordering the tape and planning the two passes */
  uint64_t run_ns;            /* host time of rai_eval spent in the rules (allocation, launches, detach) */
} rai_graph_stats;
int rai_graph_get_stats(rai_graph_stats *out, int32_t reset);

#ifdef __cplusplus
}
#endif
#endif /* RAI_GRAPH_H */
