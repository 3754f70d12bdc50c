// Lazy tensor graph, dispatcher and evaluator for the Hip device: the host-side
// machinery of rai-core that sits in front of the kernels.
//   rai-core/src/tensor.rs:28-37,229   Tensor = ref-counted node {device, dtype, shape, op, inputs, data}
//   rai-core/src/ops/*.rs               one builder per primitive; a bad shape yields an Err node
//   rai-core/src/utils.rs:35-66         iterative DFS topological sort that skips evaluated nodes
//   rai-core/src/dispatch.rs:159-212    (device, op) -> rule table with runtime registration
//   rai-core/src/eval.rs:31-51          eval(): per node look up the rule, run it, detach
// On top of that an elementwise-fusion pass: a chain of elementwise primitives
// (unary, arithmetic binary, float casts, constants) whose intermediate results
// nobody else can observe is evaluated by one launch of a small register-machine
// kernel (fused.h) that rounds exactly where node-by-node evaluation would.
#include <chrono>
#include <cmath>
#include <string>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include "attention.h"
#include "fused.h"
#include "gemm.h"
#include "rai_graph.h"

using namespace rai;

struct rai_tensor {
  int refs;
  uint64_t id;
  int dev, dtype;
  std::vector<int64_t> shape;
  int op, sub;                    // rai_op_kind and its sub-kind (unary / binary / reduce op)
  double p0, p1, p2;              // scalar parameters (fill value, arange start/step, powf exponent)
  std::vector<int64_t> ip;        // integer parameters (dims, target shape, narrow start/len, keep_dim)
  std::vector<rai_tensor *> inputs;
  std::string err;                // message of an Err node
  std::vector<uint8_t> host;      // FromArray payload
  bool evaluated;
  rai_hip_tensor view;            // storage once evaluated (may alias an input's buffer)
  void *buf;                      // retained allocation the view points into
  // A concatenation along `cap_dim` whose buffer was laid out for `cap` elements along that dim (strided view):
  // the next concatenation that appends to this node writes its new part into the slack instead of copying both
  // (once: `extended` says somebody already did).
  int cap_dim;
  int64_t cap;
  bool extended;
  // Scratch of the evaluation in progress, valid while mark == the evaluation's epoch: position in the tape, the
  // edges from tape nodes that use this node (a run of the evaluation's flat user list), planning flags, the
  // composition this node is the root of, and a stamp the matchers use to tell a composition's nodes apart.
  uint64_t mark;
  int tape_idx;
  int n_users, users_at;
  uint32_t flags;
  int comp;
  int group;   // index of the Linear group this node leads (flag kGroupLead)
  uint64_t stamp;
};

namespace {

uint64_t g_next_id = 1;
uint64_t g_epoch = 0;        // one per rai_eval call
uint64_t g_stamp = 0;        // one per attempted composition
enum : uint32_t { kInlined = 1u, kAbsorbed = 2u, kRoot = 4u, kOutput = 8u, kCoOutput = 16u, kGroupLead = 32u, kGrouped = 64u };
inline bool in_tape(const rai_tensor *t) { return t->mark == g_epoch; }
inline bool has_flag(const rai_tensor *t, uint32_t f) { return in_tape(t) && (t->flags & f); }
std::vector<const rai_tensor *> g_users;   // flat user lists of the evaluation in progress
bool g_fusion = true;
bool g_group_linears = true;   // RAI_HIP_GRAPH_NO_LINEAR_GROUPS=1 (read per evaluation) turns the grouping of Linears off
bool g_compose = true;
rai_graph_stats g_stats = {0, 0, 0, 0, 0, 0, 0, 0};

int64_t numel_of(const std::vector<int64_t> &s) {
  int64_t n = 1;
  for (int64_t d : s) n *= d;
  return n;
}

rai_tensor *new_node(int dev, int dtype, const std::vector<int64_t> &shape, int op, std::vector<rai_tensor *> inputs) {
  rai_tensor *t = new rai_tensor();
  t->refs = 1;
  t->id = g_next_id++;
  t->dev = dev;
  t->dtype = dtype;
  t->shape = shape;
  t->op = op;
  t->sub = 0;
  t->p0 = t->p1 = t->p2 = 0.0;
  t->inputs = std::move(inputs);
  for (rai_tensor *i : t->inputs) ++i->refs;
  t->evaluated = false;
  memset(&t->view, 0, sizeof(t->view));
  t->buf = nullptr;
  t->cap_dim = -1;
  t->cap = 0;
  t->extended = false;
  t->mark = 0;
  t->tape_idx = -1;
  t->n_users = t->users_at = 0;
  t->flags = 0;
  t->comp = -1;
  t->group = -1;
  t->stamp = 0;
  return t;
}

// Err node (rai-core/src/ops/err.rs): keeps the op it replaces and its inputs; eval reports it.
rai_tensor *err_node(int dev, int dtype, const std::vector<int64_t> &shape, std::vector<rai_tensor *> inputs,
                     const std::string &msg) {
  rai_tensor *t = new_node(dev, dtype, shape, RAI_OP_ERR, std::move(inputs));
  t->err = msg;
  return t;
}

std::string shape_str(const std::vector<int64_t> &s) {
  std::string r = "[";
  for (size_t i = 0; i < s.size(); ++i) r += (i ? ", " : "") + std::to_string(s[i]);
  return r + "]";
}
std::string incompatible(const rai_tensor *a, const rai_tensor *b) {
  return "IncompatibleShape { lhs: " + shape_str(a->shape) + ", rhs: " + shape_str(b->shape) + " }";
}

// numpy-style right-aligned broadcast (rai-core/src/shape.rs:88-127)
bool broadcast_shapes(const std::vector<int64_t> &l, const std::vector<int64_t> &r, std::vector<int64_t> *out, bool *lb,
                      bool *rb) {
  std::vector<int64_t> a = l, b = r;
  *lb = *rb = false;
  if (a.size() < b.size()) { a.insert(a.begin(), b.size() - a.size(), 1); *lb = true; }
  else if (b.size() < a.size()) { b.insert(b.begin(), a.size() - b.size(), 1); *rb = true; }
  out->clear();
  for (size_t i = 0; i < a.size(); ++i) {
    if (a[i] == b[i]) out->push_back(a[i]);
    else if (a[i] == 1) { out->push_back(b[i]); *lb = true; }
    else if (b[i] == 1) { out->push_back(a[i]); *rb = true; }
    else return false;
  }
  return true;
}

int norm_dim(int d, int rank) { return d < 0 ? d + rank : d; }

// ------------------------------------------------------------------ storage helpers
void drop_storage(rai_tensor *t) {
  if (t->buf) (void)rai_hip_release(t->buf);
  t->buf = nullptr;
  t->evaluated = false;
  t->cap_dim = -1;
}

void contiguous_view(rai_tensor *t, void *data) {
  rai_hip_tensor &v = t->view;
  memset(&v, 0, sizeof(v));
  v.data = data;
  v.dtype = t->dtype;
  v.rank = (int32_t)t->shape.size();
  int64_t st = 1;
  for (int i = v.rank - 1; i >= 0; --i) {
    v.shape[i] = t->shape[i];
    v.stride[i] = st;
    st *= t->shape[i];
  }
  v.offset = 0;
}

// Fresh contiguous output for a node (functional semantics: outputs never alias inputs).
int alloc_output(rai_tensor *t) {
  void *p = nullptr;
  const size_t bytes = (size_t)numel_of(t->shape) * dtype_size(t->dtype);
  RAI_TRY(rai_hip_alloc(t->dev, bytes ? bytes : 1, &p));
  t->buf = p;
  contiguous_view(t, p);
  return RAI_OK;
}

// The node's data becomes a view of `src`'s buffer.
void alias_storage(rai_tensor *t, const rai_tensor *src, const rai_hip_tensor &v) {
  t->view = v;
  t->buf = src->buf;
  if (t->buf) (void)rai_hip_retain(t->buf);
}

// ------------------------------------------------------------------ evaluation rules (one per primitive)
typedef int (*rule_fn)(rai_tensor *);

int ev_full(rai_tensor *t) {
  RAI_TRY(alloc_output(t));
  ++g_stats.kernel_launches;
  return rai_hip_fill(t->dev, &t->view, t->p0);
}
int ev_arange(rai_tensor *t) {
  RAI_TRY(alloc_output(t));
  ++g_stats.kernel_launches;
  return rai_hip_arange(t->dev, &t->view, t->p0, t->p2);
}
int ev_from_array(rai_tensor *t) {
  RAI_TRY(alloc_output(t));
  return rai_hip_h2d(t->dev, t->view.data, t->host.data(), t->host.size());
}
int ev_to_dtype(rai_tensor *t) {
  RAI_TRY(alloc_output(t));
  ++g_stats.kernel_launches;
  return rai_hip_cast(t->dev, &t->inputs[0]->view, &t->view);
}
int ev_unary(rai_tensor *t) {
  RAI_TRY(alloc_output(t));
  ++g_stats.kernel_launches;
  return rai_hip_unary(t->dev, t->sub, &t->inputs[0]->view, &t->view, t->p0);
}
int ev_binary(rai_tensor *t) {
  RAI_TRY(alloc_output(t));
  ++g_stats.kernel_launches;
  return rai_hip_binary(t->dev, t->sub, &t->inputs[0]->view, &t->inputs[1]->view, &t->view);
}
int ev_matmul(rai_tensor *t) {
  RAI_TRY(alloc_output(t));
  ++g_stats.kernel_launches;
  return rai_hip_matmul(t->dev, &t->inputs[0]->view, &t->inputs[1]->view, &t->view);
}
int ev_softmax(rai_tensor *t) {
  RAI_TRY(alloc_output(t));
  ++g_stats.kernel_launches;
  return rai_hip_softmax(t->dev, &t->inputs[0]->view, (int32_t)t->ip[0], &t->view);
}
int ev_log_softmax(rai_tensor *t) {
  RAI_TRY(alloc_output(t));
  ++g_stats.kernel_launches;
  return rai_hip_log_softmax(t->dev, &t->inputs[0]->view, (int32_t)t->ip[0], &t->view);
}
int ev_reduce(rai_tensor *t) {
  RAI_TRY(alloc_output(t));
  ++g_stats.kernel_launches;
  std::vector<int32_t> dims(t->ip.begin() + 1, t->ip.end());
  return rai_hip_reduce(t->dev, t->sub, &t->inputs[0]->view, dims.data(), (int32_t)dims.size(), (int32_t)t->ip[0], &t->view);
}
int ev_argmax(rai_tensor *t) {
  RAI_TRY(alloc_output(t));
  ++g_stats.kernel_launches;
  return rai_hip_argmax(t->dev, &t->inputs[0]->view, (int32_t)t->ip[0], (int32_t)t->ip[1], &t->view);
}
int ev_argmin(rai_tensor *t) {
  RAI_TRY(alloc_output(t));
  ++g_stats.kernel_launches;
  return rai_hip_argmin(t->dev, &t->inputs[0]->view, (int32_t)t->ip[0], (int32_t)t->ip[1], &t->view);
}
int ev_index_select(rai_tensor *t) {
  RAI_TRY(alloc_output(t));
  ++g_stats.kernel_launches;
  return rai_hip_index_select(t->dev, &t->inputs[0]->view, &t->inputs[1]->view, (int32_t)t->ip[0], &t->view);
}
// A contiguous stand-in for an input view (the reference does the same with `.contiguous()`,
// candle.rs:845,998-999); `tmp` owns the copy, if one was needed, until the rule returns.
struct TempContiguous {
  void *buf = nullptr;
  rai_hip_tensor view;
  int make(int dev, const rai_hip_tensor &src) {
    view = src;
    if (is_contiguous(&src)) return RAI_OK;
    int64_t n = 1;
    for (int i = 0; i < src.rank; ++i) n *= src.shape[i];
    const size_t bytes = (size_t)n * dtype_size(src.dtype);
    RAI_TRY(rai_hip_alloc(dev, bytes ? bytes : 1, &buf));
    view.data = buf;
    view.offset = 0;
    int64_t st = 1;
    for (int i = src.rank - 1; i >= 0; --i) { view.stride[i] = st; st *= src.shape[i]; }
    ++g_stats.kernel_launches;
    return rai_hip_copy(dev, &src, &view);
  }
  ~TempContiguous() { if (buf) (void)rai_hip_release(buf); }
};
int ev_gather(rai_tensor *t) {
  RAI_TRY(alloc_output(t));
  TempContiguous x, ix;
  RAI_TRY(x.make(t->dev, t->inputs[0]->view));
  RAI_TRY(ix.make(t->dev, t->inputs[1]->view));
  ++g_stats.kernel_launches;
  return rai_hip_gather(t->dev, &x.view, &ix.view, (int32_t)t->ip[0], &t->view);
}
int ev_index_add(rai_tensor *t) {  // inputs are ordered [x, source, index]
  RAI_TRY(alloc_output(t));
  TempContiguous x, src;
  RAI_TRY(x.make(t->dev, t->inputs[0]->view));
  RAI_TRY(src.make(t->dev, t->inputs[1]->view));
  ++g_stats.kernel_launches;
  return rai_hip_index_add(t->dev, &x.view, &t->inputs[2]->view, &src.view, (int32_t)t->ip[0], &t->view);
}
int ev_scatter_add(rai_tensor *t) {  // inputs are ordered [x, source, index]
  RAI_TRY(alloc_output(t));
  TempContiguous x, src, ix;
  RAI_TRY(x.make(t->dev, t->inputs[0]->view));
  RAI_TRY(src.make(t->dev, t->inputs[1]->view));
  RAI_TRY(ix.make(t->dev, t->inputs[2]->view));
  ++g_stats.kernel_launches;
  return rai_hip_scatter_add(t->dev, &x.view, &ix.view, &src.view, (int32_t)t->ip[0], &t->view);
}
int ev_where(rai_tensor *t) {  // inputs are ordered [on_true, on_false, cond] (ops/where.rs:37-45)
  RAI_TRY(alloc_output(t));
  ++g_stats.kernel_launches;
  return rai_hip_where(t->dev, &t->inputs[2]->view, &t->inputs[0]->view, &t->inputs[1]->view, &t->view);
}
int ev_to_contiguous(rai_tensor *t) {
  RAI_TRY(alloc_output(t));
  ++g_stats.kernel_launches;
  return rai_hip_copy(t->dev, &t->inputs[0]->view, &t->view);
}
int ev_to_device(rai_tensor *t) {  // ops/to_device.rs: the node lives on the target device, its input on the source
  RAI_TRY(alloc_output(t));
  ++g_stats.kernel_launches;
  return rai_hip_to_device(t->inputs[0]->dev, &t->inputs[0]->view, t->dev, &t->view);
}
// A key / value cache grows by concatenation along the sequence dim every step (phi2.rs:233-243): cat([cache, new], 2).
// Copying the whole cache each time is O(T) per step and layer.  Instead such a concatenation (two inputs, the dim
// before the last, the second input the shorter one) gets a buffer with room to grow along that dim, laid out with
// the capacity as the stride, and the next concatenation that appends to its result writes only the new part into
// the slack and shares the buffer.  The earlier tensor keeps its shape and its contents (its view never covered the
// slack), so nothing observable changes; a second concatenation onto the same tensor copies as usual.
int64_t grown_capacity(int64_t len) { return (len + len / 4 + 64 + 63) / 64 * 64; }

int append_in_place(rai_tensor *t, int dim) {
  rai_tensor *base = t->inputs[0], *add = t->inputs[1];
  rai_hip_tensor v = base->view;
  v.shape[dim] = t->shape[dim];
  rai_hip_tensor dst = v;              // the slice the new part fills
  dst.shape[dim] = add->shape[dim];
  dst.offset += base->shape[dim] * dst.stride[dim];
  ++g_stats.kernel_launches;
  RAI_TRY(rai_hip_copy(t->dev, &add->view, &dst));
  alias_storage(t, base, v);
  t->cap_dim = dim;
  t->cap = base->cap;
  base->extended = true;
  return RAI_OK;
}

int ev_concatenate(rai_tensor *t) {
  const int dim = (int)t->ip[0];
  const int rank = (int)t->shape.size();
  const bool cache_like = t->inputs.size() == 2 && rank >= 3 && dim == rank - 2 && numel_of(t->inputs[1]->shape) > 0 &&
                          t->inputs[1]->shape[dim] <= t->inputs[0]->shape[dim];
  if (cache_like) {
    rai_tensor *base = t->inputs[0];
    if (base->cap_dim == dim && !base->extended && t->shape[dim] <= base->cap && base->buf) return append_in_place(t, dim);
    // first growth: a buffer with slack along `dim`, viewed through strides that skip it
    const int64_t cap = grown_capacity(t->shape[dim]);
    std::vector<int64_t> padded = t->shape;
    padded[dim] = cap;
    void *p = nullptr;
    RAI_TRY(rai_hip_alloc(t->dev, (size_t)numel_of(padded) * dtype_size(t->dtype), &p));
    t->buf = p;
    rai_hip_tensor &v = t->view;
    memset(&v, 0, sizeof(v));
    v.data = p;
    v.dtype = t->dtype;
    v.rank = rank;
    int64_t st = 1;
    for (int i = rank - 1; i >= 0; --i) {
      v.shape[i] = t->shape[i];
      v.stride[i] = st;
      st *= padded[i];
    }
    t->cap_dim = dim;
    t->cap = cap;
  } else {
    RAI_TRY(alloc_output(t));
  }
  int64_t at = 0;
  for (rai_tensor *in : t->inputs) {
    rai_hip_tensor dst = t->view;  // the slice of the output this input fills
    dst.shape[dim] = in->shape[dim];
    dst.offset += at * dst.stride[dim];
    at += in->shape[dim];
    if (numel_of(in->shape) == 0) continue;
    ++g_stats.kernel_launches;
    RAI_TRY(rai_hip_copy(t->dev, &in->view, &dst));
  }
  return RAI_OK;
}
// ---- views: no launch, the node shares the input's buffer
int ev_transpose(rai_tensor *t) {
  rai_hip_tensor v = t->inputs[0]->view;
  const int a = (int)t->ip[0], b = (int)t->ip[1];
  std::swap(v.shape[a], v.shape[b]);
  std::swap(v.stride[a], v.stride[b]);
  alias_storage(t, t->inputs[0], v);
  return RAI_OK;
}
int ev_permute(rai_tensor *t) {
  const rai_hip_tensor &s = t->inputs[0]->view;
  rai_hip_tensor v = s;
  for (int i = 0; i < v.rank; ++i) {
    v.shape[i] = s.shape[t->ip[i]];
    v.stride[i] = s.stride[t->ip[i]];
  }
  alias_storage(t, t->inputs[0], v);
  return RAI_OK;
}
int ev_narrow(rai_tensor *t) {
  rai_hip_tensor v = t->inputs[0]->view;
  const int dim = (int)t->ip[0];
  v.offset += t->ip[1] * v.stride[dim];
  v.shape[dim] = t->ip[2];
  alias_storage(t, t->inputs[0], v);
  return RAI_OK;
}
int ev_broadcast(rai_tensor *t) {
  const rai_hip_tensor &s = t->inputs[0]->view;
  rai_hip_tensor v = s;
  v.rank = (int32_t)t->shape.size();
  const int lead = v.rank - s.rank;
  for (int i = 0; i < v.rank; ++i) {
    v.shape[i] = t->shape[i];
    if (i < lead) v.stride[i] = 0;
    else v.stride[i] = s.shape[i - lead] == t->shape[i] ? s.stride[i - lead] : 0;
  }
  alias_storage(t, t->inputs[0], v);
  return RAI_OK;
}
int ev_reshape(rai_tensor *t) {
  rai_tensor *in = t->inputs[0];
  if (is_contiguous(&in->view)) {
    rai_hip_tensor v;
    memset(&v, 0, sizeof(v));
    v.data = in->view.data;
    v.dtype = in->view.dtype;
    v.offset = in->view.offset;
    v.rank = (int32_t)t->shape.size();
    int64_t st = 1;
    for (int i = v.rank - 1; i >= 0; --i) {
      v.shape[i] = t->shape[i];
      v.stride[i] = st;
      st *= t->shape[i];
    }
    alias_storage(t, in, v);
    return RAI_OK;
  }
  // inserting or dropping dims of size 1 (unsqueeze, squeeze) is a view of any layout
  {
    std::vector<int64_t> keep_shape, keep_stride;
    for (int i = 0; i < in->view.rank; ++i)
      if (in->view.shape[i] != 1) { keep_shape.push_back(in->view.shape[i]); keep_stride.push_back(in->view.stride[i]); }
    std::vector<int64_t> want;
    for (int64_t d : t->shape)
      if (d != 1) want.push_back(d);
    if (want == keep_shape && t->shape.size() <= RAI_HIP_MAX_RANK) {
      rai_hip_tensor v = in->view;
      v.rank = (int32_t)t->shape.size();
      size_t k = 0;
      for (int i = 0; i < v.rank; ++i) {
        v.shape[i] = t->shape[i];
        v.stride[i] = t->shape[i] == 1 ? 1 : keep_stride[k++];
      }
      alias_storage(t, in, v);
      return RAI_OK;
    }
  }
  // any other reshape of a non-contiguous view has to materialise it first
  RAI_TRY(alloc_output(t));
  rai_hip_tensor as_in = t->view;
  as_in.rank = in->view.rank;
  int64_t st = 1;
  for (int i = as_in.rank - 1; i >= 0; --i) {
    as_in.shape[i] = in->view.shape[i];
    as_in.stride[i] = st;
    st *= in->view.shape[i];
  }
  ++g_stats.kernel_launches;
  return rai_hip_copy(t->dev, &in->view, &as_in);
}

const rule_fn kBuiltin[RAI_OP_COUNT_] = {
    ev_full, ev_arange, ev_from_array, ev_to_dtype, ev_unary, ev_binary, ev_matmul, ev_softmax, ev_log_softmax, ev_reduce,
    ev_argmax, ev_argmin, ev_index_select, ev_narrow, ev_concatenate, ev_where, ev_transpose, ev_reshape, ev_permute,
    ev_broadcast, ev_to_contiguous, nullptr /* Err nodes never reach a rule */, ev_gather, ev_index_add, ev_scatter_add,
    ev_to_device};
rule_fn g_rules[RAI_OP_COUNT_];
bool g_rules_init = false;
void init_rules() {
  if (g_rules_init) return;
  for (int i = 0; i < RAI_OP_COUNT_; ++i) g_rules[i] = kBuiltin[i];
  g_rules_init = true;
}

const char *op_name(int op) {
  static const char *n[RAI_OP_COUNT_] = {"Full", "Arange", "FromArray", "ToDType", "Unary", "Binary", "MatMul", "Softmax",
                                         "LogSoftmax", "Reduce", "ArgMax", "ArgMin", "IndexSelect", "Narrow",
                                         "Concatenate", "Where", "Transpose", "Reshape", "Permute", "Broadcast",
                                         "ToContiguous", "Err", "Gather", "IndexAdd", "ScatterAdd", "ToDevice"};
  return op >= 0 && op < RAI_OP_COUNT_ ? n[op] : "?";
}

// ------------------------------------------------------------------ topological order (utils.rs:35-66)
int topo_sort(rai_tensor *const *outputs, int n, std::vector<rai_tensor *> *tape) {
  ++g_epoch;   // a node is in this tape exactly when its mark carries this epoch
  std::vector<std::pair<rai_tensor *, bool>> stack;
  for (int o = 0; o < n; ++o) {
    stack.push_back({outputs[o], outputs[o]->inputs.empty()});
    while (!stack.empty()) {
      auto [t, inputs_done] = stack.back();
      stack.pop_back();
      if (in_tape(t) || t->evaluated) continue;
      if (t->op == RAI_OP_ERR) return fail(RAI_ERR_BAD_SHAPE, "eval: %s", t->err.c_str());
      if (inputs_done) {
        t->mark = g_epoch;
        t->tape_idx = (int)tape->size();
        t->n_users = t->users_at = 0;
        t->flags = 0;
        t->comp = -1;
        t->group = -1;
        tape->push_back(t);
      } else {
        stack.push_back({t, true});
        for (rai_tensor *in : t->inputs) stack.push_back({in, in->inputs.empty()});
      }
    }
  }
  return RAI_OK;
}

// ------------------------------------------------------------------ fusion pass
bool fusable_dtype(int dt) { return dt == RAI_F32 || dt == RAI_BF16 || dt == RAI_F16; }
bool elementwise(const rai_tensor *t) {
  if (!fusable_dtype(t->dtype)) return false;
  switch (t->op) {
    case RAI_OP_UNARY: return fusable_dtype(t->inputs[0]->dtype);
    case RAI_OP_BINARY:
      return t->sub <= RAI_BIN_MINIMUM && fusable_dtype(t->inputs[0]->dtype) && t->inputs[1]->dtype == t->inputs[0]->dtype;
    case RAI_OP_TO_DTYPE: return fusable_dtype(t->inputs[0]->dtype);
    case RAI_OP_FULL: return true;
    default: return false;
  }
}

// Edges of the tape: how many tape nodes use each tape node and which (rai_tensor::n_users / users_at into g_users).
void index_users(const std::vector<rai_tensor *> &tape) {
  size_t edges = 0;
  for (const rai_tensor *t : tape)
    for (rai_tensor *in : t->inputs)
      if (in_tape(in)) { ++in->n_users; ++edges; }
  int at = 0;
  for (rai_tensor *t : tape) { t->users_at = at; at += t->n_users; t->n_users = 0; }
  g_users.assign(edges, nullptr);
  for (const rai_tensor *t : tape)
    for (rai_tensor *in : t->inputs)
      if (in_tape(in)) g_users[in->users_at + in->n_users++] = t;
}

// A node is folded into its consumer when it is elementwise, exactly one edge of
// the tape uses it, that user is elementwise too, it is not a requested output,
// and no handle outside the tape refers to it (refs == that one edge).
void plan_fusion(const std::vector<rai_tensor *> &tape) {
  for (rai_tensor *t : tape) {
    if (!elementwise(t) || (t->flags & (kOutput | kAbsorbed | kRoot)) || !g_rules[t->op]) continue;  // fusion never hides a missing rule
    if (t->n_users != 1 || t->refs != 1) continue;
    const rai_tensor *c = g_users[t->users_at];
    if (!elementwise(c) || (c->flags & (kAbsorbed | kRoot)) || c->shape != t->shape) continue;
    t->flags |= kInlined;
  }
}

// Emits the instructions of `t` (post-order) into the program; returns its register or -1 when the region is too large.
int emit(const rai_tensor *t, bool root, FusedProgram *p, std::unordered_map<uint64_t, int> *leaf_reg,
         std::vector<const rai_tensor *> *members) {
  auto push = [&](FusedInstr in) -> int {
    if (p->n_instr >= kFusedMaxInstr) return -1;
    p->instr[p->n_instr] = in;
    return p->n_instr++;
  };
  if (!root && !has_flag(t, kInlined)) {  // a materialised input: leaf
    auto it = leaf_reg->find(t->id);
    if (it != leaf_reg->end()) return it->second;
    if (p->n_leaves >= kFusedMaxLeaves) return -1;
    const int l = p->n_leaves++;
    p->leaf[l] = base_ptr(&t->view);
    p->leaf_dtype[l] = t->dtype;
    for (int d = 0; d < p->rank; ++d) p->lstride[l][d] = t->view.shape[d] == 1 ? 0 : t->view.stride[d];
    FusedInstr in = {};
    in.kind = FUSED_LEAF;
    in.a = (uint8_t)l;
    in.dtype = (uint8_t)t->dtype;
    const int r = push(in);
    if (r >= 0) (*leaf_reg)[t->id] = r;
    return r;
  }
  if (!root) members->push_back(t);
  FusedInstr in = {};
  in.dtype = (uint8_t)t->dtype;
  switch (t->op) {
    case RAI_OP_FULL: {
      in.kind = FUSED_CONST;
      float v = (float)t->p0;  // rounded to the node's dtype like the fill kernel does
      if (t->dtype == RAI_BF16) {
        uint32_t u;
        memcpy(&u, &v, 4);
        if ((u & 0x7fffffffu) <= 0x7f800000u) { u += 0x7fffu + ((u >> 16) & 1u); u &= 0xffff0000u; }
        memcpy(&v, &u, 4);
      } else if (t->dtype == RAI_F16) {
        v = (float)(_Float16)v;
      }
      in.param = v;
      return push(in);
    }
    case RAI_OP_UNARY: {
      const int a = emit(t->inputs[0], false, p, leaf_reg, members);
      if (a < 0) return -1;
      in.kind = FUSED_UNARY;
      in.op = (uint8_t)t->sub;
      in.a = (uint8_t)a;
      in.param = (float)t->p0;
      return push(in);
    }
    case RAI_OP_BINARY: {
      const int a = emit(t->inputs[0], false, p, leaf_reg, members);
      if (a < 0) return -1;
      const int b = emit(t->inputs[1], false, p, leaf_reg, members);
      if (b < 0) return -1;
      in.kind = FUSED_BINARY;
      in.op = (uint8_t)t->sub;
      in.a = (uint8_t)a;
      in.b = (uint8_t)b;
      return push(in);
    }
    default: {  // RAI_OP_TO_DTYPE
      const int a = emit(t->inputs[0], false, p, leaf_reg, members);
      if (a < 0) return -1;
      in.kind = FUSED_CAST;
      in.a = (uint8_t)a;
      return push(in);
    }
  }
}

bool has_inlined_input(const rai_tensor *t) {
  for (const rai_tensor *in : t->inputs)
    if (has_flag(in, kInlined)) return true;
  return false;
}

// Evaluates the region rooted at t with one launch.  RAI_ERR_UNSUPPORTED means
// "too large for one program": the caller falls back to node-by-node evaluation.
int eval_region(rai_tensor *t) {
  FusedProgram p;
  memset(&p, 0, sizeof(p));
  p.rank = (int)t->shape.size();
  p.numel = numel_of(t->shape);
  for (int d = 0; d < p.rank; ++d) p.shape[d] = t->shape[d];
  std::unordered_map<uint64_t, int> leaf_reg;
  std::vector<const rai_tensor *> members;
  if (emit(t, true, &p, &leaf_reg, &members) < 0) return RAI_ERR_UNSUPPORTED;
  RAI_TRY(alloc_output(t));
  p.out = t->view.data;
  p.out_dtype = t->dtype;
  ++g_stats.kernel_launches;
  ++g_stats.fused_regions;
  g_stats.fused_nodes += members.size() + 1;
  return launch_fused_elementwise(t->dev, p);
}

// Node-by-node evaluation of an inlined sub-tree (used when a region did not fit).
int eval_plain(rai_tensor *t);
int eval_inputs_plain(rai_tensor *t) {
  for (rai_tensor *in : t->inputs)
    if (!in->evaluated && has_flag(in, kInlined)) RAI_TRY(eval_plain(in));
  return RAI_OK;
}
int eval_plain(rai_tensor *t) {
  RAI_TRY(eval_inputs_plain(t));
  rule_fn rule = g_rules[t->op];
  RAI_REQUIRE(rule, RAI_ERR_UNSUPPORTED, "Unimplemented { op: %s, device: Hip }", op_name(t->op));
  RAI_TRY(rule(t));
  t->evaluated = true;
  ++g_stats.nodes_evaluated;
  return RAI_OK;
}

// ------------------------------------------------------------------ composition pass
// rai's modules are compositions of primitives (rai-nn/src/{linear,layer_norm,rms_norm}.rs, the rotary embedding and
// the attention block of rai-models/src/llm/phi2.rs); recorded node by node they are 10-20 launches each.  This pass
// recognises those compositions in the tape, by structure, and evaluates each with the one fused launcher that
// exists for it.  A composition is taken only when every interior node is invisible from outside it: unevaluated, not
// a requested output, no handle outside the tape, every consumer inside the composition.  The fused launchers keep
// f32 between the steps the reference rounds after, so a composed result agrees with the node-by-node one within
// the dtype's tolerance, not bit for bit (the elementwise pass above is the bit-exact one).
enum CompKind { COMP_LINEAR = 0, COMP_LAYER_NORM, COMP_RMS_NORM, COMP_ROPE, COMP_ATTENTION, COMP_DECODE_ATTN };
struct Composite {
  int kind;
  rai_tensor *in[7];   // operands: evaluated before the root is reached (they precede it in the tape); null: absent
  double f0;           // eps / scale
  int64_t i0, i1, i2;  // rotary dim and offset / causal flag and f32 scores / activation / (1 + w) norm
  // nodes that the root's launch materialises besides the root: they may be held from outside (the model keeps its
  // key / value caches), but every use inside the tape lies within the composition
  rai_tensor *co[2];
  // a Linear whose added tensor is itself "Linear + tensor" (root `dual_inner`, unobservable): at one row the two
  // products run as one launch and dual_inner is never materialised
  rai_tensor *dual_inner;
  std::vector<rai_tensor *> interior;
};

struct Matcher {
  std::vector<rai_tensor *> interior;
  bool ok = true;
  // descends into an unevaluated node of kind `op`; records it as interior
  rai_tensor *node(rai_tensor *t, int op) {
    if (!ok || !t || t->evaluated || t->op != op) { ok = false; return nullptr; }
    interior.push_back(t);
    return t;
  }
  bool bin(rai_tensor *t, int sub, rai_tensor **a, rai_tensor **b) {
    rai_tensor *n = node(t, RAI_OP_BINARY);
    if (!n || n->sub != sub) { ok = false; return false; }
    *a = n->inputs[0];
    *b = n->inputs[1];
    return true;
  }
  // which binary / unary primitive an unevaluated node is (-1: none); records nothing
  int bin_kind(const rai_tensor *t) const { return ok && t && !t->evaluated && t->op == RAI_OP_BINARY ? t->sub : -1; }
  int un_kind(const rai_tensor *t) const { return ok && t && !t->evaluated && t->op == RAI_OP_UNARY ? t->sub : -1; }
  // whether konst() would accept the node; records nothing
  bool is_konst(const rai_tensor *t) const {
    return t && (t->op == RAI_OP_FULL || (!t->evaluated && t->op == RAI_OP_TO_DTYPE && t->inputs[0]->op == RAI_OP_FULL));
  }
  // the operand behind any run of unevaluated Reshape nodes (unsqueeze is a reshape, hlops/unsqueeze.rs)
  rai_tensor *strip_reshapes(rai_tensor *t) {
    while (ok && t && !t->evaluated && t->op == RAI_OP_RESHAPE) { interior.push_back(t); t = t->inputs[0]; }
    return t;
  }
  rai_tensor *un(rai_tensor *t, int sub) {
    rai_tensor *n = node(t, RAI_OP_UNARY);
    if (!n || n->sub != sub) { ok = false; return nullptr; }
    return n->inputs[0];
  }
  // the operand behind an optional Broadcast view
  rai_tensor *strip_bc(rai_tensor *t) {
    if (ok && t && !t->evaluated && t->op == RAI_OP_BROADCAST) { interior.push_back(t); return t->inputs[0]; }
    return t;
  }
  // the operand behind an optional cast to `dtype` (ToDType of an equal dtype never makes a node)
  rai_tensor *strip_cast(rai_tensor *t, int dtype) {
    if (ok && t && !t->evaluated && t->op == RAI_OP_TO_DTYPE && t->dtype == dtype) { interior.push_back(t); return t->inputs[0]; }
    return t;
  }
  // a scalar constant: Full, or Full cast to the tensor's dtype (ops/full.rs:85-92)
  bool konst(rai_tensor *t, double *v) {
    if (!ok || !t) return ok = false;
    if (t->op == RAI_OP_FULL) { if (!t->evaluated) interior.push_back(t); *v = t->p0; return true; }
    if (!t->evaluated && t->op == RAI_OP_TO_DTYPE && t->inputs[0]->op == RAI_OP_FULL) {
      interior.push_back(t);
      if (!t->inputs[0]->evaluated) interior.push_back(t->inputs[0]);
      *v = t->inputs[0]->p0;
      return true;
    }
    return ok = false;
  }
  // sum over the last dim, keep_dim
  rai_tensor *sum_last_keep(rai_tensor *t) {
    rai_tensor *n = node(t, RAI_OP_REDUCE);
    if (!n) return nullptr;
    const int rank = (int)n->inputs[0]->shape.size();
    if (n->sub != RAI_RED_SUM || n->ip.size() != 2 || n->ip[0] != 1 || n->ip[1] != rank - 1) { ok = false; return nullptr; }
    return n->inputs[0];
  }
  rai_tensor *narrow(rai_tensor *t, int64_t dim, int64_t *start, int64_t *len) {
    rai_tensor *n = node(t, RAI_OP_NARROW);
    if (!n || n->ip[0] != dim) { ok = false; return nullptr; }
    *start = n->ip[1];
    *len = n->ip[2];
    return n->inputs[0];
  }
  // hlops/mean.rs:4-7 over the last dim, keep_dim: sum / n
  bool mean_of(rai_tensor *t, rai_tensor *x) {
    rai_tensor *s, *nc;
    double n = 0;
    if (!bin(t, RAI_BIN_DIV, &s, &nc) || !konst(nc, &n)) return false;
    if (sum_last_keep(s) != x || !ok || n != (double)x->shape.back()) return ok = false;
    return true;
  }
};

std::unordered_map<uint64_t, bool> g_causal_masks;   // mask node id -> "is the causal mask"; cleared per eval

bool vec_param(const rai_tensor *p, int64_t n, int dtype) { return p && p->shape.size() == 1 && p->shape[0] == n && p->dtype == dtype; }
bool norm_dtype(int dt) { return dt == RAI_F32 || dt == RAI_BF16 || dt == RAI_F16; }

// rai-nn/src/layer_norm.rs:32-42: w * ((x - mean) * rsqrt(var + eps)) + b, var = sum((x - mean)^2) / n (hlops/var.rs:33-38)
bool match_layer_norm(rai_tensor *t, Composite *c) {
  Matcher m;
  rai_tensor *y, *bb, *wb, *xs, *d, *rb, *x, *mb, *ve, *var, *epsc, *s, *nc, *x2, *mb2;
  if (!norm_dtype(t->dtype) || t->shape.empty() || !m.bin(t, RAI_BIN_ADD, &y, &bb)) return false;
  rai_tensor *bias = m.strip_bc(bb);
  if (!m.bin(y, RAI_BIN_MUL, &wb, &xs)) return false;
  rai_tensor *w = m.strip_bc(wb);
  const int64_t n = t->shape.back();
  if (!vec_param(w, n, t->dtype) || !vec_param(bias, n, t->dtype)) return false;
  if (!m.bin(xs, RAI_BIN_MUL, &d, &rb) || !m.bin(d, RAI_BIN_SUB, &x, &mb) || x->shape != t->shape) return false;
  if (!m.mean_of(m.strip_bc(mb), x)) return false;
  ve = m.un(m.strip_bc(rb), RAI_UN_RSQRT);
  double eps = 0, nn = 0;
  if (!ve || !m.bin(ve, RAI_BIN_ADD, &var, &epsc) || !m.konst(epsc, &eps)) return false;
  if (!m.bin(var, RAI_BIN_DIV, &s, &nc) || !m.konst(nc, &nn) || nn != (double)n) return false;
  rai_tensor *sq = m.sum_last_keep(s);
  rai_tensor *d2 = sq ? m.un(sq, RAI_UN_SQUARE) : nullptr;
  if (!d2 || !m.bin(d2, RAI_BIN_SUB, &x2, &mb2) || x2 != x || !m.mean_of(m.strip_bc(mb2), x) || !m.ok) return false;
  c->kind = COMP_LAYER_NORM;
  c->in[0] = x; c->in[1] = w; c->in[2] = bias;
  c->f0 = eps;
  c->interior = m.interior;
  return true;
}

// rai-nn/src/rms_norm.rs:18-22: w * x * rsqrt(sum((x / sqrt(n))^2) + eps)
bool match_rms_norm(rai_tensor *t, Composite *c) {
  Matcher m;
  rai_tensor *wx, *rb, *wb, *x, *ve, *s, *epsc, *x2, *cc;
  if (!norm_dtype(t->dtype) || t->shape.empty() || !m.bin(t, RAI_BIN_MUL, &wx, &rb) || !m.bin(wx, RAI_BIN_MUL, &wb, &x)) return false;
  rai_tensor *w = m.strip_bc(wb);
  const int64_t n = t->shape.back();
  if (!vec_param(w, n, t->dtype) || x->shape != t->shape) return false;
  ve = m.un(m.strip_bc(rb), RAI_UN_RSQRT);
  double eps = 0, div = 0;
  if (!ve || !m.bin(ve, RAI_BIN_ADD, &s, &epsc) || !m.konst(epsc, &eps)) return false;
  rai_tensor *sq = m.sum_last_keep(s);
  rai_tensor *xd = sq ? m.un(sq, RAI_UN_SQUARE) : nullptr;
  // the reference records (x * s).square() with s = 1 / sqrt(n) (rms_norm.rs:19-20); x / sqrt(n) is the same value
  // recorded as a division and is taken as well
  if (!xd) return false;
  if (m.bin_kind(xd) == RAI_BIN_MUL) {
    double mul = 0;
    if (!m.bin(xd, RAI_BIN_MUL, &x2, &cc) || x2 != x || !m.konst(cc, &mul) || !m.ok) return false;
    if (fabs(mul * mul * (double)n - 1.0) > 1e-3) return false;
  } else {
    if (!m.bin(xd, RAI_BIN_DIV, &x2, &cc) || x2 != x || !m.konst(cc, &div) || !m.ok) return false;
    if (fabs(div * div - (double)n) > 1e-3 * (double)n) return false;
  }
  c->kind = COMP_RMS_NORM;
  c->in[0] = x; c->in[1] = w;
  c->f0 = eps;
  c->interior = m.interior;
  return true;
}

// RmsNorm::fwd of rai-models/src/llm/gemma.rs:42-54: f32 inside for 16-bit inputs,
// (x / sqrt(sum(x^2) / n + eps)).to_dtype(dt) * (w + 1)
bool match_gemma_rms_norm(rai_tensor *t, Composite *c) {
  Matcher m;
  rai_tensor *xn, *wb, *num, *den, *w, *one_c, *ms, *epsc, *sq, *nc;
  if (!norm_dtype(t->dtype) || t->shape.empty() || m.bin_kind(t) != RAI_BIN_MUL || !m.bin(t, RAI_BIN_MUL, &xn, &wb)) return false;
  rai_tensor *wp = m.strip_bc(wb);
  double one = 0, eps = 0, nn = 0;
  if (m.bin_kind(wp) != RAI_BIN_ADD || !m.bin(wp, RAI_BIN_ADD, &w, &one_c) || !m.konst(one_c, &one) || one != 1.0) return false;
  const int64_t n = t->shape.back();
  if (!vec_param(w, n, t->dtype)) return false;
  xn = m.strip_cast(xn, t->dtype);
  if (m.bin_kind(xn) != RAI_BIN_DIV || !m.bin(xn, RAI_BIN_DIV, &num, &den)) return false;
  rai_tensor *root = m.un(m.strip_bc(den), RAI_UN_SQRT);
  if (!root || !m.bin(root, RAI_BIN_ADD, &ms, &epsc) || !m.konst(epsc, &eps)) return false;
  if (!m.bin(ms, RAI_BIN_DIV, &sq, &nc) || !m.konst(nc, &nn) || nn != (double)n) return false;
  rai_tensor *sx = m.sum_last_keep(sq);
  rai_tensor *xi = sx ? m.un(sx, RAI_UN_SQUARE) : nullptr;
  if (!xi || xi != num || !m.ok) return false;
  rai_tensor *x = m.strip_cast(xi, RAI_F32);
  if (x->dtype != t->dtype || x->shape != t->shape) return false;
  c->kind = COMP_RMS_NORM;
  c->in[0] = x; c->in[1] = w;
  c->f0 = eps;
  c->i2 = 1;
  c->interior = m.interior;
  return true;
}

// rai-nn/src/linear.rs:59-69: x @ broadcast_left(W).t() [+ b]; fills x, w, bias (null without one)
bool linear_core(Matcher &m, rai_tensor *t, rai_tensor **x, rai_tensor **w, rai_tensor **bias) {
  if ((t->dtype != RAI_BF16 && t->dtype != RAI_F32) || t->shape.size() < 2) return m.ok = false;
  rai_tensor *mm = t;
  *bias = nullptr;
  if (m.bin_kind(t) == RAI_BIN_ADD) {
    rai_tensor *bb;
    if (!m.bin(t, RAI_BIN_ADD, &mm, &bb)) return false;
    *bias = m.strip_bc(bb);
    if (!vec_param(*bias, t->shape.back(), t->dtype)) return m.ok = false;
  }
  rai_tensor *mn = m.node(mm, RAI_OP_MATMUL);
  if (!mn) return false;
  *x = mn->inputs[0];
  rai_tensor *wt = m.node(mn->inputs[1], RAI_OP_TRANSPOSE);
  if (!wt) return false;
  const int r = (int)wt->shape.size();
  if (!((wt->ip[0] == r - 2 && wt->ip[1] == r - 1) || (wt->ip[0] == r - 1 && wt->ip[1] == r - 2))) return m.ok = false;
  *w = m.strip_bc(wt->inputs[0]);
  if (!m.ok || (*w)->shape.size() != 2 || (*w)->dtype != t->dtype || (*x)->dtype != t->dtype ||
      (*x)->shape.size() != t->shape.size())
    return m.ok = false;
  if ((*w)->shape[0] != t->shape.back() || (*w)->shape[1] != (*x)->shape.back()) return m.ok = false;
  return true;
}

// The activations of rai-core/src/hlops/activations.rs:5-32 by structure: fills the argument and the RAI_UN_* code
bool activation_of(Matcher &m, rai_tensor *t, rai_tensor **x, int *act) {
  const int kind = m.bin_kind(t);
  rai_tensor *a, *b;
  double c = 0;
  if (kind == RAI_BIN_DIV) {   // silu: x / (exp(-x) + 1)
    rai_tensor *e, *one;
    if (!m.bin(t, RAI_BIN_DIV, &a, &b) || !m.bin(b, RAI_BIN_ADD, &e, &one) || !m.konst(one, &c) || c != 1.0) return m.ok = false;
    rai_tensor *ng = m.un(e, RAI_UN_EXP);
    if (!ng || m.un(ng, RAI_UN_NEG) != a || !m.ok) return m.ok = false;
    *x = a; *act = RAI_UN_SILU;
    return true;
  }
  if (kind == RAI_BIN_MAXIMUM) {   // relu: max(x, zeros_like(x))
    if (!m.bin(t, RAI_BIN_MAXIMUM, &a, &b) || !m.konst(b, &c) || c != 0.0) return m.ok = false;
    *x = a; *act = RAI_UN_RELU;
    return true;
  }
  if (kind != RAI_BIN_MUL) return m.ok = false;
  rai_tensor *l, *r, *one, *inner, *p, *q;
  if (!m.bin(t, RAI_BIN_MUL, &l, &r) || !m.bin(l, RAI_BIN_MUL, &p, &q)) return false;
  const bool half_first = m.is_konst(p);    // new_gelu: 0.5 * x; gelu: x * 0.5
  if (!m.konst(half_first ? p : q, &c) || c != 0.5) return m.ok = false;
  rai_tensor *arg = half_first ? q : p;
  if (!m.bin(r, RAI_BIN_ADD, &one, &inner) || !m.konst(one, &c) || c != 1.0) return m.ok = false;
  if (m.un_kind(inner) == RAI_UN_TANH && half_first) {   // 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3)))
    rai_tensor *u = m.un(inner, RAI_UN_TANH), *kc, *sum, *x1, *cub, *c4, *pw;
    if (!u || !m.bin(u, RAI_BIN_MUL, &kc, &sum) || !m.konst(kc, &c) || fabs(c - 0.7978845608028654) > 1e-6) return m.ok = false;
    if (!m.bin(sum, RAI_BIN_ADD, &x1, &cub) || x1 != arg || !m.bin(cub, RAI_BIN_MUL, &c4, &pw) || !m.konst(c4, &c) ||
        fabs(c - 0.044715) > 1e-7)
      return m.ok = false;
    rai_tensor *pn = m.node(pw, RAI_OP_UNARY);
    if (!pn || pn->sub != RAI_UN_POWF || pn->p0 != 3.0 || pn->inputs[0] != arg) return m.ok = false;
    *x = arg; *act = RAI_UN_NEW_GELU;
    return true;
  }
  if (m.un_kind(inner) == RAI_UN_ERF && !half_first) {   // x 0.5 (1 + erf(x / sqrt 2))
    rai_tensor *u = m.un(inner, RAI_UN_ERF), *x1, *cs;
    if (!u || !m.bin(u, RAI_BIN_DIV, &x1, &cs) || x1 != arg || !m.konst(cs, &c) || fabs(c - 1.4142135623730951) > 1e-6)
      return m.ok = false;
    *x = arg; *act = RAI_UN_GELU;
    return true;
  }
  return m.ok = false;
}

// [activation of] a Linear, with or without bias
bool act_linear(Matcher &m, rai_tensor *t, rai_tensor **x, rai_tensor **w, rai_tensor **bias, int *act) {
  *act = -1;
  {
    Matcher tr = m;
    rai_tensor *arg;
    int a;
    if (activation_of(tr, t, &arg, &a) && linear_core(tr, arg, x, w, bias)) {
      // every interior use of the activation's argument is inside the activation: checked with the rest of the seal
      *act = a;
      m = tr;
      return true;
    }
  }
  return linear_core(m, t, x, w, bias);
}

// A Linear as the model code records it, widened by what follows it directly: the activation applied to its output
// (MLP::fwd phi2.rs:99-101, qwen2.rs:100-104) and / or one tensor added to the result (the residual sums of
// DecoderLayer::fwd phi2.rs:298, qwen2.rs:262-265), all of which the Linear launcher applies in its epilogue.  A plain
// product without bias, activation or residual is left to the MatMul rule (one launch either way) unless it has a
// single row: then it is taken, so that it can share a launch with the other Linears of that row (the bias-free
// q / k / v and gate / up projections of gemma.rs and qwen2.rs in a decode step).
bool match_linear(rai_tensor *t, Composite *c) {
  rai_tensor *x = nullptr, *w = nullptr, *bias = nullptr, *res = nullptr;
  int act = -1;
  Matcher m;
  const bool one_row = g_group_linears && !t->shape.empty() && numel_of(t->shape) == t->shape.back();
  bool found = act_linear(m, t, &x, &w, &bias, &act) && (bias || act >= 0 || one_row);
  if (!found && !t->evaluated && t->op == RAI_OP_BINARY && t->sub == RAI_BIN_ADD) {
    for (int side = 0; side < 2 && !found; ++side) {   // linear + r or r + linear
      Matcher mr;
      mr.interior.push_back(t);
      rai_tensor *lin = t->inputs[side], *other = t->inputs[1 - side];
      if (other->shape != t->shape || other->dtype != t->dtype) continue;
      if (act_linear(mr, lin, &x, &w, &bias, &act)) { m = mr; res = other; found = true; }
    }
  }
  if (!found || !m.ok) return false;
  c->kind = COMP_LINEAR;
  c->in[0] = x; c->in[1] = w; c->in[2] = bias; c->in[3] = res;
  c->i0 = act;
  c->interior = m.interior;
  return true;
}

// rai-models/src/llm/phi2.rs:66-77: cat([xs_rot * cos + cat([-x2, x1]) * sin, xs_pass]) on [B, H, S, D], tables narrowed to
// rows [offset, offset + S)
bool match_rope(rai_tensor *t, Composite *c) {
  Matcher m;
  if (!norm_dtype(t->dtype) || t->shape.size() != 4) return false;
  rai_tensor *cat = m.node(t, RAI_OP_CONCATENATE);
  if (!cat || cat->ip[0] != 3 || cat->inputs.size() != 2) return false;
  int64_t st = 0, len = 0, rd = 0, off_c = 0, off_s = 0, sl = 0;
  rai_tensor *xs = m.narrow(cat->inputs[1], 3, &st, &len);          // xs_pass
  if (!xs || xs->shape != t->shape) return false;
  rd = st;
  if (rd <= 0 || rd % 2 || st + len != t->shape[3]) return false;
  rai_tensor *p1, *p2, *xr, *cb, *rh, *sb;
  if (!m.bin(cat->inputs[0], RAI_BIN_ADD, &p1, &p2) || !m.bin(p1, RAI_BIN_MUL, &xr, &cb) || !m.bin(p2, RAI_BIN_MUL, &rh, &sb)) return false;
  if (m.narrow(xr, 3, &st, &len) != xs || st != 0 || len != rd) return false;       // xs_rot (recorded once more below: same node)
  rai_tensor *cosn = m.strip_bc(cb), *sinn = m.strip_bc(sb);
  rai_tensor *cos_t = m.narrow(cosn, 0, &off_c, &sl);
  if (!cos_t || sl != t->shape[2]) return false;
  rai_tensor *sin_t = m.narrow(sinn, 0, &off_s, &sl);
  if (!sin_t || sl != t->shape[2] || off_s != off_c) return false;
  rai_tensor *rhc = m.node(rh, RAI_OP_CONCATENATE);
  if (!rhc || rhc->ip[0] != 3 || rhc->inputs.size() != 2) return false;
  rai_tensor *x2 = m.un(rhc->inputs[0], RAI_UN_NEG);
  if (!x2) return false;
  rai_tensor *a = m.narrow(x2, 3, &st, &len);
  if (a != xr || st != rd / 2 || len != rd / 2) return false;
  rai_tensor *b = m.narrow(rhc->inputs[1], 3, &st, &len);
  if (b != xr || st != 0 || len != rd / 2 || !m.ok) return false;
  if (cos_t->shape.size() != 2 || cos_t->shape[1] != rd || sin_t->shape != cos_t->shape || cos_t->dtype != t->dtype ||
      sin_t->dtype != t->dtype)
    return false;
  c->kind = COMP_ROPE;
  c->in[0] = xs; c->in[1] = cos_t; c->in[2] = sin_t;
  c->i0 = rd; c->i1 = off_c;
  c->interior = m.interior;
  return true;
}

// rai-models/src/llm/phi2.rs:244-262: softmax(where(mask, -inf, q.f32 @ (k.f32.t() * scale))).to_dtype(v) @ v, then
// transpose(1, 2) and reshape to [B, S, H * D].  The mask, when present, must be the causal one of phi2.rs:104-109.
bool match_attention(rai_tensor *t, Composite *c) {
  Matcher m;
  if ((t->dtype != RAI_BF16 && t->dtype != RAI_F32 && t->dtype != RAI_F16) || t->shape.size() != 3) return false;
  rai_tensor *rs = m.node(t, RAI_OP_RESHAPE);
  rai_tensor *tr = rs ? m.node(rs->inputs[0], RAI_OP_TRANSPOSE) : nullptr;
  if (!tr || tr->shape.size() != 4 || !((tr->ip[0] == 1 && tr->ip[1] == 2) || (tr->ip[0] == 2 && tr->ip[1] == 1))) return false;
  rai_tensor *pv = m.node(tr->inputs[0], RAI_OP_MATMUL);
  if (!pv) return false;
  rai_tensor *v = pv->inputs[1];
  rai_tensor *sm = m.node(m.strip_cast(pv->inputs[0], t->dtype), RAI_OP_SOFTMAX);
  if (!sm || sm->dtype != RAI_F32 || sm->ip[0] != 3) return false;
  rai_tensor *w = sm->inputs[0];
  rai_tensor *mask = nullptr;
  if (!w->evaluated && w->op == RAI_OP_WHERE) {   // inputs [on_true, on_false, cond]
    m.interior.push_back(w);
    double fill = 0;
    if (!m.konst(w->inputs[0], &fill) || !(fill < 0 && std::isinf(fill))) return false;
    mask = m.strip_bc(w->inputs[2]);
    w = w->inputs[1];
  }
  rai_tensor *qk = m.node(w, RAI_OP_MATMUL);
  if (!qk) return false;
  rai_tensor *q = m.strip_cast(qk->inputs[0], RAI_F32);
  rai_tensor *kt, *sc;
  double scale = 0;
  if (!m.bin(qk->inputs[1], RAI_BIN_MUL, &kt, &sc) || !m.konst(sc, &scale)) return false;
  rai_tensor *ktn = m.node(kt, RAI_OP_TRANSPOSE);
  if (!ktn || !((ktn->ip[0] == 2 && ktn->ip[1] == 3) || (ktn->ip[0] == 3 && ktn->ip[1] == 2))) return false;
  rai_tensor *k = m.strip_cast(ktn->inputs[0], RAI_F32);
  if (!m.ok || q->shape.size() != 4 || k->shape.size() != 4 || v->shape != k->shape) return false;
  if (q->dtype != t->dtype || k->dtype != t->dtype || v->dtype != t->dtype) return false;
  const int64_t B = q->shape[0], H = q->shape[1], S = q->shape[2], D = q->shape[3], T = k->shape[2];
  if (k->shape[0] != B || k->shape[1] != H || k->shape[3] != D || t->shape[0] != B || t->shape[1] != S || t->shape[2] != H * D)
    return false;
  int causal = 0;
  if (mask) {   // u8 [S, T] uploaded from the host: 1 exactly where key j lies after query i
    if (mask->op != RAI_OP_FROM_ARRAY || mask->dtype != RAI_U8 || mask->shape.size() != 2 || mask->shape[0] != S ||
        mask->shape[1] != T || (int64_t)mask->host.size() != S * T || S > T)
      return false;
    auto seen = g_causal_masks.find(mask->id);   // one mask node serves every layer: check its bytes once per eval
    if (seen == g_causal_masks.end()) {
      bool is_causal = true;
      for (int64_t i = 0; i < S && is_causal; ++i)
        for (int64_t j = 0; j < T; ++j)
          if ((mask->host[i * T + j] != 0) != (j > i + (T - S))) { is_causal = false; break; }
      seen = g_causal_masks.emplace(mask->id, is_causal).first;
    }
    if (!seen->second) return false;
    causal = 1;
  }
  c->kind = COMP_ATTENTION;
  c->in[0] = q; c->in[1] = k; c->in[2] = v;
  c->f0 = scale;
  c->i0 = causal;
  c->i1 = 1;   // scores and softmax in f32 (phi2.rs:248-251)
  c->interior = m.interior;
  return true;
}

// RotaryEmbedding::fwd of qwen2.rs:60-71 / gemma.rs:92-103 on [B, H, S, D]: x * cos + rotate_half(x) * sin over the
// whole head, the tables narrowed to rows [offset, offset + S) and unsqueezed twice
bool match_rope_full(rai_tensor *t, Composite *c) {
  Matcher m;
  if (!norm_dtype(t->dtype) || t->shape.size() != 4 || m.bin_kind(t) != RAI_BIN_ADD) return false;
  rai_tensor *p1, *p2, *x, *cb, *rh, *sb;
  if (!m.bin(t, RAI_BIN_ADD, &p1, &p2) || !m.bin(p1, RAI_BIN_MUL, &x, &cb) || !m.bin(p2, RAI_BIN_MUL, &rh, &sb)) return false;
  if (x->shape != t->shape || x->dtype != t->dtype) return false;
  const int64_t D = t->shape[3], S = t->shape[2];
  if (D % 2) return false;
  int64_t off_c = 0, off_s = 0, sl = 0, st = 0, len = 0;
  // The narrowed and unsqueezed tables are shared by the q and the k embedding (one pair per call of
  // RotaryEmbedding::fwd): they are views that cost no launch and stay ordinary nodes; only the table behind them
  // and the offset are read here.
  auto table_behind = [](rai_tensor *n, int64_t *start, int64_t *rows) -> rai_tensor * {
    while (n && !n->evaluated && n->op == RAI_OP_RESHAPE) n = n->inputs[0];
    if (!n || n->evaluated || n->op != RAI_OP_NARROW || n->ip[0] != 0) return nullptr;
    *start = n->ip[1];
    *rows = n->ip[2];
    return n->inputs[0];
  };
  rai_tensor *cos_t = table_behind(m.strip_bc(cb), &off_c, &sl);
  if (!cos_t || sl != S) return false;
  rai_tensor *sin_t = table_behind(m.strip_bc(sb), &off_s, &sl);
  if (!sin_t || sl != S || off_s != off_c) return false;
  rai_tensor *rhc = m.node(rh, RAI_OP_CONCATENATE);
  if (!rhc || rhc->ip[0] != 3 || rhc->inputs.size() != 2) return false;
  rai_tensor *x2 = m.un(rhc->inputs[0], RAI_UN_NEG);
  if (!x2 || m.narrow(x2, 3, &st, &len) != x || st != D / 2 || len != D - D / 2) return false;
  if (m.narrow(rhc->inputs[1], 3, &st, &len) != x || st != 0 || len != D / 2 || !m.ok) return false;
  if (cos_t->shape.size() != 2 || cos_t->shape[1] != D || sin_t->shape != cos_t->shape || cos_t->dtype != t->dtype ||
      sin_t->dtype != t->dtype)
    return false;
  c->kind = COMP_ROPE;
  c->in[0] = x; c->in[1] = cos_t; c->in[2] = sin_t;
  c->i0 = D;
  c->i1 = off_c;
  c->interior = m.interior;
  return true;
}

// Whether `mask` is the additive causal mask of prepare_decoder_attention_mask (qwen2.rs:306-336, gemma.rs:341-362)
// for S queries on T keys: f32 [S, S] uploaded from the host with -inf exactly above the diagonal and 0 elsewhere,
// zeros for the T - S cached positions concatenated in front, broadcast to [B, 1, S, T] and cast to the model dtype.
// The nodes are shared by all layers and evaluated as they are; this only reads them.
bool is_additive_causal_mask(const rai_tensor *mask, int64_t S, int64_t T) {
  const rai_tensor *n = mask;
  for (int hop = 0; hop < 4 && n && !n->evaluated && (n->op == RAI_OP_BROADCAST || n->op == RAI_OP_TO_DTYPE); ++hop) n = n->inputs[0];
  if (!n || n->evaluated) return false;
  if (n->op == RAI_OP_CONCATENATE) {
    if (n->inputs.size() != 2 || n->ip[0] != 1 || n->shape.size() != 2) return false;
    const rai_tensor *z = n->inputs[0];
    if (z->op != RAI_OP_FULL || z->p0 != 0.0 || z->shape.size() != 2 || z->shape[0] != S || z->shape[1] != T - S) return false;
    n = n->inputs[1];
  } else if (T != S) {
    return false;
  }
  if (n->op != RAI_OP_FROM_ARRAY || n->dtype != RAI_F32 || n->shape.size() != 2 || n->shape[0] != S || n->shape[1] != S ||
      (int64_t)n->host.size() != S * S * 4)
    return false;
  auto seen = g_causal_masks.find(n->id);   // one mask serves every layer: its bytes are checked once per eval
  if (seen == g_causal_masks.end()) {
    const float *v = reinterpret_cast<const float *>(n->host.data());
    bool is_causal = true;
    for (int64_t i = 0; i < S && is_causal; ++i)
      for (int64_t j = 0; j < S; ++j) {
        const float e = v[i * S + j];
        if (j > i ? !(std::isinf(e) && e < 0) : e != 0.f) { is_causal = false; break; }
      }
    seen = g_causal_masks.emplace(n->id, is_causal).first;
  }
  return seen->second;
}

// Attention::fwd of qwen2.rs:205-221 / gemma.rs:238-254 in the model dtype: softmax(q k^T * scale [+ mask]) v,
// transposed and reshaped to [B, S, H * D], with repeat_kv (gemma.rs:191-201: unsqueeze, broadcast, reshape) seen
// through, so that the kernel reads each key / value head once instead of a materialised copy per query head.
bool match_attention_seq(rai_tensor *t, Composite *c) {
  Matcher m;
  if ((t->dtype != RAI_BF16 && t->dtype != RAI_F32 && t->dtype != RAI_F16) || t->shape.size() != 3) return false;
  rai_tensor *rs = m.node(t, RAI_OP_RESHAPE);
  rai_tensor *tr = rs ? m.node(rs->inputs[0], RAI_OP_TRANSPOSE) : nullptr;
  if (!tr || tr->shape.size() != 4 || !((tr->ip[0] == 1 && tr->ip[1] == 2) || (tr->ip[0] == 2 && tr->ip[1] == 1))) return false;
  rai_tensor *pv = m.node(tr->inputs[0], RAI_OP_MATMUL);
  if (!pv) return false;
  rai_tensor *sm = m.node(pv->inputs[0], RAI_OP_SOFTMAX);
  if (!sm || sm->dtype != t->dtype || sm->ip[0] != 3) return false;
  rai_tensor *w = sm->inputs[0], *mask = nullptr, *qk_n, *sc;
  if (m.bin_kind(w) == RAI_BIN_ADD) {
    rai_tensor *mb;
    if (!m.bin(w, RAI_BIN_ADD, &w, &mb)) return false;
    mask = m.strip_bc(mb);
  }
  double scale = 0;
  if (!m.bin(w, RAI_BIN_MUL, &qk_n, &sc) || !m.konst(sc, &scale)) return false;
  rai_tensor *qk = m.node(qk_n, RAI_OP_MATMUL);
  if (!qk) return false;
  rai_tensor *q = qk->inputs[0];
  rai_tensor *ktn = m.node(qk->inputs[1], RAI_OP_TRANSPOSE);
  if (!ktn || !((ktn->ip[0] == 2 && ktn->ip[1] == 3) || (ktn->ip[0] == 3 && ktn->ip[1] == 2))) return false;
  // repeat_kv: reshape [B, Hkv * rep, T, D] of broadcast [B, Hkv, rep, T, D] of reshape [B, Hkv, 1, T, D]
  auto behind_repeat = [&](rai_tensor *x) -> rai_tensor * {
    if (x->evaluated || x->op != RAI_OP_RESHAPE || x->shape.size() != 4) return x;
    rai_tensor *bc = x->inputs[0];
    if (bc->evaluated || bc->op != RAI_OP_BROADCAST || bc->shape.size() != 5) return x;
    rai_tensor *us = bc->inputs[0];
    if (us->evaluated || us->op != RAI_OP_RESHAPE || us->shape.size() != 5 || us->shape[2] != 1) return x;
    rai_tensor *src = us->inputs[0];
    if (src->shape.size() != 4 || src->shape[0] != bc->shape[0] || src->shape[1] != bc->shape[1] ||
        src->shape[2] != bc->shape[3] || src->shape[3] != bc->shape[4] || x->shape[1] != bc->shape[1] * bc->shape[2])
      return x;
    m.interior.push_back(x); m.interior.push_back(bc); m.interior.push_back(us);
    return src;
  };
  rai_tensor *k = behind_repeat(ktn->inputs[0]), *v = behind_repeat(pv->inputs[1]);
  if (!m.ok || q->shape.size() != 4 || k->shape.size() != 4 || v->shape != k->shape) return false;
  if (q->dtype != t->dtype || k->dtype != t->dtype || v->dtype != t->dtype) return false;
  const int64_t B = q->shape[0], H = q->shape[1], S = q->shape[2], D = q->shape[3], T = k->shape[2], Hkv = k->shape[1];
  if (k->shape[0] != B || Hkv < 1 || H % Hkv || k->shape[3] != D || t->shape[0] != B || t->shape[1] != S || t->shape[2] != H * D)
    return false;
  int causal = 0;
  if (mask) {
    if (S > T || !is_additive_causal_mask(mask, S, T)) return false;
    causal = 1;
  }
  c->kind = COMP_ATTENTION;
  c->in[0] = q; c->in[1] = k; c->in[2] = v;
  c->f0 = scale;
  c->i0 = causal;
  c->i1 = 0;   // scores in the model dtype
  c->interior = m.interior;
  return true;
}

// A single-token step of Attention::fwd (phi2.rs:202-264, qwen2.rs:166-221, gemma.rs:203-259) whose key / value
// caches have room to grow in place: rotary embedding of q and of the new k, both cache concatenations and the
// attention block are one launch of the decode attention kernel, which appends the new rows itself.  The two
// concatenation nodes are materialised by that launch (Composite::co): they share the old caches' buffers, one row
// longer.  Taken from the second cached step on (the first one grows the caches, ev_concatenate).
bool match_rope(rai_tensor *t, Composite *c);
bool match_rope_full(rai_tensor *t, Composite *c);
bool match_attention(rai_tensor *t, Composite *c);
bool match_attention_seq(rai_tensor *t, Composite *c);
bool match_decode_attention(rai_tensor *t, Composite *c) {
  Composite at = {}, rq = {}, rk = {};
  if (!match_attention(t, &at) && !match_attention_seq(t, &at)) return false;
  rai_tensor *q = at.in[0], *kc = at.in[1], *vc = at.in[2];
  if (at.i0 != 0 || q->shape[2] != 1 || (t->dtype != RAI_BF16 && t->dtype != RAI_F32)) return false;
  auto growable = [](const rai_tensor *cat) {
    if (cat->evaluated || cat->op != RAI_OP_CONCATENATE || cat->inputs.size() != 2 || cat->ip[0] != 2 || cat->shape.size() != 4)
      return false;
    const rai_tensor *base = cat->inputs[0], *add = cat->inputs[1];
    // a cache without room to grow (the prefill's, or one somebody already appended to) is moved into a buffer with
    // room by the launch itself (run_decode_attention)
    return base->evaluated && base->buf && base->shape.size() == 4 && add->shape.size() == 4 && add->shape[2] == 1;
  };
  if (!growable(kc) || !growable(vc)) return false;
  rai_tensor *knew = kc->inputs[1], *vx = vc->inputs[1];
  if (!match_rope(q, &rq) && !match_rope_full(q, &rq)) return false;
  if (!match_rope(knew, &rk) && !match_rope_full(knew, &rk)) return false;
  const int64_t T = kc->inputs[0]->shape[2];
  if (rq.in[1] != rk.in[1] || rq.in[2] != rk.in[2] || rq.i0 != rk.i0 || rq.i1 != rk.i1 || rq.i1 != T ||
      vc->inputs[0]->shape[2] != T)
    return false;
  c->kind = COMP_DECODE_ATTN;
  c->in[0] = rq.in[0]; c->in[1] = rk.in[0]; c->in[2] = vx;          // the new token's q, k, v before the rotary embedding
  c->in[3] = kc->inputs[0]; c->in[4] = vc->inputs[0];               // the caches so far
  c->in[5] = rq.in[1]; c->in[6] = rq.in[2];                         // cos / sin tables
  c->f0 = at.f0;
  c->i0 = rq.i0;    // rotary dim
  c->i1 = at.i1;    // f32 scores
  c->i2 = T;
  c->co[0] = kc; c->co[1] = vc;
  c->interior = at.interior;
  c->interior.insert(c->interior.end(), rq.interior.begin(), rq.interior.end());
  c->interior.insert(c->interior.end(), rk.interior.begin(), rk.interior.end());
  return true;
}

// Arrival counters of the decode attention kernel's context splits: one zeroed buffer per device, grown on demand
// (every launch leaves them at zero).
int decode_counters(int dev, size_t bytes, int **out) {
  static int *buf[16];
  static size_t have[16];
  RAI_REQUIRE(dev >= 0 && dev < 16, RAI_ERR_BAD_ARG, "device %d out of range", dev);
  if (bytes > have[dev]) {
    void *p = nullptr;
    RAI_TRY(rai_hip_alloc(dev, bytes, &p));
    RAI_HIP_TRY(hipMemsetAsync(p, 0, bytes, stream_of(dev)));
    if (buf[dev]) (void)rai_hip_release(buf[dev]);   // stream order: earlier launches are done with it
    buf[dev] = (int *)p;
    have[dev] = bytes;
  }
  *out = buf[dev];
  return RAI_OK;
}

int run_decode_attention(rai_tensor *t, const Composite &c) {
  rai_tensor *qx = c.in[0], *kx = c.in[1], *vx = c.in[2], *kb = c.in[3], *vb = c.in[4];
  const int64_t B = qx->shape[0], Hq = qx->shape[1], D = qx->shape[3], Hkv = kb->shape[1], T = c.i2;
  auto has_room = [&](const rai_tensor *b) { return b->cap_dim == 2 && !b->extended && T + 1 <= b->cap; };
  const bool in_place = has_room(kb) && has_room(vb) && kb->cap == vb->cap;
  const int64_t cap = in_place ? kb->cap : grown_capacity(T + 1);
  auto rows_ok = [&](const rai_tensor *x, int64_t H) {   // [B, H, 1, D] with the heads of a sequence side by side
    const rai_hip_tensor &v = x->view;
    return v.rank == 4 && v.shape[0] == B && v.shape[1] == H && v.shape[2] == 1 && v.shape[3] == D && v.stride[3] == 1 &&
           (H == 1 || v.stride[1] == D) && (uintptr_t)base_ptr(&v) % 16 == 0 && (B == 1 || v.stride[0] % 8 == 0);
  };
  auto cache_ok = [&](const rai_hip_tensor &v) {   // [B, Hkv, T, D] laid out for `cap` rows per head
    return v.rank == 4 && v.shape[0] == B && v.shape[1] == Hkv && v.shape[2] == T && v.shape[3] == D && v.stride[3] == 1 &&
           v.stride[2] == D && v.stride[1] == cap * D && (B == 1 || v.stride[0] == Hkv * cap * D) &&
           (uintptr_t)base_ptr(&v) % 16 == 0;
  };
  RAI_REQUIRE(rows_ok(qx, Hq) && rows_ok(kx, Hkv) && rows_ok(vx, Hkv) && D % 8 == 0 && kb->view.rank == 4 && vb->view.rank == 4 &&
                  kb->view.shape[2] == T && vb->view.shape[2] == T && (!in_place || (cache_ok(kb->view) && cache_ok(vb->view))),
              RAI_ERR_BAD_STRIDE, "decode attention: operand layout not served");
  const rai_hip_tensor &ct = c.in[5]->view, &sn = c.in[6]->view;
  RAI_REQUIRE(is_contiguous(&ct) && is_contiguous(&sn) && ct.rank == 2 && ct.shape[1] == c.i0 && T < ct.shape[0] &&
                  ct.dtype == t->dtype && sn.dtype == t->dtype,
              RAI_ERR_BAD_STRIDE, "decode attention: rotary tables not served");
  hipStream_t st = stream_of(t->dev);
  if (!st) return RAI_ERR_HIP;
  void *ws = nullptr;
  int *counters = nullptr;
  RAI_TRY(decode_counters(t->dev, attention_decode_counter_bytes((int)B, (int)Hq), &counters));
  // caches without room: both move, once, into buffers laid out for `cap` rows per head (two copies; from then on
  // every step appends in place)
  rai_hip_tensor cache_view[2] = {kb->view, vb->view};
  void *grown[2] = {nullptr, nullptr};
  if (!in_place) {
    for (int i = 0; i < 2; ++i) {
      const rai_tensor *base = i ? vb : kb;
      int rc = rai_hip_alloc(t->dev, (size_t)(B * Hkv * cap * D) * dtype_size(t->dtype), &grown[i]);
      rai_hip_tensor &v = cache_view[i];
      if (rc == RAI_OK) {
        memset(&v, 0, sizeof(v));
        v.data = grown[i];
        v.dtype = t->dtype;
        v.rank = 4;
        v.shape[0] = B; v.shape[1] = Hkv; v.shape[2] = T; v.shape[3] = D;
        v.stride[0] = Hkv * cap * D; v.stride[1] = cap * D; v.stride[2] = D; v.stride[3] = 1;
        ++g_stats.kernel_launches;
        rc = rai_hip_copy(t->dev, &base->view, &v);
      }
      if (rc != RAI_OK) {
        for (int j = 0; j <= i; ++j)
          if (grown[j]) (void)rai_hip_release(grown[j]);
        return rc;
      }
    }
  }
  auto drop_grown = [&]() {
    for (int j = 0; j < 2; ++j)
      if (grown[j]) (void)rai_hip_release(grown[j]);
  };
  if (!cache_ok(cache_view[0]) || !cache_ok(cache_view[1])) { drop_grown(); return fail(RAI_ERR_BAD_STRIDE, "decode attention: cache layout not served"); }
  int arc = rai_hip_alloc(t->dev, attention_decode_ws_bytes((int)B, (int)Hq, (int)D), &ws);
  if (arc == RAI_OK) arc = alloc_output(t);
  if (arc != RAI_OK) { if (ws) (void)rai_hip_release(ws); drop_grown(); return arc; }
  AttnDecodeArgs a;
  memset(&a, 0, sizeof(a));
  a.qkv = base_ptr(&qx->view);
  a.k_new = base_ptr(&kx->view);
  a.v_new = base_ptr(&vx->view);
  a.q_row_stride = qx->view.stride[0]; a.k_row_stride = kx->view.stride[0]; a.v_row_stride = vx->view.stride[0];
  a.kcache = base_ptr(&cache_view[0]);
  a.vcache = base_ptr(&cache_view[1]);
  a.out = t->view.data;
  a.out_row_stride = Hq * D;
  a.cos_t = base_ptr(&ct); a.sin_t = base_ptr(&sn);
  a.pos_dev = nullptr;
  a.pos_host = (int)T;
  a.rot = (int)c.i0;
  a.B = (int)B; a.Hq = (int)Hq; a.Hkv = (int)Hkv; a.D = (int)D; a.Tmax = (int)cap;
  a.scale = (float)c.f0;
  a.f32_scores = (int)c.i1;
  a.dtype = t->dtype;
  a.ws = (float *)ws;
  a.counters = counters;
  const int rc = launch_attention_decode(st, a);
  (void)rai_hip_release(ws);   // stream order keeps it intact until the launch is through
  if (rc != RAI_OK) { drop_grown(); return rc; }
  // the caches, one row longer: in the old caches' buffers, or in the grown ones, which the new nodes then own
  for (int i = 0; i < 2; ++i) {
    rai_tensor *cat = c.co[i], *base = cat->inputs[0];
    rai_hip_tensor v = cache_view[i];
    v.shape[2] = T + 1;
    if (in_place) {
      alias_storage(cat, base, v);
      base->extended = true;
    } else {
      cat->view = v;
      cat->buf = grown[i];
    }
    cat->cap_dim = 2;
    cat->cap = cap;
    cat->evaluated = true;
    ++g_stats.nodes_evaluated;
  }
  return RAI_OK;
}

// Compositions found in the tape: g_comps[t->comp] for a root t (flag kRoot), interior nodes carry kAbsorbed.
std::vector<Composite> g_comps;

// Registers composition c with root t when it is sealed: every interior node is pending, claimed by nobody else, has
// a rule (fusing never hides a missing rule), is referenced only by edges of the tape, and all of those edges come
// from inside the composition; operands are not interior; co-outputs are read, inside the tape, by the composition
// only.
bool claim(rai_tensor *t, Composite &c, rai_tensor *stands_for_root = nullptr) {
  const uint64_t stamp = ++g_stamp;
  // a node whose recorded use of the interior the root takes over (the regrouped sum below): counts as the root
  // where users are checked, and may be an operand
  if (stands_for_root) stands_for_root->stamp = stamp;
  for (int i = 0; i < 2; ++i)
    if (c.co[i]) c.co[i]->stamp = stamp;   // inside for the purpose of "who uses this node", yet materialised
  // interior = everything the matcher walked through except the root itself (the same node may have been reached
  // twice): stamped so that "inside" is one comparison
  std::vector<rai_tensor *> interior;
  for (rai_tensor *n : c.interior)
    if (n != t && n->stamp != stamp) { n->stamp = stamp; interior.push_back(n); }
  auto users_inside = [&](const rai_tensor *n) {
    for (int u = 0; u < n->n_users; ++u) {
      const rai_tensor *usr = g_users[n->users_at + u];
      if (usr != t && usr->stamp != stamp) return false;
    }
    return true;
  };
  for (rai_tensor *n : interior)   // evaluated constants are operands, not interior
    if (n->evaluated || !in_tape(n) || (n->flags & (kAbsorbed | kRoot | kCoOutput)) || !g_rules[n->op] ||
        n->refs != n->n_users || !users_inside(n))
      return false;
  for (int i = 0; i < 7; ++i)
    if (c.in[i] && c.in[i] != stands_for_root && c.in[i]->stamp == stamp) return false;   // an operand must be materialised
  for (int i = 0; i < 2; ++i) {
    rai_tensor *n = c.co[i];
    if (n && (n->evaluated || !in_tape(n) || (n->flags & (kAbsorbed | kRoot | kCoOutput)) || !g_rules[n->op] || !users_inside(n)))
      return false;
  }
  c.interior = interior;
  for (rai_tensor *n : interior) n->flags |= kAbsorbed;
  for (int i = 0; i < 2; ++i)
    if (c.co[i]) c.co[i]->flags |= kCoOutput;
  t->flags |= kRoot;
  t->comp = (int)g_comps.size();
  g_comps.push_back(c);
  return true;
}

// DecoderLayer::fwd of phi2.rs:298 sums two Linear outputs and the layer's input: (attn + mlp) + x.  One Linear
// launch takes one added tensor, so the sums are regrouped as attn + (mlp + x): the inner sum node, which nothing
// else can observe, receives mlp's Linear with x added, the outer one attn's Linear with that added.  Two launches
// instead of three (and of four without any composition); the result differs from the recorded grouping by
// rounding only, like every composed result.
bool claim_two_linears_and_residual(rai_tensor *t) {
  if (t->evaluated || t->op != RAI_OP_BINARY || t->sub != RAI_BIN_ADD || (t->dtype != RAI_BF16 && t->dtype != RAI_F32)) return false;
  for (int side = 0; side < 2; ++side) {
    rai_tensor *sum = t->inputs[side], *x = t->inputs[1 - side];
    if (sum->evaluated || !in_tape(sum) || sum->op != RAI_OP_BINARY || sum->sub != RAI_BIN_ADD || sum->refs != 1 ||
        sum->n_users != 1 || (sum->flags & (kAbsorbed | kRoot | kCoOutput | kOutput)) || x->shape != t->shape ||
        x->dtype != t->dtype || sum->shape != t->shape)
      continue;
    if (!x->evaluated && !(in_tape(x) && x->tape_idx < sum->tape_idx)) continue;   // x must be there when `sum` runs
    Composite outer = {}, inner = {};
    Matcher mp, mq;
    int act_p = -1, act_q = -1;
    mp.interior.push_back(t);
    mq.interior.push_back(sum);
    if (!act_linear(mp, sum->inputs[0], &outer.in[0], &outer.in[1], &outer.in[2], &act_p) || !mp.ok) continue;
    if (!act_linear(mq, sum->inputs[1], &inner.in[0], &inner.in[1], &inner.in[2], &act_q) || !mq.ok) continue;
    inner.kind = outer.kind = COMP_LINEAR;
    inner.in[3] = x;   inner.i0 = act_q; inner.interior = mq.interior;
    outer.in[3] = sum; outer.i0 = act_p; outer.interior = mp.interior;
    // the inner composition first: if the outer one then fails, the inner one stands by itself as "Linear + x" with
    // `sum` as its root, which would change what `sum` means: so the outer one is checked (not registered) first
    Composite probe = outer;
    const size_t before = g_comps.size();
    if (!claim(t, probe, sum)) continue;
    if (!claim(sum, inner)) {   // undo the outer claim
      for (rai_tensor *n : g_comps.back().interior) n->flags &= ~kAbsorbed;
      t->flags &= ~kRoot;
      t->comp = -1;
      g_comps.resize(before);
      continue;
    }
    // one row, no activation on either product, parameters in place: one launch for both (run_root)
    const Composite &po = g_comps[t->comp], &pi = g_comps[sum->comp];
    const int64_t N = t->shape.back();
    if (g_group_linears && t->dtype == RAI_BF16 && numel_of(t->shape) == N && act_p < 0 && act_q < 0 && !(sum->flags & kOutput) &&
        po.in[1]->evaluated && pi.in[1]->evaluated && (!po.in[2] || po.in[2]->evaluated) && (!pi.in[2] || pi.in[2]->evaluated)) {
      g_comps[t->comp].dual_inner = sum;
      sum->flags |= kGrouped;
    }
    return true;
  }
  return false;
}

void plan_compositions(const std::vector<rai_tensor *> &tape) {
  typedef bool (*match_fn)(rai_tensor *, Composite *);
  static const match_fn kMatchers[] = {match_layer_norm, match_rms_norm,  match_gemma_rms_norm,   match_linear,   match_rope,
                                       match_rope_full,  match_decode_attention, match_attention, match_attention_seq};
  g_causal_masks.clear();
  g_comps.clear();
  // consumers before producers: the widest composition around a node (a Linear with its activation and residual)
  // claims it before a narrower one (the Linear alone) is tried
  for (size_t ti = tape.size(); ti-- > 0;) {
    rai_tensor *t = tape[ti];
    if ((t->flags & (kAbsorbed | kRoot | kCoOutput)) || !g_rules[t->op]) continue;
    // cheap gate: every composition's root is one of these primitives
    const bool row_product = t->op == RAI_OP_MATMUL && g_group_linears && numel_of(t->shape) == t->shape.back();
    if (t->op != RAI_OP_BINARY && t->op != RAI_OP_RESHAPE && t->op != RAI_OP_CONCATENATE && !row_product) continue;
    if (claim_two_linears_and_residual(t)) continue;
    for (match_fn f : kMatchers) {
      Composite c = {};
      if (f(t, &c) && claim(t, c)) break;
    }
  }
}

// Linears of one activation row.  The q, k and v projections and the first MLP Linear of a decoder block read the same
// normalised row (phi2.rs:293-297; qwen2.rs:205-210 and 100-104 read theirs through RMSNorm): at one row each is a
// matrix-vector product that cannot fill the GPU by itself, so up to kGemvGroupMax Linear compositions that share
// their input run as one launch, at the position of the first of them in the tape (their weights and biases are
// parameters, there before the tape starts).  When the shared input is a LayerNorm / RMSNorm composition that nothing
// else reads, the norm goes into the same launch (the launcher applies it in its prologue) and is never materialised.
struct LinearGroup {
  std::vector<rai_tensor *> members;   // tape order; members[0] leads
  rai_tensor *norm;                    // root of the absorbed norm composition, or null
  // a view between the norm and the Linears that changes nothing at one row (the last-position `narrow` in front of
  // the head, phi2.rs:343-345), absorbed with the norm; or null
  rai_tensor *view;
};
std::vector<LinearGroup> g_groups;

// An unevaluated Narrow or Reshape that keeps every element (and so, at one row, the layout), seen by the tape only
bool identity_view(const rai_tensor *v) {
  return !v->evaluated && in_tape(v) && (v->op == RAI_OP_NARROW || v->op == RAI_OP_RESHAPE) && v->inputs.size() == 1 &&
         numel_of(v->shape) == numel_of(v->inputs[0]->shape) && v->refs == v->n_users &&
         !(v->flags & (kOutput | kAbsorbed | kRoot | kCoOutput | kGroupLead | kGrouped | kInlined)) && g_rules[v->op];
}

bool group_member(const rai_tensor *t) {
  if (!(t->flags & kRoot) || (t->flags & (kGroupLead | kGrouped)) || t->dtype != RAI_BF16) return false;
  const Composite &c = g_comps[t->comp];
  if (c.kind != COMP_LINEAR || c.in[3]) return false;
  const rai_tensor *x = c.in[0], *w = c.in[1], *b = c.in[2];
  const int64_t K = x->shape.back();
  if (numel_of(x->shape) != K || !gemv_group_serves((int)K, 1)) return false;
  return w->evaluated && (!b || b->evaluated);
}

void plan_linear_groups(const std::vector<rai_tensor *> &tape) {
  g_groups.clear();
  struct Open { rai_tensor *x; int group; };
  Open open[8];   // the groups met last: members of one group lie close together in the tape
  int n_open = 0, next = 0;
  for (rai_tensor *t : tape) {
    if (t->evaluated || !group_member(t)) continue;
    rai_tensor *x = g_comps[t->comp].in[0];
    int gi = -1;
    for (int i = 0; i < n_open; ++i)
      if (open[i].x == x && (int)g_groups[open[i].group].members.size() < kGemvGroupMax) gi = open[i].group;
    if (gi < 0) {
      gi = (int)g_groups.size();
      g_groups.push_back(LinearGroup{{}, nullptr, nullptr});
      open[next] = Open{x, gi};
      next = (next + 1) % 8;
      if (n_open < 8) ++n_open;
    }
    g_groups[gi].members.push_back(t);
  }
  for (size_t gi = 0; gi < g_groups.size(); ++gi) {
    LinearGroup &g = g_groups[gi];
    if (g.members.size() < 2) {
      // a single Linear stays by itself unless the norm in front of it can go into its launch
      rai_tensor *x1 = g_comps[g.members[0]->comp].in[0];
      if (identity_view(x1)) x1 = x1->inputs[0];
      const bool norm_root = !x1->evaluated && in_tape(x1) && (x1->flags & kRoot) && x1->refs == x1->n_users &&
                             (g_comps[x1->comp].kind == COMP_LAYER_NORM || g_comps[x1->comp].kind == COMP_RMS_NORM);
      if (!norm_root) { g.members.clear(); continue; }
    }
    g.members[0]->flags |= kGroupLead;
    g.members[0]->group = (int)gi;
    for (size_t i = 1; i < g.members.size(); ++i) g.members[i]->flags |= kGrouped;
    // the shared input: a norm composition read by this group only?
    rai_tensor *x = g_comps[g.members[0]->comp].in[0], *view = nullptr;
    if (identity_view(x)) { view = x; x = x->inputs[0]; }
    if (x->evaluated || !in_tape(x) || !(x->flags & kRoot) || (x->flags & (kOutput | kCoOutput | kGroupLead | kGrouped)) || x->refs != x->n_users ||
        x->dtype != RAI_BF16)
      continue;
    const Composite &nc = g_comps[x->comp];
    if (nc.kind != COMP_LAYER_NORM && nc.kind != COMP_RMS_NORM) continue;
    const uint64_t stamp = ++g_stamp;
    for (rai_tensor *m : g.members) {
      m->stamp = stamp;
      for (rai_tensor *n : g_comps[m->comp].interior) n->stamp = stamp;
    }
    bool sealed = true;
    if (view) {
      for (int u = 0; u < view->n_users && sealed; ++u) sealed = g_users[view->users_at + u]->stamp == stamp;
      view->stamp = stamp;
    }
    for (int u = 0; u < x->n_users && sealed; ++u) sealed = g_users[x->users_at + u]->stamp == stamp;
    if (!sealed) continue;
    g.norm = x;
    g.view = view;
    x->flags |= kAbsorbed;   // never materialised: the loop passes over it
    if (view) view->flags |= kAbsorbed;
  }
  for (LinearGroup &g : g_groups)   // a single Linear whose norm stayed outside: an ordinary composition again
    if (g.members.size() == 1 && !g.norm) {
      g.members[0]->flags &= ~kGroupLead;
      g.members[0]->group = -1;
      g.members.clear();
    }
}

int run_composite(rai_tensor *t, const Composite &c);
int eval_pending_inputs(rai_tensor *t);

// One launch for the whole group; RAI_ERR_UNSUPPORTED / RAI_ERR_BAD_STRIDE when the operands' layout is not served
// (nothing has been written then).
int launch_linear_group(const LinearGroup &g) {
  const rai_tensor *lead = g.members[0];
  const Composite *nc = g.norm ? &g_comps[g.norm->comp] : nullptr;
  const rai_tensor *x = nc ? nc->in[0] : g_comps[lead->comp].in[0];
  const int64_t K = x->shape.back();
  RAI_REQUIRE(x->dtype == RAI_BF16 && is_contiguous(&x->view), RAI_ERR_BAD_STRIDE, "linear group: input row not dense");
  GemvGroupArgs a;
  memset(&a, 0, sizeof(a));
  a.x = base_ptr(&x->view);
  a.K = (int)K;
  a.count = (int)g.members.size();
  a.ln_kind = -1;
  if (nc) {
    const rai_tensor *w = nc->in[1], *b = nc->kind == COMP_LAYER_NORM ? nc->in[2] : nullptr;
    RAI_REQUIRE(is_contiguous(&w->view) && (!b || is_contiguous(&b->view)), RAI_ERR_BAD_STRIDE, "linear group: norm parameters not dense");
    a.ln_w = base_ptr(&w->view);
    a.ln_b = b ? base_ptr(&b->view) : nullptr;
    a.ln_eps = (float)nc->f0;
    a.ln_kind = nc->kind == COMP_LAYER_NORM ? 0 : (nc->i2 ? 2 : 1);
  }
  for (int i = 0; i < a.count; ++i) {
    const Composite &c = g_comps[g.members[i]->comp];
    const rai_hip_tensor &w = c.in[1]->view;
    RAI_REQUIRE(w.rank == 2 && w.stride[1] == 1 && w.shape[1] == K && (!c.in[2] || is_contiguous(&c.in[2]->view)), RAI_ERR_BAD_STRIDE,
                "linear group: weight layout not served");
    a.W[i] = base_ptr(&w);
    a.ldw[i] = w.stride[0];
    a.bias[i] = c.in[2] ? base_ptr(&c.in[2]->view) : nullptr;
    a.N[i] = (int)w.shape[0];
    a.act[i] = (int)c.i0;
  }
  hipStream_t st = stream_of(lead->dev);
  if (!st) return RAI_ERR_HIP;
  for (int i = 0; i < a.count; ++i) {
    RAI_TRY(alloc_output(g.members[i]));
    a.out[i] = g.members[i]->view.data;
  }
  return launch_gemv_group(st, a);
}

// A composition's root through its fused launcher, or -- when that declines the operands' layout -- the recorded
// nodes one by one.
int run_dual_linear(rai_tensor *t, const Composite &outer, const Composite &inner) {
  const rai_tensor *x1 = outer.in[0], *w1 = outer.in[1], *b1 = outer.in[2], *x2 = inner.in[0], *w2 = inner.in[1], *b2 = inner.in[2],
                   *res = inner.in[3];
  const int64_t N = t->shape.back(), K1 = x1->shape.back(), K2 = x2->shape.back();
  auto row = [](const rai_tensor *v, int64_t n) { return v->dtype == RAI_BF16 && numel_of(v->shape) == n && is_contiguous(&v->view); };
  auto weight = [&](const rai_tensor *w, int64_t K) {
    return w->dtype == RAI_BF16 && w->view.rank == 2 && w->view.shape[0] == N && w->view.shape[1] == K && w->view.stride[1] == 1;
  };
  RAI_REQUIRE(row(x1, K1) && row(x2, K2) && row(res, N) && weight(w1, K1) && weight(w2, K2) && (!b1 || row(b1, N)) && (!b2 || row(b2, N)),
              RAI_ERR_BAD_STRIDE, "two Linears of one row: operand layout not served");
  hipStream_t st = stream_of(t->dev);
  if (!st) return RAI_ERR_HIP;
  RAI_TRY(alloc_output(t));
  return launch_linear_dual_row(st, t->dev, base_ptr(&x1->view), (int)K1, base_ptr(&w1->view), w1->view.stride[0], b1 ? base_ptr(&b1->view) : nullptr,
                                base_ptr(&x2->view), (int)K2, base_ptr(&w2->view), w2->view.stride[0], b2 ? base_ptr(&b2->view) : nullptr,
                                base_ptr(&res->view), t->view.data, (int)N);
}

int run_root(rai_tensor *t) {
  const Composite &c = g_comps[t->comp];
  if (c.dual_inner) {
    rai_tensor *sum = c.dual_inner;
    const Composite &inner = g_comps[sum->comp];
    int st = run_dual_linear(t, c, inner);
    if (st == RAI_OK) {
      ++g_stats.kernel_launches;
      g_stats.composed_regions += 2;
      g_stats.composed_nodes += c.interior.size() + inner.interior.size() + 2;
      return RAI_OK;
    }
    if (st != RAI_ERR_BAD_STRIDE && st != RAI_ERR_UNSUPPORTED && st != RAI_ERR_BAD_SHAPE && st != RAI_ERR_BAD_DTYPE) return st;
    drop_storage(t);
    // not served: the inner sum by itself first, then this root as an ordinary Linear with it added
    sum->flags &= ~kGrouped;
    g_comps[t->comp].dual_inner = nullptr;
    st = run_root(sum);
    if (st != RAI_OK) { drop_storage(sum); return st; }
    sum->evaluated = true;
    ++g_stats.nodes_evaluated;
  }
  int st = run_composite(t, c);
  if (st == RAI_OK) {
    ++g_stats.kernel_launches;
    ++g_stats.composed_regions;
    g_stats.composed_nodes += c.interior.size() + 1;
  } else if (st == RAI_ERR_BAD_STRIDE || st == RAI_ERR_UNSUPPORTED || st == RAI_ERR_BAD_SHAPE || st == RAI_ERR_BAD_DTYPE) {
    drop_storage(t);
    st = eval_pending_inputs(t);
    if (st == RAI_OK) st = g_rules[t->op](t);
  }
  return st;
}

int run_linear_group(const LinearGroup &g) {
  int st = launch_linear_group(g);
  if (st == RAI_OK) {
    ++g_stats.kernel_launches;
    if (g.norm) {
      ++g_stats.composed_regions;
      g_stats.composed_nodes += g_comps[g.norm->comp].interior.size() + 1;
    }
    for (rai_tensor *m : g.members) {
      ++g_stats.composed_regions;
      g_stats.composed_nodes += g_comps[m->comp].interior.size() + 1;
      if (m != g.members[0]) { m->evaluated = true; ++g_stats.nodes_evaluated; }   // the loop does the leader's
    }
    return RAI_OK;
  }
  if (st != RAI_ERR_BAD_STRIDE && st != RAI_ERR_UNSUPPORTED && st != RAI_ERR_BAD_SHAPE && st != RAI_ERR_BAD_DTYPE) return st;
  // not served as a group: the norm and every member by themselves
  for (rai_tensor *m : g.members) drop_storage(m);
  if (g.norm) {
    RAI_TRY(run_root(g.norm));
    g.norm->evaluated = true;
    ++g_stats.nodes_evaluated;
    if (g.view) {
      RAI_TRY(g_rules[g.view->op](g.view));
      g.view->evaluated = true;
      ++g_stats.nodes_evaluated;
    }
  }
  for (rai_tensor *m : g.members) {
    st = run_root(m);
    if (st != RAI_OK) { drop_storage(m); return st; }
    if (m != g.members[0]) { m->evaluated = true; ++g_stats.nodes_evaluated; }
  }
  return RAI_OK;
}

int run_composite(rai_tensor *t, const Composite &c) {
  if (c.kind == COMP_DECODE_ATTN) return run_decode_attention(t, c);
  RAI_TRY(alloc_output(t));
  switch (c.kind) {
    case COMP_LINEAR:
      return rai_hip_linear(t->dev, &c.in[0]->view, &c.in[1]->view, c.in[2] ? &c.in[2]->view : nullptr, (int32_t)c.i0,
                            c.in[3] ? &c.in[3]->view : nullptr, &t->view);
    case COMP_LAYER_NORM:
      return rai_hip_layer_norm(t->dev, &c.in[0]->view, &c.in[1]->view, &c.in[2]->view, c.f0, &t->view);
    case COMP_RMS_NORM:
      return rai_hip_rms_norm(t->dev, &c.in[0]->view, &c.in[1]->view, c.f0, (int32_t)c.i2, &t->view);
    case COMP_ROPE:
      return rai_hip_rope(t->dev, &c.in[0]->view, &c.in[1]->view, &c.in[2]->view, (int32_t)c.i0, c.i1, &t->view);
    case COMP_ATTENTION:
      return rai_hip_attention(t->dev, &c.in[0]->view, &c.in[1]->view, &c.in[2]->view, c.f0, (int32_t)c.i0, (int32_t)c.i1, &t->view);
    default:
      return fail(RAI_ERR_BAD_ARG, "unknown composition %d", c.kind);
  }
}

// Node-by-node evaluation of a composition's interior (when the fused launcher declines the operands' layout).
int eval_pending_inputs(rai_tensor *t) {
  for (rai_tensor *in : t->inputs) {
    if (in->evaluated) continue;
    RAI_TRY(eval_pending_inputs(in));
    rule_fn rule = g_rules[in->op];
    RAI_REQUIRE(rule, RAI_ERR_UNSUPPORTED, "Unimplemented { op: %s, device: Hip }", op_name(in->op));
    int st = rule(in);
    if (st != RAI_OK) { drop_storage(in); return st; }
    in->evaluated = true;
    ++g_stats.nodes_evaluated;
  }
  return RAI_OK;
}

void detach(rai_tensor *t) {  // tensor.rs: drop the inputs so the graph behind an evaluated node can be freed
  std::vector<rai_tensor *> ins;
  ins.swap(t->inputs);
  for (rai_tensor *i : ins) rai_tensor_release(i);
}

}  // namespace

extern "C" {

// ------------------------------------------------------------------ creation
rai_tensor *rai_full(double value, int32_t dtype, const int64_t *shape, int32_t rank, int32_t dev) {
  rai_tensor *t = new_node(dev, dtype, std::vector<int64_t>(shape, shape + rank), RAI_OP_FULL, {});
  t->p0 = value;
  return t;
}

rai_tensor *rai_arange(double start, double stop, double step, int32_t dtype, int32_t dev) {
  // ops/arange.rs:102-117: ceil((stop - start) / step) elements
  int64_t n = step != 0.0 ? (int64_t)ceil((stop - start) / step) : 0;
  if (n < 0) n = 0;
  rai_tensor *t = new_node(dev, dtype, {n}, RAI_OP_ARANGE, {});
  t->p0 = start;
  t->p1 = stop;
  t->p2 = step;
  return t;
}

rai_tensor *rai_from_array(const void *host, int32_t dtype, const int64_t *shape, int32_t rank, int32_t dev) {
  rai_tensor *t = new_node(dev, dtype, std::vector<int64_t>(shape, shape + rank), RAI_OP_FROM_ARRAY, {});
  const size_t bytes = (size_t)numel_of(t->shape) * dtype_size(dtype);
  t->host.assign((const uint8_t *)host, (const uint8_t *)host + bytes);
  return t;
}

// ------------------------------------------------------------------ primitives
rai_tensor *rai_to_dtype(rai_tensor *x, int32_t dtype) {
  if (x->dtype == dtype) {  // ops/to_dtype.rs:45-55: same dtype returns the tensor itself
    ++x->refs;
    return x;
  }
  return new_node(x->dev, dtype, x->shape, RAI_OP_TO_DTYPE, {x});
}

rai_tensor *rai_unary(int32_t op, rai_tensor *x, double param) {
  rai_tensor *t = new_node(x->dev, x->dtype, x->shape, RAI_OP_UNARY, {x});
  t->sub = op;
  t->p0 = param;
  return t;
}

rai_tensor *rai_binary(int32_t op, rai_tensor *lhs, rai_tensor *rhs) {
  // ops/mod.rs:298-340: operands are wrapped in Broadcast nodes where needed; the output takes lhs' dtype
  // (comparisons: U8)
  const int out_dtype = op >= RAI_BIN_EQ ? RAI_U8 : lhs->dtype;
  std::vector<int64_t> shape;
  bool lb, rb;
  if (!broadcast_shapes(lhs->shape, rhs->shape, &shape, &lb, &rb))
    return err_node(lhs->dev, out_dtype, {}, {lhs, rhs}, incompatible(lhs, rhs));
  rai_tensor *l = lb ? rai_broadcast_to(lhs, shape.data(), (int32_t)shape.size()) : lhs;
  rai_tensor *r = rb ? rai_broadcast_to(rhs, shape.data(), (int32_t)shape.size()) : rhs;
  rai_tensor *t = new_node(lhs->dev, out_dtype, shape, RAI_OP_BINARY, {l, r});
  t->sub = op;
  if (lb) rai_tensor_release(l);
  if (rb) rai_tensor_release(r);
  return t;
}

rai_tensor *rai_matmul(rai_tensor *lhs, rai_tensor *rhs) {
  // ops/matmul.rs:34-70 + shape.rs:130-160: rank-1 operands are promoted, leading dims broadcast
  rai_tensor *a = lhs, *b = rhs;
  const bool a1 = lhs->shape.size() == 1, b1 = rhs->shape.size() == 1;
  if (lhs->shape.empty() || rhs->shape.empty()) return err_node(lhs->dev, lhs->dtype, {}, {lhs, rhs}, incompatible(lhs, rhs));
  if (a1) { int64_t s[2] = {1, lhs->shape[0]}; a = rai_reshape(lhs, s, 2); }
  if (b1) { int64_t s[2] = {rhs->shape[0], 1}; b = rai_reshape(rhs, s, 2); }
  auto done = [&](rai_tensor *res) {
    if (a1) rai_tensor_release(a);
    if (b1) rai_tensor_release(b);
    return res;
  };
  const size_t ra = a->shape.size(), rbk = b->shape.size();
  const int64_t m = a->shape[ra - 2], k = a->shape[ra - 1], k2 = b->shape[rbk - 2], n = b->shape[rbk - 1];
  if (k != k2) return done(err_node(lhs->dev, lhs->dtype, {}, {lhs, rhs}, incompatible(lhs, rhs)));
  std::vector<int64_t> batch;
  bool lb = false, rb = false;
  if (ra > 2 || rbk > 2) {
    std::vector<int64_t> ab(a->shape.begin(), a->shape.end() - 2), bb(b->shape.begin(), b->shape.end() - 2);
    if (!broadcast_shapes(ab, bb, &batch, &lb, &rb)) return done(err_node(lhs->dev, lhs->dtype, {}, {lhs, rhs}, incompatible(lhs, rhs)));
  }
  std::vector<int64_t> sa = batch, sb = batch, so = batch;
  sa.push_back(m); sa.push_back(k);
  sb.push_back(k); sb.push_back(n);
  so.push_back(m); so.push_back(n);
  rai_tensor *aa = lb ? rai_broadcast_to(a, sa.data(), (int32_t)sa.size()) : a;
  rai_tensor *bb2 = rb ? rai_broadcast_to(b, sb.data(), (int32_t)sb.size()) : b;
  rai_tensor *t = new_node(lhs->dev, lhs->dtype, so, RAI_OP_MATMUL, {aa, bb2});
  if (lb) rai_tensor_release(aa);
  if (rb) rai_tensor_release(bb2);
  if (a1 || b1) {  // drop the promoted dims again
    std::vector<int64_t> s = so;
    if (b1) s.pop_back();
    if (a1) s.erase(s.end() - (b1 ? 1 : 2));
    rai_tensor *r = rai_reshape(t, s.data(), (int32_t)s.size());
    rai_tensor_release(t);
    t = r;
  }
  return done(t);
}

static rai_tensor *softmax_like(int op, rai_tensor *x, int32_t dim) {
  const int rank = (int)x->shape.size();
  const int d = norm_dim(dim, rank);
  if (d < 0 || d >= rank) return err_node(x->dev, x->dtype, x->shape, {x}, "dim out of range");
  rai_tensor *t = new_node(x->dev, x->dtype, x->shape, op, {x});
  t->ip = {d};
  return t;
}
rai_tensor *rai_softmax(rai_tensor *x, int32_t dim) { return softmax_like(RAI_OP_SOFTMAX, x, dim); }
rai_tensor *rai_log_softmax(rai_tensor *x, int32_t dim) { return softmax_like(RAI_OP_LOG_SOFTMAX, x, dim); }

rai_tensor *rai_reduce(int32_t op, rai_tensor *x, const int32_t *dims, int32_t ndims, int32_t keep_dim) {
  // shape.rs:162-173 shape_reduce
  const int rank = (int)x->shape.size();
  std::vector<int64_t> nd;
  for (int i = 0; i < ndims; ++i) {
    const int d = norm_dim(dims[i], rank);
    if (d < 0 || d >= rank) return err_node(x->dev, x->dtype, {}, {x}, "dim out of range");
    nd.push_back(d);
  }
  std::vector<int64_t> shape;
  for (int i = 0; i < rank; ++i) {
    bool red = false;
    for (int64_t d : nd) red |= d == i;
    if (!red) shape.push_back(x->shape[i]);
    else if (keep_dim) shape.push_back(1);
  }
  rai_tensor *t = new_node(x->dev, x->dtype, shape, RAI_OP_REDUCE, {x});
  t->sub = op;
  t->ip.push_back(keep_dim);
  for (int64_t d : nd) t->ip.push_back(d);
  return t;
}

static rai_tensor *arg_like(int op, rai_tensor *x, int32_t dim, int32_t keep_dim) {
  // ops/argmax.rs:48-61: output dtype U32
  const int rank = (int)x->shape.size();
  const int d = norm_dim(dim, rank);
  if (d < 0 || d >= rank) return err_node(x->dev, RAI_U32, {}, {x}, "dim out of range");
  std::vector<int64_t> shape;
  for (int i = 0; i < rank; ++i) {
    if (i != d) shape.push_back(x->shape[i]);
    else if (keep_dim) shape.push_back(1);
  }
  rai_tensor *t = new_node(x->dev, RAI_U32, shape, op, {x});
  t->ip = {d, keep_dim};
  return t;
}
rai_tensor *rai_argmax(rai_tensor *x, int32_t dim, int32_t keep_dim) { return arg_like(RAI_OP_ARGMAX, x, dim, keep_dim); }
rai_tensor *rai_argmin(rai_tensor *x, int32_t dim, int32_t keep_dim) { return arg_like(RAI_OP_ARGMIN, x, dim, keep_dim); }

rai_tensor *rai_index_select(rai_tensor *x, int32_t dim, rai_tensor *index) {
  // ops/index_select.rs:52-61: the selected dim becomes index.elem_count()
  const int rank = (int)x->shape.size();
  const int d = norm_dim(dim, rank);
  if (d < 0 || d >= rank) return err_node(x->dev, x->dtype, {}, {x, index}, "dim out of range");
  std::vector<int64_t> shape = x->shape;
  shape[d] = numel_of(index->shape);
  rai_tensor *t = new_node(x->dev, x->dtype, shape, RAI_OP_INDEX_SELECT, {x, index});
  t->ip = {d};
  return t;
}

static bool index_dtype(int dt) { return dt == RAI_U8 || dt == RAI_U32 || dt == RAI_I64; }

rai_tensor *rai_gather(rai_tensor *x, int32_t dim, rai_tensor *index) {
  // ops/gather.rs:47-60: equal ranks, equal shapes once `dim` is removed; the output has index's shape
  const int rank = (int)x->shape.size();
  const int d = norm_dim(dim, rank);
  if (d < 0 || d >= rank) return err_node(x->dev, x->dtype, {}, {x, index}, "dim out of range");
  if (index->shape.size() != x->shape.size() || !index_dtype(index->dtype))
    return err_node(x->dev, x->dtype, index->shape, {x, index}, incompatible(x, index));
  for (int i = 0; i < rank; ++i)
    if (i != d && index->shape[i] != x->shape[i]) return err_node(x->dev, x->dtype, index->shape, {x, index}, incompatible(x, index));
  rai_tensor *t = new_node(x->dev, x->dtype, index->shape, RAI_OP_GATHER, {x, index});
  t->ip = {d};
  return t;
}

rai_tensor *rai_index_add(rai_tensor *x, int32_t dim, rai_tensor *index, rai_tensor *source) {
  // ops/index_add.rs:52-62 (its asserts are a TODO there; the shapes candle's index_add requires are checked here)
  const int rank = (int)x->shape.size();
  const int d = norm_dim(dim, rank);
  if (d < 0 || d >= rank) return err_node(x->dev, x->dtype, x->shape, {x, source, index}, "dim out of range");
  bool ok = index->shape.size() == 1 && index_dtype(index->dtype) && source->shape.size() == x->shape.size() &&
            source->dtype == x->dtype;
  for (int i = 0; ok && i < rank; ++i) ok = source->shape[i] == (i == d ? index->shape[0] : x->shape[i]);
  if (!ok) return err_node(x->dev, x->dtype, x->shape, {x, source, index}, incompatible(x, source));
  rai_tensor *t = new_node(x->dev, x->dtype, x->shape, RAI_OP_INDEX_ADD, {x, source, index});
  t->ip = {d};
  return t;
}

rai_tensor *rai_scatter_add(rai_tensor *x, int32_t dim, rai_tensor *index, rai_tensor *source) {
  // ops/scatter_add.rs:52-60
  const int rank = (int)x->shape.size();
  const int d = norm_dim(dim, rank);
  if (d < 0 || d >= rank) return err_node(x->dev, x->dtype, x->shape, {x, source, index}, "dim out of range");
  bool ok = index->shape == source->shape && index->shape.size() == x->shape.size() && index_dtype(index->dtype) &&
            source->dtype == x->dtype;
  for (int i = 0; ok && i < rank; ++i) ok = i == d || index->shape[i] == x->shape[i];
  if (!ok) return err_node(x->dev, x->dtype, x->shape, {x, source, index}, incompatible(x, source));
  rai_tensor *t = new_node(x->dev, x->dtype, x->shape, RAI_OP_SCATTER_ADD, {x, source, index});
  t->ip = {d};
  return t;
}

rai_tensor *rai_narrow(rai_tensor *x, int32_t dim, int64_t start, int64_t len) {
  const int rank = (int)x->shape.size();
  const int d = norm_dim(dim, rank);
  if (d < 0 || d >= rank || start < 0 || len < 0 || start + len > x->shape[d])
    return err_node(x->dev, x->dtype, x->shape, {x}, "narrow out of range");
  std::vector<int64_t> shape = x->shape;
  shape[d] = len;
  rai_tensor *t = new_node(x->dev, x->dtype, shape, RAI_OP_NARROW, {x});
  t->ip = {d, start, len};
  return t;
}

rai_tensor *rai_concatenate(rai_tensor *const *xs, int32_t n, int32_t dim) {
  // ops/concatenate.rs:54-67
  rai_tensor *t1 = xs[0];
  const int rank = (int)t1->shape.size();
  const int d = norm_dim(dim, rank);
  std::vector<rai_tensor *> ins(xs, xs + n);
  if (d < 0 || d >= rank) return err_node(t1->dev, t1->dtype, t1->shape, ins, "dim out of range");
  std::vector<int64_t> shape = t1->shape;
  shape[d] = 0;
  for (int i = 0; i < n; ++i) {
    if ((int)xs[i]->shape.size() != rank || xs[i]->dtype != t1->dtype)
      return err_node(t1->dev, t1->dtype, t1->shape, ins, incompatible(t1, xs[i]));
    for (int k = 0; k < rank; ++k)
      if (k != d && xs[i]->shape[k] != t1->shape[k]) return err_node(t1->dev, t1->dtype, t1->shape, ins, incompatible(t1, xs[i]));
    shape[d] += xs[i]->shape[d];
  }
  rai_tensor *t = new_node(t1->dev, t1->dtype, shape, RAI_OP_CONCATENATE, ins);
  t->ip = {d};
  return t;
}

rai_tensor *rai_where(rai_tensor *cond, rai_tensor *on_true, rai_tensor *on_false) {
  // ops/where.rs:37-45: shape of the condition, dtype of the branches, inputs [on_true, on_false, cond]
  if (on_true->dtype != on_false->dtype || on_true->shape != cond->shape || on_false->shape != cond->shape)
    return err_node(cond->dev, on_true->dtype, cond->shape, {on_true, on_false, cond}, incompatible(on_true, on_false));
  return new_node(cond->dev, on_true->dtype, cond->shape, RAI_OP_WHERE, {on_true, on_false, cond});
}

rai_tensor *rai_transpose(rai_tensor *x, int32_t dim0, int32_t dim1) {
  const int rank = (int)x->shape.size();
  const int a = norm_dim(dim0, rank), b = norm_dim(dim1, rank);
  if (a < 0 || a >= rank || b < 0 || b >= rank) return err_node(x->dev, x->dtype, x->shape, {x}, "dim out of range");
  std::vector<int64_t> shape = x->shape;
  std::swap(shape[a], shape[b]);
  rai_tensor *t = new_node(x->dev, x->dtype, shape, RAI_OP_TRANSPOSE, {x});
  t->ip = {a, b};
  return t;
}

rai_tensor *rai_reshape(rai_tensor *x, const int64_t *shape, int32_t rank) {
  // ops/reshape.rs:50-78: an equal shape returns the tensor itself; a different element count is an Err node
  std::vector<int64_t> s(shape, shape + rank);
  if (s == x->shape) {
    ++x->refs;
    return x;
  }
  if (numel_of(s) != numel_of(x->shape)) {
    rai_tensor *e = err_node(x->dev, x->dtype, s, {x},
                             "IncompatibleShape { lhs: " + shape_str(x->shape) + ", rhs: " + shape_str(s) + " }");
    return e;
  }
  rai_tensor *t = new_node(x->dev, x->dtype, s, RAI_OP_RESHAPE, {x});
  t->ip = s;
  return t;
}

rai_tensor *rai_permute(rai_tensor *x, const int32_t *dims, int32_t rank) {
  if (rank != (int32_t)x->shape.size()) return err_node(x->dev, x->dtype, x->shape, {x}, "permute rank mismatch");
  std::vector<int64_t> shape(rank), ip(rank);
  std::vector<bool> seen(rank, false);
  for (int i = 0; i < rank; ++i) {
    const int d = norm_dim(dims[i], rank);
    if (d < 0 || d >= rank || seen[d]) return err_node(x->dev, x->dtype, x->shape, {x}, "permute dims are not a permutation");
    seen[d] = true;
    shape[i] = x->shape[d];
    ip[i] = d;
  }
  rai_tensor *t = new_node(x->dev, x->dtype, shape, RAI_OP_PERMUTE, {x});
  t->ip = ip;
  return t;
}

rai_tensor *rai_broadcast_to(rai_tensor *x, const int64_t *shape, int32_t rank) {
  std::vector<int64_t> s(shape, shape + rank), out;
  bool lb, rb;
  if (!broadcast_shapes(x->shape, s, &out, &lb, &rb) || out != s)
    return err_node(x->dev, x->dtype, s, {x},
                    "IncompatibleShape { lhs: " + shape_str(x->shape) + ", rhs: " + shape_str(s) + " }");
  return new_node(x->dev, x->dtype, s, RAI_OP_BROADCAST, {x});
}

rai_tensor *rai_to_device(rai_tensor *x, int32_t dev) {
  if (x->dev == dev) {   // ops/to_device.rs:49-52: already there, the same tensor
    ++x->refs;
    return x;
  }
  return new_node(dev, x->dtype, x->shape, RAI_OP_TO_DEVICE, {x});
}
rai_tensor *rai_to_contiguous(rai_tensor *x) { return new_node(x->dev, x->dtype, x->shape, RAI_OP_TO_CONTIGUOUS, {x}); }

// ------------------------------------------------------------------ handles and metadata
void rai_tensor_retain(rai_tensor *t) {
  if (t) ++t->refs;
}

void rai_tensor_release(rai_tensor *t) {
  // iterative: a long chain of nodes must not recurse once per node
  std::vector<rai_tensor *> work;
  if (t) work.push_back(t);
  while (!work.empty()) {
    rai_tensor *n = work.back();
    work.pop_back();
    if (--n->refs > 0) continue;
    for (rai_tensor *i : n->inputs) work.push_back(i);
    if (n->buf) (void)rai_hip_release(n->buf);
    delete n;
  }
}

int32_t rai_tensor_rank(const rai_tensor *t) { return (int32_t)t->shape.size(); }
int32_t rai_tensor_dtype(const rai_tensor *t) { return t->dtype; }
int32_t rai_tensor_device(const rai_tensor *t) { return t->dev; }
int32_t rai_tensor_op(const rai_tensor *t) { return t->op; }
int32_t rai_tensor_shape(const rai_tensor *t, int64_t *shape_out) {
  for (size_t i = 0; i < t->shape.size(); ++i) shape_out[i] = t->shape[i];
  return (int32_t)t->shape.size();
}
int32_t rai_tensor_is_evaluated(const rai_tensor *t) { return t->evaluated ? 1 : 0; }
int32_t rai_tensor_num_inputs(const rai_tensor *t) { return (int32_t)t->inputs.size(); }
uint64_t rai_tensor_id(const rai_tensor *t) { return t->id; }
const char *rai_tensor_error(const rai_tensor *t) { return t->op == RAI_OP_ERR ? t->err.c_str() : nullptr; }

int rai_tensor_storage(const rai_tensor *t, rai_hip_tensor *out) {
  RAI_REQUIRE(t && out, RAI_ERR_BAD_ARG, "null argument");
  RAI_REQUIRE(t->evaluated, RAI_ERR_BAD_ARG, "tensor %llu is not evaluated", (unsigned long long)t->id);
  *out = t->view;
  return RAI_OK;
}

// ------------------------------------------------------------------ evaluation
rai_tensor *rai_from_storage(const rai_hip_tensor *view, void *buf, int32_t dev) {
  if (!view || !buf || view->rank < 0 || view->rank > RAI_HIP_MAX_RANK || dtype_size(view->dtype) == 0) return nullptr;
  std::vector<int64_t> shape(view->shape, view->shape + view->rank);
  rai_tensor *t = new_node(dev, view->dtype, shape, RAI_OP_FROM_ARRAY, {});
  if (rai_hip_retain(buf) != RAI_OK) { rai_tensor_release(t); return nullptr; }
  t->view = *view;
  t->buf = buf;
  t->evaluated = true;
  return t;
}

void *rai_tensor_buffer(const rai_tensor *t) { return t && t->evaluated ? t->buf : nullptr; }

int rai_graph_eval_order(rai_tensor *const *outputs, int32_t n, uint64_t *ids, int32_t capacity, int32_t *count) {
  RAI_REQUIRE(outputs && count && n >= 0, RAI_ERR_BAD_ARG, "null argument");
  std::vector<rai_tensor *> tape;
  RAI_TRY(topo_sort(outputs, n, &tape));
  *count = (int32_t)tape.size();
  for (int i = 0; i < *count && i < capacity; ++i) ids[i] = tape[i]->id;
  return RAI_OK;
}

int rai_eval(rai_tensor *const *outputs, int32_t n, int32_t retain_graph) {
  RAI_REQUIRE(outputs && n >= 0, RAI_ERR_BAD_ARG, "null argument");
  init_rules();
  g_group_linears = getenv("RAI_HIP_GRAPH_NO_LINEAR_GROUPS") == nullptr;
  const auto t_start = std::chrono::steady_clock::now();
  std::vector<rai_tensor *> tape;
  RAI_TRY(topo_sort(outputs, n, &tape));
  for (int i = 0; i < n; ++i)
    if (in_tape(outputs[i])) outputs[i]->flags |= kOutput;
  index_users(tape);
  g_comps.clear();
  g_groups.clear();
  if (g_compose) {
    plan_compositions(tape);
    if (g_group_linears) plan_linear_groups(tape);
  }
  if (g_fusion) plan_fusion(tape);
  const auto t_planned = std::chrono::steady_clock::now();
  g_stats.plan_ns += (uint64_t)std::chrono::duration_cast<std::chrono::nanoseconds>(t_planned - t_start).count();
  int rc = RAI_OK;
  // The walk owns one reference to every tape node and hands it back as it passes the node, after dropping the
  // node's inputs (eval.rs:45-49 detaches inside the loop): an intermediate result is freed as soon as its last
  // consumer has run, so a long tape reuses the buffers of its early nodes instead of holding every activation of
  // every layer until the end.  (Taken after planning, which compares reference counts with in-tape uses.)
  for (rai_tensor *t : tape) ++t->refs;
  // A composition's operands are kept by pointer; most are held by the root's own inputs, but one reached behind a
  // shared view (the rotary tables) is not once that view has been passed: the plan holds a reference of its own to
  // every operand until the composition's root has run (or, for roots that never run themselves, until the end).
  std::vector<char> operands_held(g_comps.size(), 1);
  auto release_operands = [&](int ci) {
    if (ci < 0 || !operands_held[ci]) return;
    operands_held[ci] = 0;
    for (rai_tensor *o : g_comps[ci].in)
      if (o) rai_tensor_release(o);
  };
  for (const Composite &c : g_comps)
    for (rai_tensor *o : c.in)
      if (o) ++o->refs;
  std::vector<rai_tensor *> late;   // co-outputs: materialised by a root further on, handed back after the walk
  size_t at = 0;
  for (; at < tape.size(); ++at) {
    rai_tensor *t = tape[at];
    auto hand_back = [&]() {
      if (t->flags & kCoOutput) { late.push_back(t); return; }
      if ((t->flags & kRoot) && t->evaluated) release_operands(t->comp);
      if (t->evaluated && !retain_graph) detach(t);
      rai_tensor_release(t);
    };
    if (t->evaluated || (t->flags & (kInlined | kAbsorbed | kCoOutput | kGrouped))) {   // a co-output comes with its root
      hand_back();
      continue;
    }
    rule_fn rule = g_rules[t->op];
    if (!rule) { rc = fail(RAI_ERR_UNSUPPORTED, "Unimplemented { op: %s, device: Hip }", op_name(t->op)); break; }
    int st = RAI_ERR_UNSUPPORTED;
    if (t->flags & kGroupLead) {
      st = run_linear_group(g_groups[t->group]);
    } else if (t->flags & kRoot) {
      st = run_root(t);
    } else if (elementwise(t) && has_inlined_input(t)) {
      // the rules of the inlined members must exist too: fusion never hides a missing rule
      st = eval_region(t);
      if (st == RAI_ERR_UNSUPPORTED) {  // region too large for one program: evaluate its members one by one
        drop_storage(t);
        st = eval_inputs_plain(t);
        if (st == RAI_OK) st = rule(t);
      }
    } else {
      st = rule(t);
    }
    if (st != RAI_OK) {
      drop_storage(t);
      rc = st;
      break;
    }
    t->evaluated = true;
    ++g_stats.nodes_evaluated;
    hand_back();
  }
  for (rai_tensor *t : late) {
    if (rc == RAI_OK && t->evaluated && !retain_graph) detach(t);
    rai_tensor_release(t);
  }
  for (; at < tape.size(); ++at) rai_tensor_release(tape[at]);   // after a failure: the nodes the walk never passed
  for (size_t ci = 0; ci < g_comps.size(); ++ci) release_operands((int)ci);
  g_stats.run_ns += (uint64_t)std::chrono::duration_cast<std::chrono::nanoseconds>(std::chrono::steady_clock::now() - t_planned).count();
  return rc;
}

int rai_tensor_to_host(rai_tensor *t, void *dst, size_t bytes) {
  RAI_REQUIRE(t && dst, RAI_ERR_BAD_ARG, "null argument");
  if (!t->evaluated) {
    rai_tensor *outs[1] = {t};
    RAI_TRY(rai_eval(outs, 1, 0));
  }
  const size_t want = (size_t)numel_of(t->shape) * dtype_size(t->dtype);
  RAI_REQUIRE(bytes == want, RAI_ERR_BAD_SHAPE, "to_host: tensor holds %zu bytes, buffer has %zu", want, bytes);
  if (want == 0) return RAI_OK;
  if (is_contiguous(&t->view)) return rai_hip_d2h(t->dev, dst, base_ptr(&t->view), want);
  // Tensor::as_vec of a strided view: contiguous copy first
  void *tmp = nullptr;
  RAI_TRY(rai_hip_alloc(t->dev, want, &tmp));
  rai_hip_tensor c;
  memset(&c, 0, sizeof(c));
  c.data = tmp;
  c.dtype = t->dtype;
  c.rank = t->view.rank;
  int64_t st = 1;
  for (int i = c.rank - 1; i >= 0; --i) {
    c.shape[i] = t->view.shape[i];
    c.stride[i] = st;
    st *= c.shape[i];
  }
  int rc = rai_hip_copy(t->dev, &t->view, &c);
  if (rc == RAI_OK) rc = rai_hip_d2h(t->dev, dst, tmp, want);
  (void)rai_hip_release(tmp);
  return rc;
}

// ------------------------------------------------------------------ dispatcher
int rai_dispatch_unregister(int32_t op_kind) {
  RAI_REQUIRE(op_kind >= 0 && op_kind < RAI_OP_COUNT_, RAI_ERR_BAD_ARG, "op kind %d", op_kind);
  init_rules();
  g_rules[op_kind] = nullptr;
  return RAI_OK;
}
int rai_dispatch_register_builtin(int32_t op_kind) {
  RAI_REQUIRE(op_kind >= 0 && op_kind < RAI_OP_COUNT_, RAI_ERR_BAD_ARG, "op kind %d", op_kind);
  init_rules();
  g_rules[op_kind] = kBuiltin[op_kind];
  return RAI_OK;
}
int32_t rai_dispatch_has_rule(int32_t op_kind) {
  init_rules();
  return op_kind >= 0 && op_kind < RAI_OP_COUNT_ && g_rules[op_kind] != nullptr;
}

// ------------------------------------------------------------------ fusion control and counters
int rai_graph_set_compose(int32_t enabled) {
  g_compose = enabled != 0;
  return RAI_OK;
}
int rai_graph_set_fusion(int32_t enabled) {
  g_fusion = enabled != 0;
  return RAI_OK;
}
int rai_graph_get_stats(rai_graph_stats *out, int32_t reset) {
  if (out) *out = g_stats;
  if (reset) g_stats = rai_graph_stats{0, 0, 0, 0};
  return RAI_OK;
}

}  // extern "C"
