/*
 * rai_hip.h — C ABI of librai_hip.so, the gfx950 (MI355X) execution device for
 * the rai lazy-tensor framework.
 *
 * Every entry point below is what a `Hip` device in rai-core would bind through
 * `extern "C"`: one launcher per primitive that rai's evaluator dispatches
 * (`trait Eval<D, P>::eval`, rai-core/src/backend/mod.rs:48-54), plus the storage
 * calls behind `TensorLike` (rai-core/src/tensor.rs:19-26).  The comment above
 * each declaration cites the reference implementation it replaces
 * (paths relative to the rai source tree, v0.11.0).
 *
 * Conventions
 *   - Plain C: pointers, sizes, PODs.  No C++/torch types.
 *   - Every function returns 0 on success or a negative rai_hip_status;
 *     rai_hip_last_error() returns a thread-local message for the last failure.
 *     The reference backend `unwrap()`s every backend error (panic); a binding
 *     should panic/raise on any non-zero status.
 *   - All device work is enqueued on one HIP stream per device and is
 *     asynchronous; only rai_hip_sync / rai_hip_d2h / rai_hip_timer_elapsed_ms block.
 *   - A tensor is a strided view: element (i0..ir) lives at
 *     data + (offset + sum(i_k * stride[k])) * sizeof(dtype).  Strides are in
 *     elements, may be 0 (broadcast) and are never negative.
 *   - Outputs never alias inputs (functional semantics, like the reference).
 */
#ifndef RAI_HIP_H
#define RAI_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RAI_HIP_MAX_RANK 8

/* rai-core/src/dtype.rs: U8, U32, I64, F16, BF16, F32, F64 */
typedef enum rai_hip_dtype {
  RAI_U8 = 0,
  RAI_U32 = 1,
  RAI_I64 = 2,
  RAI_F16 = 3,
  RAI_BF16 = 4,
  RAI_F32 = 5,
  RAI_F64 = 6
} rai_hip_dtype;

typedef enum rai_hip_status {
  RAI_OK = 0,
  RAI_ERR_BAD_DTYPE = -1,
  RAI_ERR_BAD_SHAPE = -2,
  RAI_ERR_BAD_STRIDE = -3,
  RAI_ERR_OOM = -4,
  RAI_ERR_HIP = -5,
  RAI_ERR_BAD_ARG = -6,
  RAI_ERR_UNSUPPORTED = -7, /* rai-core/src/error.rs:10-14 Error::Unimplemented */
  RAI_ERR_INDEX = -8,       /* gather index out of range: never silent */
  RAI_ERR_PARAM_NOT_FOUND = -9, /* rai-core/src/error.rs Error::ParamNotFound (nn.rs:198-204) */
  RAI_ERR_IO = -10          /* unreadable or malformed checkpoint file */
} rai_hip_status;

/* Strided tensor view over device memory (the storage half of
 * rai-core/src/tensor.rs:19-37; candle's Layout{shape,stride,start_offset}). */
typedef struct rai_hip_tensor {
  void *data;     /* device pointer to the start of the underlying buffer */
  int32_t dtype;  /* rai_hip_dtype */
  int32_t rank;   /* 0..RAI_HIP_MAX_RANK */
  int64_t shape[RAI_HIP_MAX_RANK];
  int64_t stride[RAI_HIP_MAX_RANK]; /* elements */
  int64_t offset;                   /* elements */
} rai_hip_tensor;

/* Unary primitives of rai-core/src/ops/ evaluated at
 * rai-core/src/backend/candle.rs:445-473,525-553,608-656,947-978 */
typedef enum rai_hip_unary_op {
  RAI_UN_SIN = 0,
  RAI_UN_COS = 1,
  RAI_UN_NEG = 2,
  RAI_UN_SQUARE = 3,
  RAI_UN_SQRT = 4,
  RAI_UN_RSQRT = 5, /* sqrt then reciprocal, candle.rs:545-553 */
  RAI_UN_ABS = 6,
  RAI_UN_EXP = 7,
  RAI_UN_LOG = 8,
  RAI_UN_LOG2 = 9,  /* ln(x)/ln(2), candle.rs:628-636 */
  RAI_UN_LOG10 = 10,
  RAI_UN_ERF = 11,
  RAI_UN_TANH = 12,
  RAI_UN_POWF = 13, /* param = exponent */
  RAI_UN_SIGN = 14, /* (x>=0) - (x<=0), candle.rs:595-606 */
  /* fused activations (rai-core/src/hlops/activations.rs:5-32) */
  RAI_UN_GELU = 15,     /* x*0.5*(1+erf(x/sqrt(2))) */
  RAI_UN_NEW_GELU = 16, /* tanh approximation */
  RAI_UN_SILU = 17,     /* x/(exp(-x)+1) */
  RAI_UN_RELU = 18,
  RAI_UN_COUNT_
} rai_hip_unary_op;

/* rai-core/src/backend/candle.rs:275-325 (arith), :658-760 (compare, max/min) */
typedef enum rai_hip_binary_op {
  RAI_BIN_ADD = 0,
  RAI_BIN_SUB = 1,
  RAI_BIN_MUL = 2,
  RAI_BIN_DIV = 3,
  RAI_BIN_MAXIMUM = 4,
  RAI_BIN_MINIMUM = 5,
  RAI_BIN_EQ = 6, /* comparisons write U8 0/1 */
  RAI_BIN_NE = 7,
  RAI_BIN_GT = 8,
  RAI_BIN_GE = 9,
  RAI_BIN_LT = 10,
  RAI_BIN_LE = 11,
  RAI_BIN_COUNT_
} rai_hip_binary_op;

typedef enum rai_hip_reduce_op { RAI_RED_SUM = 0, RAI_RED_MAX = 1, RAI_RED_MIN = 2 } rai_hip_reduce_op;

/* ------------------------------------------------------------------ runtime */

/* Thread-local text of the last failure on the calling thread ("" if none). */
const char *rai_hip_last_error(void);

/* Number of visible HIP devices (rai-core/src/device.rs:198-204 cuda_if_available). */
int rai_hip_device_count(int *count);

/* Lazily create the per-device context: one stream, allocator pools.  Idempotent.
 * Replaces the device cache at rai-core/src/backend/candle.rs:139-195. */
int rai_hip_init(int dev);

/* Block until everything enqueued on the device's stream has finished. */
int rai_hip_sync(int dev);

/* Ref-counted device allocation (refcount starts at 1).  Freed blocks go back to
 * a per-device size-class pool, so steady-state evaluation calls no hipMalloc;
 * blocks of up to 32 MiB are cut from 256 MiB slabs, so the first use of a size
 * costs no hipMalloc of its own either.
 * Replaces candle's Arc<Storage> behind rai-core/src/tensor.rs:151-165 set_data. */
int rai_hip_alloc(int dev, size_t bytes, void **out);
int rai_hip_retain(void *ptr);
int rai_hip_release(void *ptr);
/* bytes currently handed out / bytes held in the pool / number of real hipMalloc calls */
int rai_hip_mem_stats(int dev, uint64_t *in_use, uint64_t *pooled, uint64_t *n_device_mallocs);
/* Return pooled blocks to the driver (blocks cut from a slab stay pooled: a slab is
 * never handed back piecemeal). */
int rai_hip_trim(int dev);

/* Host<->device copies of raw bytes.  h2d is stream-ordered and returns after the
 * host buffer is consumed; d2h synchronises (TensorLike::as_vec / as_bytes,
 * rai-core/src/backend/candle.rs:41-67; FromArray, candle.rs:258-273). */
int rai_hip_h2d(int dev, void *dst_dev, const void *src_host, size_t bytes);
int rai_hip_d2h(int dev, void *dst_host, const void *src_dev, size_t bytes);
int rai_hip_d2d(int dev, void *dst_dev, const void *src_dev, size_t bytes);

/* ToDevice<Hip>: rai-core/src/ops/to_device.rs:48-59, evaluated at backend/candle.rs:776-790.
 * Copies the strided tensor `in`, resident on HIP device src_dev, into the contiguous
 * tensor `out` on HIP device dst_dev (same dtype and shape).  src_dev == dst_dev is a
 * plain strided copy on that device's stream; across devices the source is made
 * contiguous on its own device and moved with a peer copy ordered after the source
 * stream's work.  (Host -> device is rai_hip_h2d into a fresh buffer, device -> host is
 * rai_hip_d2h of a contiguous copy: the two other directions of the reference's op.) */
int rai_hip_to_device(int src_dev, const rai_hip_tensor *in, int dst_dev, const rai_hip_tensor *out);

/* hipEvent timers on the device's stream (measurement only). */
int rai_hip_timer_create(int dev, void **timer);
int rai_hip_timer_start(void *timer);
int rai_hip_timer_stop(void *timer);
int rai_hip_timer_elapsed_ms(void *timer, float *ms); /* blocks on the stop event */
int rai_hip_timer_destroy(void *timer);

/* ----------------------------------------------------- creation primitives */

/* Full<T>: rai-core/src/backend/candle.rs:197-209, ops/full.rs:63-72.
 * `out` must be contiguous. */
int rai_hip_fill(int dev, const rai_hip_tensor *out, double value);

/* Arange<T>: candle.rs:241-256, ops/arange.rs:102-117.  out[i] = start + i*step. */
int rai_hip_arange(int dev, const rai_hip_tensor *out, double start, double step);

/* ------------------------------------------------- elementwise primitives */

/* ToDType<T>: candle.rs:762-774.  Float->bf16/f16 rounds to nearest even;
 * float->integer truncates toward zero (Rust `as`), saturating. */
int rai_hip_cast(int dev, const rai_hip_tensor *in, const rai_hip_tensor *out);

/* Strided copy, same dtype, same shape; `out` may itself be a strided view
 * (used for ToContiguous candle.rs:980-988, Reshape of a non-contiguous view
 * :565-573, Concatenate :880-889 — one call per piece into a narrowed output). */
int rai_hip_copy(int dev, const rai_hip_tensor *in, const rai_hip_tensor *out);

/* Unary primitives and fused activations; `in` may be strided, `out` contiguous. */
int rai_hip_unary(int dev, int op, const rai_hip_tensor *in, const rai_hip_tensor *out, double param);

/* Broadcast binary: operands already expanded to the output shape by stride-0
 * views (rai-core/src/ops/mod.rs:298-340 wraps them in Broadcast nodes).
 * Arithmetic output dtype = operand dtype; comparisons write U8. */
int rai_hip_binary(int dev, int op, const rai_hip_tensor *lhs, const rai_hip_tensor *rhs,
                   const rai_hip_tensor *out);

/* Where: candle.rs:901-915 — out = cond ? on_true : on_false, cond is U8/U32/I64
 * (non-zero = true). */
int rai_hip_where(int dev, const rai_hip_tensor *cond, const rai_hip_tensor *on_true,
                  const rai_hip_tensor *on_false, const rai_hip_tensor *out);

/* ------------------------------------------------------------- reductions */

/* ReduceSum/Max/Min over `ndims` axes of `in` (candle.rs:475-523).  `out` is
 * contiguous with the reduced axes removed (keep_dim=0) or kept as size 1. */
int rai_hip_reduce(int dev, int op, const rai_hip_tensor *in, const int32_t *dims, int32_t ndims,
                   int32_t keep_dim, const rai_hip_tensor *out);

/* Softmax along `dim`: candle.rs:793-826 (max, sub, exp, sum, div) in one pass.
 * Arithmetic in f32 (f64 for F64), result rounded once to the tensor dtype. */
int rai_hip_softmax(int dev, const rai_hip_tensor *in, int32_t dim, const rai_hip_tensor *out);
int rai_hip_log_softmax(int dev, const rai_hip_tensor *in, int32_t dim, const rai_hip_tensor *out);

/* ArgMax/ArgMin along `dim`: candle.rs:917-944, ops/argmax.rs:48-61.  Output U32.
 * The result is that of a sequential scan from element 0 which replaces its running
 * best only on a strict comparison (`>` for argmax, `<` for argmin): the first index
 * wins ties, -0.0 and +0.0 tie, and because every comparison with NaN is false a NaN
 * is never taken over a number while a NaN at element 0 is never replaced (NaN wins
 * from index 0 only; an all-NaN axis yields 0).  That NaN rule restates how candle's
 * CPU loop is believed to behave; nothing in the reference's tests pins it.
 * `out` has `dim` removed or kept as 1.
 * A long axis is cut over several blocks whose partial results and per-row arrival counters live in one fixed
 * array per GPU, shared by rai_hip_argmax, rai_hip_argmin and rai_hip_argmax_static (inputs too large for it use
 * the grown workspace and a second launch).  Like every entry point here the call is enqueued on the library's one
 * stream of the device, so calls are ordered and safe; kernels of these three entry points forced to overlap on
 * one GPU by other means would race on that array. */
int rai_hip_argmax(int dev, const rai_hip_tensor *in, int32_t dim, int32_t keep_dim,
                   const rai_hip_tensor *out);
int rai_hip_argmin(int dev, const rai_hip_tensor *in, int32_t dim, int32_t keep_dim,
                   const rai_hip_tensor *out);

/* rai_hip_argmax for callers that cannot allocate (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the
 * reference.  Same arguments and same result as rai_hip_argmax, but the per-(row, split)
 * partial results of the long-axis kernel live in a fixed array in device memory
 * instead of the grown-on-demand workspace, and the call performs no hipMalloc /
 * hipFree: rai_hip_init(dev) must have succeeded before (otherwise RAI_ERR_HIP).
 * Limit: rows x splits <= 65536 partial results (the axis is only split while that
 * product stays below 512, twice the CU count, so in effect: at most 65536 rows; more
 * returns RAI_ERR_UNSUPPORTED).  All calls on one GPU, of this entry point and of
 * rai_hip_argmax / rai_hip_argmin, share that GPU's array and its arrival counters:
 * kernels of theirs that overlap on one device race; calls on the library's stream are
 * ordered and safe.  The counters are left at zero by every completed launch. */
int rai_hip_argmax_static(int dev, const rai_hip_tensor *in, int32_t dim, int32_t keep_dim,
                          const rai_hip_tensor *out);

/* ---------------------------------------------------------------- indexing */

/* IndexSelect: candle.rs:867-878, ops/index_select.rs:52-61.  index is a rank-1
 * U8/U32/I64 tensor; out.shape[dim] == index length.  An index >= in.shape[dim]
 * makes the call fail with RAI_ERR_INDEX at the next synchronising call and the
 * offending row is zero-filled. */
int rai_hip_index_select(int dev, const rai_hip_tensor *in, const rai_hip_tensor *index, int32_t dim,
                         const rai_hip_tensor *out);
/* Gather: candle.rs:838-849, ops/gather.rs:47-60.  x and index have equal rank and equal extents off `dim`;
 * out has index's shape and x's dtype: out[.., j, ..] = x[.., index[.., j, ..], ..].  Contiguous operands
 * (the reference makes the index contiguous itself, candle.rs:845).  Out-of-range indices as index_select. */
int rai_hip_gather(int dev, const rai_hip_tensor *x, const rai_hip_tensor *index, int32_t dim, const rai_hip_tensor *out);
/* IndexAdd: candle.rs:851-865, ops/index_add.rs:52-62 (the vjp of IndexSelect, ops/index_select.rs:40-48).
 * index is rank 1 (u8/u32/i64), source has x's shape with extent len(index) on `dim`:
 * out = x, then out[.., index[l], ..] += source[.., l, ..] for l = 0, 1, ... in that order, each sum rounded
 * to the dtype.  x, source and out contiguous; out may alias x.  An out-of-range index contributes nothing
 * and makes the next synchronising call fail with RAI_ERR_INDEX. */
int rai_hip_index_add(int dev, const rai_hip_tensor *x, const rai_hip_tensor *index, const rai_hip_tensor *source,
                      int32_t dim, const rai_hip_tensor *out);
/* ScatterAdd: candle.rs:990-1004, ops/scatter_add.rs:52-60 (the vjp of Gather, ops/gather.rs:36-43).
 * index and source share one shape with x's rank and x's extents off `dim`:
 * out = x, then out[.., index[.., j, ..], ..] += source[.., j, ..] for j = 0, 1, ... in that order, each sum
 * rounded to the dtype.  Contiguous operands; out-of-range indices as index_add. */
int rai_hip_scatter_add(int dev, const rai_hip_tensor *x, const rai_hip_tensor *index, const rai_hip_tensor *source,
                        int32_t dim, const rai_hip_tensor *out);
/* Number of out-of-range indices seen by gathers since the last call (syncs). */
int rai_hip_index_errors(int dev, uint64_t *count);

/* ------------------------------------------------------------ contraction */

/* MatMul: candle.rs:327-443, ops/matmul.rs:34-70, shape.rs:130-160.
 * a[..., M, K] x b[..., K, N] -> out[..., M, N]; leading dims already broadcast
 * to out's (stride 0 allowed); any strides accepted for the last two dims.
 * bf16/f16 accumulate in f32 and round once; f32 accumulates in f32. */
int rai_hip_matmul(int dev, const rai_hip_tensor *a, const rai_hip_tensor *b, const rai_hip_tensor *out);

/* ------------------------------------------- fused compositions (rai-nn) */

/* Linear::fwd rai-nn/src/linear.rs:59-69: out[.., n] = act(sum_k x[.., k] w[n, k] + bias[n]) (+ residual).
 * w is [N, K] row-major; bias (nullable) is [N]; act is a rai_hip_unary_op
 * activation or -1; residual (nullable) has out's shape.  x rows must be
 * K-contiguous. */
int rai_hip_linear(int dev, const rai_hip_tensor *x, const rai_hip_tensor *w, const rai_hip_tensor *bias,
                   int32_t act, const rai_hip_tensor *residual, const rai_hip_tensor *out);

/* Several Linear layers that read the same input, evaluated as ONE contraction over
 * their concatenated weight rows -- the form the decoders use for q|k|v|fc1
 * (rai-models/src/llm/phi2.rs:99-101,202-206), for dense|fc2 with the two biases
 * (phi2.rs:293-299) and for the gated MLP act(gate(x)) * up(x) (qwen2.rs:100-104).
 * bf16 only.  x [M,K], w [N,K] (K-contiguous rows), bias / bias2 nullable [N] (both
 * added in f32), act (or -1) applied to columns n >= act_from, residual nullable [M,N].
 *   glu == 0: columns [0, n1) go to out1 [M,n1], columns [n1, N) to out2 [M,N-n1]
 *             (n1 = out1's width; n1 == N: out2 null; a residual needs n1 == N).
 *   glu != 0: w's rows are interleaved gate_0, up_0, gate_1, ...; out1 [M,N/2] gets
 *             act(gate) * up with the reference's roundings of gate, act(gate), up.
 * k_splits: 0 = automatic; > 0 asks the tile kernel (M > 64) for that many K splits. */
int rai_hip_linear_packed(int dev, const rai_hip_tensor *x, const rai_hip_tensor *w, const rai_hip_tensor *bias,
                          const rai_hip_tensor *bias2, int32_t act, int32_t act_from, const rai_hip_tensor *residual,
                          int32_t glu, int32_t k_splits, const rai_hip_tensor *out1, const rai_hip_tensor *out2);

/* LayerNorm::fwd rai-nn/src/layer_norm.rs:32-42 over the last dim (population
 * variance, eps inside the square root); w, b nullable together. */
int rai_hip_layer_norm(int dev, const rai_hip_tensor *x, const rai_hip_tensor *w, const rai_hip_tensor *b,
                       double eps, const rai_hip_tensor *out);

/* RmsNorm::fwd rai-nn/src/rms_norm.rs:18-22 (add_one=0) and Gemma's
 * rai-models/src/llm/gemma.rs:42-54 (add_one=1: x/sqrt(mean(x^2)+eps) * (1+w)). */
int rai_hip_rms_norm(int dev, const rai_hip_tensor *x, const rai_hip_tensor *w, double eps, int32_t add_one,
                     const rai_hip_tensor *out);

/* Rotary embedding, NeoX rotate-half over the first rot_dim of the last dim of
 * x[B, H, S, D] (any strides): rai-models/src/llm/phi2.rs:44-78, qwen2.rs:33-72,
 * gemma.rs:64-103.  cos/sin tables are [max_pos, rot_dim] in x's dtype or F32;
 * rows offset..offset+S are used. */
int rai_hip_rope(int dev, const rai_hip_tensor *x, const rai_hip_tensor *cos, const rai_hip_tensor *sin,
                 int32_t rot_dim, int64_t offset, const rai_hip_tensor *out);
/* Build the tables on device: inv_freq[i] = theta^(-2i/rot_dim) (f32 powf as
 * phi2.rs:48-51 when f64_powf=0; f64 powf then cast as qwen2.rs:45-48 when 1),
 * angle = pos * inv_freq in f32, table[pos][i] = table[pos][i+rot_dim/2]. */
int rai_hip_rope_tables(int dev, double theta, int32_t rot_dim, int32_t f64_powf, const rai_hip_tensor *cos,
                        const rai_hip_tensor *sin);

/* Scaled-dot-product attention over q[B, Hq, S, D], k/v[B, Hkv, T, D] with
 * Hq % Hkv == 0 (repeat_kv gemma.rs:191-201 is implied, never materialised).
 * causal!=0 masks key j > (T - S) + i as phi2.rs:104-117 / gemma.rs:341-362.
 * f32_scores!=0 follows phi2.rs:244-260 (f32 logits and softmax); otherwise
 * scores are rounded to the tensor dtype before softmax as qwen2.rs:205-216.
 * out is [B, S, Hq*D] contiguous (the transpose(1,2)+reshape of phi2.rs:261-262). */
int rai_hip_attention(int dev, const rai_hip_tensor *q, const rai_hip_tensor *k, const rai_hip_tensor *v,
                      double scale, int32_t causal, int32_t f32_scores, const rai_hip_tensor *out);

/* ------------------------------------------- decoder-only model drivers */

typedef enum rai_hip_arch {
  RAI_ARCH_PHI2 = 0,  /* rai-models/src/llm/phi2.rs */
  RAI_ARCH_QWEN2 = 1, /* rai-models/src/llm/qwen2.rs */
  RAI_ARCH_GEMMA = 2, /* rai-models/src/llm/gemma.rs */
  RAI_ARCH_PHI3 = 3   /* rai-models/src/llm/phi3.rs: the Qwen2 block with fused qkv_proj / gate_up_proj, no biases */
} rai_hip_arch;

/* Union of the serde Config structs phi2.rs:9-24, qwen2.rs:8-24, gemma.rs:12-27. */
typedef struct rai_hip_decoder_config {
  int32_t arch;
  int32_t dtype; /* RAI_BF16 or RAI_F32 */
  int32_t vocab_size;
  int32_t hidden_size;
  int32_t intermediate_size;
  int32_t num_hidden_layers;
  int32_t num_attention_heads;
  int32_t num_key_value_heads;
  int32_t head_dim;
  int32_t rotary_dim; /* phi2: partial_rotary_factor*head_dim; others: head_dim */
  int32_t max_position_embeddings;
  int32_t hidden_act; /* RAI_UN_NEW_GELU / RAI_UN_GELU / RAI_UN_SILU */
  int32_t tie_word_embeddings;
  int32_t max_batch;   /* KV cache is preallocated for max_batch x max_context */
  int32_t max_context;
  /* 0: rotary tables computed in the model dtype exactly as the reference does
   * (phi2.rs:53-57: positions and pos*inv_freq rounded to bf16 for a bf16
   * model); 1: angles computed in f32 and rounded once. */
  int32_t rope_tables_f32;
  /* Phi-2's optional LayerNorm of the query / key projections (phi2.rs:207-216).  The reference applies a
   * LayerNorm over head_dim elements to the un-split [.., heads * head_dim] projection, a graph that is only
   * well-formed for a single head; the drivers do not implement it: non-zero -> RAI_ERR_UNSUPPORTED.  (The lazy-graph
   * evaluator of rai_graph.h runs such a model node by node, Err node included, as the reference would.) */
  int32_t qk_layernorm;
  double rope_theta;
  double norm_eps;
} rai_hip_decoder_config;

typedef struct rai_hip_decoder rai_hip_decoder;

/* Model::new (phi2.rs:316-332): allocates weights (uninitialised), KV cache and
 * activation arena once; no allocation happens in forward afterwards. */
int rai_hip_decoder_create(int dev, const rai_hip_decoder_config *cfg, rai_hip_decoder **out);
int rai_hip_decoder_destroy(rai_hip_decoder *dec);
/* Module::update_by_safetensors naming (rai-core/src/nn.rs:183-205, renames
 * phi2.rs:307-313): copy one named parameter from host memory, e.g.
 * "model.layers.3.self_attn.q_proj.weight".  `data` is row-major in the model dtype. */
int rai_hip_decoder_load_param(rai_hip_decoder *dec, const char *name, const void *host_data, size_t bytes);
/* Module::update_by_safetensors (rai-core/src/nn.rs:39-55): reads every file, collects its tensors by
 * name (a later file wins on a duplicate), then looks every parameter of the model up by name, converts
 * it to the model dtype (nn.rs:198-201) and stores it.  A parameter that no file holds fails with
 * RAI_ERR_PARAM_NOT_FOUND naming it; tensors the model does not have are ignored.  Source dtypes F32,
 * F16, BF16 and F64 (the floating ones of hlops/from_safetensor.rs:51-91); anything else is
 * RAI_ERR_BAD_DTYPE, a malformed file RAI_ERR_IO. */
int rai_hip_decoder_load_safetensors(rai_hip_decoder *dec, const char *const *paths, int32_t n_paths);
/* ext::hf::load_safetensors (rai/src/lib.rs:17-42) without the hub download: the distinct shard files
 * named by the "weight_map" of a model.safetensors.index.json, resolved against the directory of the
 * index file and written to buf separated by '\n'.  A missing or non-object weight_map is RAI_ERR_IO. */
int rai_hip_safetensors_index_files(const char *index_json_path, char *buf, size_t buflen, int32_t *n_files);
/* Dtype of the decoder's parameters (RAI_F32 or RAI_BF16). */
int rai_hip_decoder_dtype(rai_hip_decoder *dec, int32_t *dtype);
/* Number of parameter names the architecture expects / i-th name (for loaders). */
int rai_hip_decoder_param_count(rai_hip_decoder *dec, int32_t *count);
int rai_hip_decoder_param_name(rai_hip_decoder *dec, int32_t i, char *buf, size_t buflen, int64_t *numel);
/* The logical shape of parameter i: a matrix [rows, cols] as the reference's module holds it (Linear: [out, in]),
 * a vector as rows == 1.  The safetensors loader requires the file's tensor to have exactly this shape. */
int rai_hip_decoder_param_shape(rai_hip_decoder *dec, int32_t i, int64_t *rows, int64_t *cols);
/* Model::fwd (phi2.rs:334-347): ids_host[batch*seq] u32 are appended after the
 * cached context; returns last-position logits [batch, vocab] as f32 in
 * logits_host (nullable) and greedy tokens (device argmax, first-max) in
 * tokens_host (nullable).  Synchronises only if an output pointer is given.
 * A single-token step (batch 1, seq 1) of a Phi-2-architecture model in bf16 whose hidden width is 2560 = 32 heads
 * x 80 (Phi-2) or 2048 = 32 heads x 64 (Phi-1 / Phi-1.5), with or without grouped-query attention, intermediate and
 * q|k|v widths multiples of 512, runs all layers as one launch of a persistent kernel; every other model, width,
 * batch or dtype takes one launch per primitive. */
int rai_hip_decoder_forward(rai_hip_decoder *dec, const uint32_t *ids_host, int32_t batch, int32_t seq,
                            float *logits_host, uint32_t *tokens_host);
/* Model::fwd (phi2.rs:334-347, qwen2.rs:338-359, gemma.rs:364-386) with both ends of the layer stack open.
 * Input: either ids_host[batch*seq] (as rai_hip_decoder_forward) or hidden_in_host, [batch*seq, hidden] rows in
 * the model dtype's storage form that take the place of the embedding lookup (for Gemma: of the already scaled
 * embeddings, gemma.rs:379); exactly one of the two is non-null.  hidden_out_host (nullable) receives the residual
 * stream after the last layer, before the final norm, as f32 [batch*seq, hidden]: with a one-layer model that is
 * what DecoderLayer::fwd returns (phi2.rs:293-299, qwen2.rs:253-266, gemma.rs:286-299).  logits_host and
 * tokens_host as in rai_hip_decoder_forward.  Always takes the launch-per-primitive path. */
int rai_hip_decoder_forward_hidden(rai_hip_decoder *dec, const uint32_t *ids_host, const void *hidden_in_host,
                                   int32_t batch, int32_t seq, float *hidden_out_host, float *logits_host,
                                   uint32_t *tokens_host);
/* Greedy loop of examples/phi2/src/main.rs:75-95 without repeat penalty: prefill
 * prompt[batch*prompt_len], then n_new single-token steps feeding the device
 * argmax back without host round trips.  tokens_host[batch*n_new]. prefill_ms /
 * decode_ms (nullable) are hipEvent times of the two phases. */
int rai_hip_decoder_generate(rai_hip_decoder *dec, const uint32_t *prompt_host, int32_t batch, int32_t prompt_len,
                             int32_t n_new, uint32_t *tokens_host, float *prefill_ms, float *decode_ms);
/* The whole loop of examples/phi2/src/main.rs:72-95 on the device: as rai_hip_decoder_generate, but each
 * token is chosen as the example does: the logits row as f32, apply_repeat_penalty (main.rs:39-50) over the
 * distinct ids among the last repeat_last_n tokens of the sequence so far (prompt included; a logit >= 0 is
 * divided by the penalty, any other multiplied; skipped when repeat_penalty < 1, main.rs:79), then
 * sample_argmax (main.rs:29-37): the maximum under f32 total order, the LAST one on ties.  The example uses
 * penalty 1.10 over 64 tokens.  The device loop always runs n_new steps; n_generated[batch] (nullable)
 * receives for each row the count the example's loop would have stopped at (it stops after pushing
 * eos_token, main.rs:83-86; pass a negative eos_token for "none"). */
int rai_hip_decoder_generate_sampled(rai_hip_decoder *dec, const uint32_t *prompt_host, int32_t batch,
                                     int32_t prompt_len, int32_t n_new, float repeat_penalty, int32_t repeat_last_n,
                                     int64_t eos_token, uint32_t *tokens_host, int32_t *n_generated, float *prefill_ms,
                                     float *decode_ms);
/* apply_repeat_penalty + sample_argmax (examples/phi2/src/main.rs:29-50) as a primitive: logits [rows, vocab]
 * f32 or bf16, context [rows, n] u32 (null: no penalty), out [rows] u32.  Context ids outside the vocabulary
 * are ignored, as the reference's set lookup ignores them. */
int rai_hip_sample_argmax(int dev, const rai_hip_tensor *logits, const rai_hip_tensor *context, float repeat_penalty,
                          const rai_hip_tensor *out);
/* Model::clear_kv_cache (phi2.rs:349-353). */
int rai_hip_decoder_clear_kv_cache(rai_hip_decoder *dec);
/* Current cached context length. */
int rai_hip_decoder_context_len(rai_hip_decoder *dec, int32_t *len);

/* Measurement aid: mean duration (hipEvents on the library's stream, one pair per launch) of the
 * persistent per-token kernel that runs all layers of a single-token step (Phi-2 architecture, bf16,
 * batch 1), launched `sweeps` times at the current context length, and the algorithmic bytes one launch
 * moves (weights, biases, norm parameters, cached K/V).  The residual stream and the cache row at the
 * current position are overwritten: clear the KV cache before the decoder is used again.
 * No counterpart in the reference (it has no kernels of its own). */
int rai_hip_decoder_time_decode_step(rai_hip_decoder *dec, int32_t sweeps, float *us_per_launch,
                                     double *bytes_per_launch);
/* Measurement only (no counterpart in the reference): launches the decode-step
 * weight-streaming kernel back to back over every layer's two packed matrices
 * (q|k|v|fc1 with the fused LayerNorm, then dense|fc2 with the residual; 2*L
 * launches per sweep) between two hipEvents on the device's stream.  Reports the
 * mean time of one launch in microseconds and the algorithmic bytes one launch
 * moves on average (weights + biases + activation vectors in and out). */
int rai_hip_decoder_time_decode_linear(rai_hip_decoder *dec, int32_t sweeps, float *us_per_launch,
                                       double *bytes_per_launch);

#ifdef __cplusplus
}
#endif
#endif /* RAI_HIP_H */
