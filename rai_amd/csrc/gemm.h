// Internal launchers of the contraction kernels, shared by the C-ABI matmul /
// linear entry points and by the decoder drivers.
#pragma once
#include "common.h"

namespace rai {

// out[m, n] = epilogue( sum_k A[m, k] * W[n, k] )     (the layout Linear produces,
// rai-nn/src/linear.rs:59-69: x @ W^T with W stored [out_features, in_features])
//
// Epilogue per column n:  v = acc + bias[n] + bias2[n];  v = act(v) for n >= act_from;
// v += residual[m, n];  round to bf16.  Columns [0, n_split) go to out1, columns
// [n_split, N) go to out2 at column n - n_split (n_split == N: single output).
struct LinearArgs {
  const void *A;       // [M, K], K-contiguous rows
  int64_t lda;
  const void *W;       // [N, K]
  int64_t ldw;
  const void *bias;    // [N] or null
  const void *bias2;   // second [N] bias added in f32 (sum of two Linear biases), or null
  const void *residual;  // [M, N] or null
  int64_t ldr;
  void *out1;
  int64_t ld1;
  void *out2;
  int64_t ld2;
  int M, N, K;
  int n_split;   // first column written to out2
  int act;       // rai_hip_unary_op activation or -1
  int act_from;  // activation applies to columns >= act_from
  // Gated MLP (rai-models/src/llm/qwen2.rs:100-104: act(gate(x)) * up(x)): W rows are
  // interleaved gate_0, up_0, gate_1, up_1, ...; N counts the interleaved rows and
  // N/2 columns are written to out1.  No residual, no output split.
  int glu;
  // Optional fused LayerNorm / RMSNorm of the rows of A before the product
  // (skinny path only): A is normalised with ln_w / ln_b over K.
  const void *ln_w;
  const void *ln_b;
  float ln_eps;
  int ln_kind;  // -1 none, 0 layernorm, 1 rmsnorm, 2 rmsnorm(1+w)
  // Optional f32 scratch for splitting K over several blocks when M x N alone
  // yields too few tiles to fill the GPU (tile kernel only).
  void *splitk_ws;
  size_t splitk_ws_bytes;
  // > 0: the tile kernel cuts K into this many splits (when the workspace holds them) instead of asking its cost
  // model; 0: automatic.
  int force_splits;
  // Optional second copy of W in MFMA-fragment order for the small-M streaming kernel (9 <= M <= 64): the
  // 16 rows x 32 columns that one wave loads with one instruction are 1 KB of consecutive memory
  // ([N / 16 row tiles][K / 32 steps][64 lanes][8 elements], see linear_fragment_layout); null: read W itself.
  const void *Wfrag;
  // Optional LayerNorm of the finished output rows, written to post_ln_out ([M, N], dense) next to out1: the pass
  // that sums the split-K partial products has the whole row at hand, so the norm that consumes the output (the next
  // block's input LayerNorm) costs no launch of its own.  Only that pass offers it: ask linear_fuses_post_norm()
  // first and run the norm separately when it says no.
  void *post_ln_out;
  const void *post_ln_w;
  const void *post_ln_b;
  float post_ln_eps;
  // Device the operands live on (its CU count and per-device counters are looked up by it); -1: the current device.
  int dev;
  // Optional second product added to the first before the epilogue (M == 1, skinny kernel only): the row A2 [K2]
  // against W2 [N, K2], as if A and A2, W and W2 were concatenated along K.  The sum of two Linears of a decoder
  // block (rai-models/src/llm/phi2.rs:298) in one launch; their biases go to bias and bias2.
  const void *A2;
  const void *W2;
  int64_t ldw2;
  int K2;
};
// True when launch_linear_bf16 with these arguments will also write post_ln_out.
bool linear_fuses_post_norm(const LinearArgs &a);
// Workspace (LinearArgs::splitk_ws) the stream-K form of the bf16 tile kernel needs for an M x N x K Linear; 0 when
// that form does not apply to the shape.  At most 192 MB.
size_t linear_streamk_workspace_bytes(int M, int N, int K);
inline LinearArgs linear_args_default() {
  LinearArgs a;
  memset(&a, 0, sizeof(a));
  a.act = -1;
  a.ln_kind = -1;
  a.dev = -1;
  return a;
}

// Elements of the fragment-major copy of a [N, K] bf16 matrix (K % 32 == 0; N is padded to a multiple of 16 with
// zero rows), and the kernel that writes it.
size_t linear_fragment_elems(int N, int K);
int launch_linear_fragment_layout(hipStream_t st, const void *W, int64_t ldw, int N, int K, void *Wfrag);

// bf16 MFMA tile kernel (M >= 1; efficient for M >= 64).
int launch_linear_bf16_mfma(hipStream_t st, const LinearArgs &a);
// bf16 weight-streaming kernel for M <= 8 (decode): HBM-bound.
int launch_linear_bf16_skinny(hipStream_t st, const LinearArgs &a);
// Picks between the two.
int launch_linear_bf16(hipStream_t st, const LinearArgs &a);

// Up to kGemvGroupMax bf16 Linears of one activation row (M == 1, K <= 4096, a multiple of 8) in one launch: member i
// is out[i][n] = act[i](sum_k norm(x)[k] * W[i][n, k] + bias[i][n]), n < N[i]; the optional norm (ln_kind as in
// LinearArgs) is applied to x once per wave, as the single-Linear kernel does.  wave_base is filled by the launcher.
constexpr int kGemvGroupMax = 4;
struct GemvGroupArgs {
  const void *x;
  int K, count;
  const void *W[kGemvGroupMax];
  int64_t ldw[kGemvGroupMax];
  const void *bias[kGemvGroupMax];   // null: none
  void *out[kGemvGroupMax];
  int N[kGemvGroupMax];
  int act[kGemvGroupMax];            // rai_hip_unary_op or -1
  const void *ln_w, *ln_b;
  float ln_eps;
  int ln_kind;
  int wave_base[kGemvGroupMax + 1];
};
bool gemv_group_serves(int K, int count);
// out[n] = x1 . W1[n] + x2 . W2[n] + bias1[n] + bias2[n] + residual[n] for one bf16 row pair (the LinearArgs::A2 form);
// RAI_ERR_UNSUPPORTED when the widths are not served.
int launch_linear_dual_row(hipStream_t st, int dev, const void *x1, int K1, const void *W1, int64_t ldw1, const void *bias1, const void *x2, int K2,
                           const void *W2, int64_t ldw2, const void *bias2, const void *residual, void *out, int N);
int launch_gemv_group(hipStream_t st, GemvGroupArgs g);

// f32 tile kernel for the same NT contraction, FMA in f32.
int launch_linear_f32(hipStream_t st, const LinearArgs &a);
bool linear_mfma_fuses_norm(int M, int K, int ln_kind);

__device__ __forceinline__ float act_eval(int act, float x);
// act(gate) * up with the reference's roundings of gate, act(gate) and up to bf16.
__device__ __forceinline__ float glu_bf16(int act, float g, float u) {
  const float gr = bf16_bits_to_f32(f32_to_bf16_bits(g));
  const float ar = bf16_bits_to_f32(f32_to_bf16_bits(act_eval(act, gr)));
  return ar * bf16_bits_to_f32(f32_to_bf16_bits(u));
}

__device__ __forceinline__ float act_eval(int act, float x) {
  switch (act) {
    case RAI_UN_GELU: return x * 0.5f * (1.0f + erff(x / 1.4142135623730951f));
    case RAI_UN_NEW_GELU: return 0.5f * x * (1.0f + tanhf(0.7978845608028654f * (x + 0.044715f * x * x * x)));
    case RAI_UN_SILU: return x / (expf(-x) + 1.0f);
    case RAI_UN_RELU: return x > 0.f ? x : 0.f;
    case RAI_UN_TANH: return tanhf(x);
    default: return x;
  }
}

}  // namespace rai
