// Decoder-only model drivers: the fused, allocation-free evaluation of
// rai-models/src/llm/phi2.rs (Model::fwd :334-347, DecoderLayer::fwd :293-299,
// Attention::fwd :202-264, MLP::fwd :99-101) and the greedy loop of
// examples/phi2/src/main.rs:75-95.
//
// Layout in HBM (per layer, built once at load time so decode streams each
// weight byte exactly once with unit stride):
//   Wa [QD + 2*KD + I, H]  rows = q_proj | k_proj | v_proj | fc1   (all read the same LayerNorm output)
//   Wb [H, QD + I]         row n = dense[n, :] | fc2[n, :]         (attn output and MLP activation are
//                                                                   adjacent columns of one buffer)
//   KV cache K, V [L][B][Hkv][Tmax][D], preallocated; appending a token writes one row.
// Per layer a prefill runs LayerNorm, one GEMM over Wa (bias + gelu on the fc1
// columns), rotary + cache append, attention, one GEMM over Wb (both biases +
// residual).  A decode step fuses the LayerNorm into the weight-streaming
// kernel: 3 launches per layer.  Context length and the current tokens live in
// device memory, so consecutive greedy steps need no host round trip.
#include <algorithm>
#include <cstdlib>
#include <map>
#include <string>
#include <vector>

#include "attention.h"
#include "decode_chain.h"
#include "decode_mega.h"
#include "gemm.h"

namespace rai {

struct ParamSlot {
  std::string name;
  int64_t rows, cols;       // logical [rows, cols] (1-D params: rows = 1)
  char *dst;                // device address of element [0, 0]
  int64_t pitch;            // elements between consecutive rows at dst
  bool loaded;
  // a parameter whose last rows2 rows go elsewhere (same pitch): Phi-3's gate_up_proj, whose gate rows and
  // up rows interleave in the packed matrix
  int64_t rows2;
  char *dst2;
};

struct Layer {
  // Phi-2 (parallel block)
  char *Wa, *ba, *Wb, *bd, *bf, *ln_w, *ln_b;
  // Qwen2 / Gemma (sequential block): Wqkv [QD+2KD, H] (+bqkv), Wo [H, QD] (+bo),
  // Wgu [2I, H] with gate/up rows interleaved, Wdown [H, I], two RMSNorm weights
  char *Wqkv, *bqkv, *Wo, *bo, *Wgu, *Wdown, *n1_w, *n2_w;
  // second copies in MFMA-fragment order for the batched-decode streaming kernel (built on first use)
  char *Wa_f, *Wb_f, *Wqkv_f, *Wo_f, *Wgu_f, *Wdown_f;
};

}  // namespace rai

using namespace rai;

struct rai_hip_decoder {
  int dev;
  rai_hip_decoder_config cfg;
  size_t es;
  int H, I, QD, KD, D, Hq, Hkv, V, L, NA, KB;
  std::vector<ParamSlot> slots;
  std::map<std::string, int> slot_by_name;
  std::vector<Layer> layers;
  char *embed, *lnf_w, *lnf_b, *head_w, *head_b;
  char *cos_t, *sin_t;  // [max_pos, rot] in the model dtype
  char *kcache, *vcache;
  // activations (sized for max_batch * max_context rows)
  char *x, *x2, *ln, *qkv, *cat, *last, *logits;
  char *attn, *glu;   // sequential block: attention output [rows, QD], gated MLP activation [rows, I]
  char *attn_ws;      // partial results of the decode attention's context splits
  int *attn_counters; // per (batch, head) arrival counters of those splits (zero between launches)
  float embed_scale;  // Gemma: sqrt(hidden) rounded to the model dtype; 1 otherwise
  uint32_t *ids, *tokens, *history;
  char *splitk_ws;        // f32 scratch for prefill GEMMs that split K
  size_t splitk_ws_bytes;
  DevState *state;
  std::vector<void *> allocs;
  int ctx_len;
  int64_t max_rows;
  int history_cap;
  // persistent per-token kernel (Phi-2, bf16, batch 1): per-layer pointer table, exchange packets
  MegaLayer *mega_layers;
  uint64_t *mega_xchg;    // packets exchanged between the blocks of the persistent decode kernel
  unsigned long long *mega_prof;  // time stamps of the persistent kernel when RAI_HIP_MEGA_PROF is set
  bool mega_ok;
  int num_cu;
  hipGraphExec_t step_graph;   // one captured single-token step (batch step_graph_batch)
  hipGraphExec_t step_graph_n; // kGraphSteps consecutive single-token steps in one graph (same batch)
  int step_graph_batch;
  bool x_holds_next;          // d->x already holds the embedding of d->tokens
  // token choice of the example loop (repeat penalty, last maximum wins) instead of plain greedy argmax
  bool sample_on;
  float sample_penalty;
  int sample_last_n;
  uint32_t *token_log;        // [max_batch][token_log_cap]: every token of each sequence so far, prompt first
  int token_log_cap;
  float *choice_val;          // [max_batch][kChoiceMaxSplits]: best value of each share of a wide logits row
  uint32_t *choice_idx;       // and its index
  unsigned long long *head_best;   // one (value, row) word per block of the head kernel that also chooses the token
  char *hidden_copy;          // [max_rows, H]: the residual stream after the last layer, kept when a caller asks for it
  bool want_hidden;           // the running forward copies its final residual stream to hidden_copy
  char *head_f;               // fragment-order copy of the lm_head matrix
  bool frag_ready;            // the fragment-order copies match the loaded parameters
  bool graph_sampled;         // what the cached step graphs were captured with
  float graph_penalty;
  int graph_last_n;
};

namespace rai {

constexpr int kChoiceMaxSplits = 64;  // shares a logits row is scanned in before the token choice
constexpr int kGraphSteps = 8;  // single-token steps recorded in the multi-step decode graph

// ------------------------------------------------------------------ small kernels
template <typename T>
__global__ void __launch_bounds__(256)
k_embed(T *out, const T *table, const uint32_t *ids, int64_t rows, int H, int vocab, unsigned long long *errors,
        float scale) {
  for (int64_t e = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; e < rows * H; e += (int64_t)gridDim.x * blockDim.x) {
    int64_t r = e / H;
    int c = (int)(e - r * H);
    uint32_t id = ids[r];
    if (id >= (uint32_t)vocab) {
      if (c == 0) atomicAdd(errors, 1ull);
      memset(&out[e], 0, sizeof(T));
    } else if (scale != 1.0f) {  // Gemma: xs * sqrt(hidden), the scalar rounded to the model dtype (gemma.rs:379)
      Scalar<T>::store(out + e, (typename Scalar<T>::compute)((float)Scalar<T>::load(table + (int64_t)id * H + c) * scale));
    } else {
      out[e] = table[(int64_t)id * H + c];
    }
  }
}

// Rotary embedding (NeoX rotate-half over the first `rot` features) applied in
// place to q, and to k while it is appended to the cache together with v.
// qkv rows are [q (QD) | k (KD) | v (KD)] per token.
template <typename T>
__global__ void __launch_bounds__(256)
k_rope_append(T *qkv, T *kcache, T *vcache, const T *cos_t, const T *sin_t, const DevState *state, int B, int S, int Hq,
              int Hkv, int D, int rot, int Tmax) {
  const int pos0 = state->pos;
  const int QD = Hq * D, KD = Hkv * D, ld = QD + 2 * KD;
  const int half = rot / 2;
  const int heads = Hq + 2 * Hkv;
  const int64_t total = (int64_t)B * S * heads * D;
  for (int64_t e = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; e < total; e += (int64_t)gridDim.x * blockDim.x) {
    int d = (int)(e % D);
    int64_t r = e / D;
    int hh = (int)(r % heads);
    r /= heads;
    int s = (int)(r % S);
    int b = (int)(r / S);
    T *row = qkv + ((int64_t)b * S + s) * ld;
    const int pos = pos0 + s;
    if (hh < Hq + Hkv) {  // q or k head: rotate
      T *hp = row + (hh < Hq ? hh * D : QD + (hh - Hq) * D);
      float v = (float)Scalar<T>::load(hp + d);
      // pair (d, d+half): the lane with d < half computes both to keep the update in place
      if (d < half) {
        float v2 = (float)Scalar<T>::load(hp + d + half);
        float c1 = (float)Scalar<T>::load(cos_t + (int64_t)pos * rot + d);
        float s1 = (float)Scalar<T>::load(sin_t + (int64_t)pos * rot + d);
        float c2 = (float)Scalar<T>::load(cos_t + (int64_t)pos * rot + d + half);
        float s2 = (float)Scalar<T>::load(sin_t + (int64_t)pos * rot + d + half);
        // reference rounds x*cos, rot*sin and their sum separately (phi2.rs:75)
        T a, bb, o1, o2;
        Scalar<T>::store(&a, v * c1);
        Scalar<T>::store(&bb, -v2 * s1);
        Scalar<T>::store(&o1, (float)Scalar<T>::load(&a) + (float)Scalar<T>::load(&bb));
        Scalar<T>::store(&a, v2 * c2);
        Scalar<T>::store(&bb, v * s2);
        Scalar<T>::store(&o2, (float)Scalar<T>::load(&a) + (float)Scalar<T>::load(&bb));
        if (hh < Hq) {
          hp[d] = o1;
          hp[d + half] = o2;
        } else {
          T *kc = kcache + (((int64_t)b * Hkv + (hh - Hq)) * Tmax + pos) * D;
          kc[d] = o1;
          kc[d + half] = o2;
        }
      } else if (d >= rot && hh >= Hq) {
        kcache[(((int64_t)b * Hkv + (hh - Hq)) * Tmax + pos) * D + d] = hp[d];
      }
    } else {
      int hv = hh - Hq - Hkv;
      vcache[(((int64_t)b * Hkv + hv) * Tmax + pos) * D + d] = row[QD + KD + hv * D + d];
    }
  }
}

// The same operation with one thread per 16-byte pack and 32-bit indexing (D, rot/2 and the row
// length multiples of the pack width; fewer than 2^31 packs).  The pack at feature d0 < rot/2 and
// its partner at d0 + rot/2 are rotated by one thread, so the update of q stays in place.
template <typename T>
__global__ void __launch_bounds__(256)
k_rope_append_vec(T *qkv, T *kcache, T *vcache, const T *cos_t, const T *sin_t, const DevState *state, int B, int S,
                  int Hq, int Hkv, int D, int rot, int Tmax) {
  constexpr int VEC = 16 / sizeof(T);
  struct alignas(16) Pack { T v[VEC]; };
  const int pos0 = state->pos;
  const int QD = Hq * D, KD = Hkv * D, ld = QD + 2 * KD;
  const int half = rot / 2;
  const uint32_t heads = Hq + 2 * Hkv, ppr = D / VEC;        // packs per head row
  const uint32_t total = (uint32_t)B * S * heads * ppr;
  for (uint32_t e = blockIdx.x * blockDim.x + threadIdx.x; e < total; e += gridDim.x * blockDim.x) {
    const uint32_t r = e / ppr, d0 = (e - r * ppr) * VEC;
    const uint32_t hh = r % heads, r2 = r / heads, s = r2 % S, b = r2 / S;
    T *row = qkv + ((int64_t)b * S + s) * ld;
    const int pos = pos0 + (int)s;
    if (hh < (uint32_t)(Hq + Hkv)) {  // q or k head
      T *hp = row + (hh < (uint32_t)Hq ? hh * D : QD + (hh - Hq) * D);
      T *kc = hh < (uint32_t)Hq ? nullptr : kcache + (((int64_t)b * Hkv + (hh - Hq)) * Tmax + pos) * D;
      if ((int)d0 < half) {
        const Pack x1 = *reinterpret_cast<const Pack *>(hp + d0), x2 = *reinterpret_cast<const Pack *>(hp + d0 + half);
        const T *ct = cos_t + (int64_t)pos * rot + d0, *st = sin_t + (int64_t)pos * rot + d0;
        const Pack c1 = *reinterpret_cast<const Pack *>(ct), s1 = *reinterpret_cast<const Pack *>(st);
        const Pack c2 = *reinterpret_cast<const Pack *>(ct + half), s2 = *reinterpret_cast<const Pack *>(st + half);
        Pack o1, o2;
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const float v = (float)Scalar<T>::load(&x1.v[j]), v2 = (float)Scalar<T>::load(&x2.v[j]);
          // the reference rounds x*cos, rot*sin and their sum separately (phi2.rs:75)
          T a, bb;
          Scalar<T>::store(&a, v * (float)Scalar<T>::load(&c1.v[j]));
          Scalar<T>::store(&bb, -v2 * (float)Scalar<T>::load(&s1.v[j]));
          Scalar<T>::store(&o1.v[j], (float)Scalar<T>::load(&a) + (float)Scalar<T>::load(&bb));
          Scalar<T>::store(&a, v2 * (float)Scalar<T>::load(&c2.v[j]));
          Scalar<T>::store(&bb, v * (float)Scalar<T>::load(&s2.v[j]));
          Scalar<T>::store(&o2.v[j], (float)Scalar<T>::load(&a) + (float)Scalar<T>::load(&bb));
        }
        T *dst = kc ? kc : hp;
        *reinterpret_cast<Pack *>(dst + d0) = o1;
        *reinterpret_cast<Pack *>(dst + d0 + half) = o2;
      } else if ((int)d0 >= rot && kc) {
        *reinterpret_cast<Pack *>(kc + d0) = *reinterpret_cast<const Pack *>(hp + d0);
      }
    } else {
      const uint32_t hv = hh - Hq - Hkv;
      *reinterpret_cast<Pack *>(vcache + (((int64_t)b * Hkv + hv) * Tmax + pos) * D + d0) =
          *reinterpret_cast<const Pack *>(row + QD + KD + hv * D + d0);
    }
  }
}

// Between two launches of the persistent decode kernel that no token selection separates.
__global__ void k_next_epoch(DevState *st) { st->epoch += 1u; }

__global__ void k_set_state(DevState *st, int pos, int step) {
  st->pos = pos;
  st->step = step;
  st->done = 0;
}

// Tail of the token-selection kernels (every thread of the block calls it with the block's chosen token):
// the token's embedding row becomes the next step's input x[b], and the last block to finish advances the
// device-side context length / step counters and the exchange epoch of the persistent decode kernel.
template <typename T>
__device__ __forceinline__ void publish_token(uint32_t chosen, int b, DevState *state, int B, int dpos, int dstep,
                                              const T *embed, T *x_next, int H, float embed_scale) {
  if (x_next) {
    const T *row = embed + (int64_t)chosen * H;
    for (int c = threadIdx.x; c < H; c += blockDim.x) {
      if (embed_scale != 1.0f)
        Scalar<T>::store(x_next + (int64_t)b * H + c, (typename Scalar<T>::compute)((float)Scalar<T>::load(row + c) * embed_scale));
      else
        x_next[(int64_t)b * H + c] = row[c];
    }
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    // no fence: `step` was read (and used for an address) before this point, and what this block wrote is
    // consumed by later kernels only
    int prev = atomicAdd(&state->done, 1);
    if (prev == B - 1) {  // every block has read `step` and written its outputs
      state->epoch += 1u;   // the next launch of the decode kernel tags its packets differently
      state->done = 0;
      state->pos += dpos;
      state->step += dstep;
    }
  }
}

// Greedy token selection for every sequence, one 1024-thread block per row of
// logits: argmax (first maximum wins; NaN never wins except at index 0), the
// token goes to tokens[b] and to history[step][b], the token's embedding row
// becomes the next step's input x[b], and the last block to finish advances the
// device-side context length / step counters.  Everything the next
// single-token step needs is then on the device.
template <typename T>
__global__ void __launch_bounds__(1024)
k_select_token(const T *logits, int64_t n, uint32_t *tokens, uint32_t *history, DevState *state, int B, int dpos,
               int dstep, const T *embed, T *x_next, int H, float embed_scale, const float *pval, const uint32_t *pidx,
               int splits) {
  __shared__ float sv[16];
  __shared__ uint32_t si[16];
  __shared__ uint32_t chosen;
  const int b = blockIdx.x;
  const int step = state->step;
  const T *x = logits + (int64_t)b * n;
  float bv = -INFINITY;
  uint32_t bi = 0xffffffffu;
  constexpr int VEC = 16 / sizeof(T);
  if (splits > 0) {
    // wide rows: launch_argmax_partials has scanned the row in `splits` shares spread over the GPU; what is left is
    // the choice among their (value, index) pairs (a share of NaNs only offers nothing)
    for (int sp = threadIdx.x; sp < splits; sp += blockDim.x) {
      const float v = pval[(int64_t)b * splits + sp];
      const uint32_t i = pidx[(int64_t)b * splits + sp];
      if (v == v && (bi == 0xffffffffu || v > bv || (v == bv && i < bi))) { bv = v; bi = i; }
    }
  } else if (n % VEC == 0 && ((uintptr_t)x & 15) == 0) {
    // 16-byte loads, four per thread in flight; every thread still visits its elements in
    // increasing index order, so the first maximum wins exactly as in the scalar scan
    struct alignas(16) Pack { T v[VEC]; };
    const Pack *xp = reinterpret_cast<const Pack *>(x);
    const int64_t chunks = n / VEC;
    for (int64_t c0 = threadIdx.x; c0 < chunks; c0 += (int64_t)blockDim.x * 4) {
      Pack pk[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t c = c0 + (int64_t)u * blockDim.x;
        if (c < chunks) pk[u] = xp[c];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t c = c0 + (int64_t)u * blockDim.x;
        if (c < chunks) {
#pragma unroll
          for (int j = 0; j < VEC; ++j) {
            const float v = (float)Scalar<T>::load(&pk[u].v[j]);
            if (v > bv || (bi == 0xffffffffu && v == v)) { bv = v; bi = (uint32_t)(c * VEC + j); }
          }
        }
      }
    }
  } else {
    for (int64_t i = threadIdx.x; i < n; i += blockDim.x) {
      float v = (float)Scalar<T>::load(x + i);
      if (v > bv || (bi == 0xffffffffu && v == v)) { bv = v; bi = (uint32_t)i; }
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    float ov = __shfl_xor(bv, o, 64);
    uint32_t oi = (uint32_t)__shfl_xor((int)bi, o, 64);
    if (oi != 0xffffffffu && (bi == 0xffffffffu || ov > bv || (ov == bv && oi < bi))) { bv = ov; bi = oi; }
  }
  if ((threadIdx.x & 63) == 0) { sv[threadIdx.x >> 6] = bv; si[threadIdx.x >> 6] = bi; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < (int)(blockDim.x >> 6); ++w) {
      float ov = sv[w];
      uint32_t oi = si[w];
      if (oi != 0xffffffffu && (bi == 0xffffffffu || ov > bv || (ov == bv && oi < bi))) { bv = ov; bi = oi; }
    }
    float first = (float)Scalar<T>::load(x);
    if (bi == 0xffffffffu || first != first) bi = 0;
    tokens[b] = bi;
    if (history) history[(int64_t)step * B + b] = bi;
    chosen = bi;
  }
  __syncthreads();
  publish_token<T>(chosen, b, state, B, dpos, dstep, embed, x_next, H, embed_scale);
}

// The token choice of the reference's example loop (examples/phi2/src/main.rs:29-50,76-87): the logits
// row as f32, the repeat penalty applied once to every token id that occurs among the last `last_n`
// tokens of the sequence so far (a logit >= 0 is divided by the penalty, any other is multiplied by it;
// skipped when the penalty is below 1), then the maximum under f32 total order (-NaN < -inf < ... < -0 <
// +0 < ... < +inf < +NaN) with the LAST maximum winning, as Iterator::max_by does.  The membership set is
// a bitmap over the vocabulary in LDS (words = ceil(n / 32)).  Returns the chosen index to every thread.
__device__ __forceinline__ uint32_t total_order_key(float v) {
  const uint32_t u = __float_as_uint(v);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
template <typename T>
__device__ uint32_t sample_row(const T *x, int64_t n, const uint32_t *window, int wn, float penalty, uint32_t *bitmap,
                               unsigned long long *s_best) {
  const int words = (int)((n + 31) / 32);
  const bool use_pen = penalty >= 1.0f && wn > 0;
  if (use_pen) {
    for (int w = threadIdx.x; w < words; w += blockDim.x) bitmap[w] = 0u;
    __syncthreads();
    for (int j = threadIdx.x; j < wn; j += blockDim.x) {
      const uint32_t t = window[j];
      if ((int64_t)t < n) atomicOr(&bitmap[t >> 5], 1u << (t & 31u));
    }
    __syncthreads();
  }
  // (key << 32 | index): the maximum of this composite is the largest key and, among equals, the largest index
  unsigned long long best = 0ull;
  auto visit = [&](float v, uint32_t i) {
    if (use_pen && ((bitmap[i >> 5] >> (i & 31u)) & 1u)) v = v >= 0.0f ? v / penalty : v * penalty;
    const unsigned long long c = ((unsigned long long)total_order_key(v) << 32) | i;
    best = c > best ? c : best;
  };
  constexpr int VEC = 16 / sizeof(T);
  if (n % VEC == 0 && ((uintptr_t)x & 15) == 0) {
    struct alignas(16) Pack { T v[VEC]; };
    const Pack *xp = reinterpret_cast<const Pack *>(x);
    const int64_t chunks = n / VEC;
    for (int64_t c0 = threadIdx.x; c0 < chunks; c0 += (int64_t)blockDim.x * 4) {
      Pack pk[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t c = c0 + (int64_t)u * blockDim.x;
        if (c < chunks) pk[u] = xp[c];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t c = c0 + (int64_t)u * blockDim.x;
        if (c < chunks) {
#pragma unroll
          for (int j = 0; j < VEC; ++j) visit((float)Scalar<T>::load(&pk[u].v[j]), (uint32_t)(c * VEC + j));
        }
      }
    }
  } else {
    for (int64_t i = threadIdx.x; i < n; i += blockDim.x) visit((float)Scalar<T>::load(x + i), (uint32_t)i);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const unsigned long long other = (unsigned long long)__shfl_xor((long long)best, o, 64);
    best = other > best ? other : best;
  }
  if ((threadIdx.x & 63) == 0) s_best[threadIdx.x >> 6] = best;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < (int)(blockDim.x >> 6); ++w) best = s_best[w] > best ? s_best[w] : best;
    s_best[0] = best;
  }
  __syncthreads();
  return (uint32_t)(s_best[0] & 0xffffffffull);
}

// The penalised choice as a primitive: one block per row of logits; context[b] holds n_context token ids.
template <typename T>
__global__ void __launch_bounds__(1024)
k_sample_rows(const T *logits, int64_t n, const uint32_t *context, int n_context, float penalty, uint32_t *out) {
  extern __shared__ uint32_t samp_bitmap[];
  __shared__ unsigned long long s_best[16];
  const int b = blockIdx.x;
  const uint32_t tok = sample_row<T>(logits + (int64_t)b * n, n, context + (int64_t)b * n_context, n_context, penalty,
                                     samp_bitmap, s_best);
  if (threadIdx.x == 0) out[b] = tok;
}

// k_select_token with the example loop's token choice.  log[b] (capacity log_cap) holds every token of
// sequence b so far, prompt first; the sequence has state->pos + dpos tokens when this runs, and the chosen
// token is appended behind them.
template <typename T>
__global__ void __launch_bounds__(1024)
k_sample_token(const T *logits, int64_t n, uint32_t *tokens, uint32_t *history, DevState *state, int B, int dpos,
               int dstep, const T *embed, T *x_next, int H, float embed_scale, uint32_t *log, int log_cap,
               float penalty, int last_n) {
  extern __shared__ uint32_t samp_bitmap[];
  __shared__ unsigned long long s_best[16];
  const int b = blockIdx.x;
  const int step = state->step;
  int n_tok = state->pos + dpos;
  if (n_tok > log_cap - 1) n_tok = log_cap - 1;   // cannot happen for a call that passed the host's checks
  const int wn = n_tok < last_n ? n_tok : last_n;
  uint32_t *row = log + (int64_t)b * log_cap;
  const uint32_t tok = sample_row<T>(logits + (int64_t)b * n, n, row + (n_tok - wn), wn, penalty, samp_bitmap, s_best);
  if (threadIdx.x == 0) {
    tokens[b] = tok;
    if (history) history[(int64_t)step * B + b] = tok;
    row[n_tok] = tok;
  }
  publish_token<T>(tok, b, state, B, dpos, dstep, embed, x_next, H, embed_scale);
}

template <typename T>
__global__ void __launch_bounds__(256) k_to_f32(float *out, const T *in, int64_t n) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    out[i] = (float)Scalar<T>::load(in + i);
}

static int grid1d(int64_t n) {
  int64_t b = (n + 255) / 256;
  return (int)(b < kNumCU * 16 ? (b < 1 ? 1 : b) : kNumCU * 16);
}

// ------------------------------------------------------------------ host-side construction
static int dalloc(rai_hip_decoder *d, size_t bytes, char **out) {
  void *p = nullptr;
  RAI_HIP_TRY(hipSetDevice(d->dev));
  hipError_t e = hipMalloc(&p, bytes ? bytes : 16);
  if (e != hipSuccess) return fail(RAI_ERR_OOM, "decoder: hipMalloc(%zu): %s", bytes, hipGetErrorString(e));
  d->allocs.push_back(p);
  *out = (char *)p;
  return RAI_OK;
}

static void add_slot(rai_hip_decoder *d, const std::string &name, int64_t rows, int64_t cols, char *dst, int64_t pitch) {
  d->slot_by_name[name] = (int)d->slots.size();
  d->slots.push_back(ParamSlot{name, rows, cols, dst, pitch, false, 0, nullptr});
}
static void add_split_slot(rai_hip_decoder *d, const std::string &name, int64_t rows, int64_t cols, char *dst, int64_t pitch,
                           int64_t rows2, char *dst2) {
  d->slot_by_name[name] = (int)d->slots.size();
  d->slots.push_back(ParamSlot{name, rows, cols, dst, pitch, false, rows2, dst2});
}

// Rotary tables.  Reference chain (phi2.rs:44-64): inv_freq computed with f32
// powf, cast to the model dtype; positions cast to the model dtype; their
// product (a K=1 matmul) rounded to the model dtype; sin/cos rounded again.
static float round_dt(float v, int dtype) {
  if (dtype != RAI_BF16) return v;
  uint32_t u;
  memcpy(&u, &v, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return v;
  u += 0x7fffu + ((u >> 16) & 1u);
  u &= 0xffff0000u;
  memcpy(&v, &u, 4);
  return v;
}

// f64 -> model dtype with a single rounding.  Going through f32 rounds twice, which differs exactly when
// the f32 value lands on a bf16 tie: the part the first rounding dropped then decides the direction.
static float round_dt_from_double(double v, int dtype) {
  const float f = (float)v;
  if (dtype != RAI_BF16) return f;
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) >= 0x7f800000u || (u & 0xffffu) != 0x8000u || (double)f == v) return round_dt(f, dtype);
  const bool away = fabs(v) > fabs((double)f);   // the exact value lies beyond the tie
  u = (u & 0xffff0000u) + (away ? 0x10000u : 0u);
  float r;
  memcpy(&r, &u, 4);
  return r;
}

static int build_rope_tables(rai_hip_decoder *d) {
  const auto &c = d->cfg;
  const int rot = c.rotary_dim, half = rot / 2, P = c.max_position_embeddings;
  std::vector<float> cs((size_t)P * rot), sn((size_t)P * rot);
  for (int i = 0; i < half; ++i) {
    float inv, inv_dt;
    if (c.arch == RAI_ARCH_PHI2) inv = 1.0f / powf((float)c.rope_theta, (float)(2 * i) / (float)rot);
    else if (c.arch == RAI_ARCH_PHI3) inv = (float)(1.0 / pow(c.rope_theta, (double)(2 * i) / (double)rot));
    else inv = 1.0f / (float)pow(c.rope_theta, (double)(2 * i) / (double)rot);
    inv_dt = round_dt(inv, c.dtype);
    if (c.arch == RAI_ARCH_PHI3)   // phi3.rs:45-51: an f64 tensor cast to the model dtype, one rounding from f64
      inv_dt = round_dt_from_double(1.0 / pow(c.rope_theta, (double)(2 * i) / (double)rot), c.dtype);
    for (int p = 0; p < P; ++p) {
      float ang;
      if (c.rope_tables_f32) ang = (float)p * inv;
      else ang = round_dt(round_dt((float)p, c.dtype) * inv_dt, c.dtype);
      float cv = round_dt(cosf(ang), c.dtype), sv = round_dt(sinf(ang), c.dtype);
      cs[(size_t)p * rot + i] = cs[(size_t)p * rot + i + half] = cv;
      sn[(size_t)p * rot + i] = sn[(size_t)p * rot + i + half] = sv;
    }
  }
  const size_t n = (size_t)P * rot;
  if (c.dtype == RAI_F32) {
    RAI_HIP_TRY(hipMemcpy(d->cos_t, cs.data(), n * 4, hipMemcpyHostToDevice));
    RAI_HIP_TRY(hipMemcpy(d->sin_t, sn.data(), n * 4, hipMemcpyHostToDevice));
  } else {
    std::vector<uint16_t> cb(n), sb(n);
    for (size_t i = 0; i < n; ++i) {
      uint32_t u;
      memcpy(&u, &cs[i], 4);
      cb[i] = (uint16_t)(u >> 16);
      memcpy(&u, &sn[i], 4);
      sb[i] = (uint16_t)(u >> 16);
    }
    RAI_HIP_TRY(hipMemcpy(d->cos_t, cb.data(), n * 2, hipMemcpyHostToDevice));
    RAI_HIP_TRY(hipMemcpy(d->sin_t, sb.data(), n * 2, hipMemcpyHostToDevice));
  }
  return RAI_OK;
}

static int create_phi2(rai_hip_decoder *d) {
  const size_t es = d->es;
  const int H = d->H, I = d->I, QD = d->QD, KD = d->KD, V = d->V;
  RAI_TRY(dalloc(d, (size_t)V * H * es, &d->embed));
  add_slot(d, "model.embed_tokens.weight", V, H, d->embed, H);
  d->layers.resize(d->L);
  // The two weight matrices of all layers sit back to back (layer l at a fixed
  // stride), so a kernel that walks through the layers computes their addresses
  // instead of loading them.
  char *wa_all = nullptr, *wb_all = nullptr;
  const size_t wa_bytes = (size_t)d->NA * H * es, wb_bytes = (size_t)H * d->KB * es;
  RAI_TRY(dalloc(d, wa_bytes * d->L, &wa_all));
  RAI_TRY(dalloc(d, wb_bytes * d->L, &wb_all));
  for (int l = 0; l < d->L; ++l) {
    Layer &ly = d->layers[l];
    ly.Wa = wa_all + wa_bytes * l;
    RAI_TRY(dalloc(d, (size_t)d->NA * es, &ly.ba));
    ly.Wb = wb_all + wb_bytes * l;
    RAI_TRY(dalloc(d, (size_t)H * es, &ly.bd));
    RAI_TRY(dalloc(d, (size_t)H * es, &ly.bf));
    RAI_TRY(dalloc(d, (size_t)H * es, &ly.ln_w));
    RAI_TRY(dalloc(d, (size_t)H * es, &ly.ln_b));
    const std::string p = "model.layers." + std::to_string(l) + ".";
    add_slot(d, p + "self_attn.q_proj.weight", QD, H, ly.Wa, H);
    add_slot(d, p + "self_attn.q_proj.bias", 1, QD, ly.ba, QD);
    add_slot(d, p + "self_attn.k_proj.weight", KD, H, ly.Wa + (size_t)QD * H * es, H);
    add_slot(d, p + "self_attn.k_proj.bias", 1, KD, ly.ba + (size_t)QD * es, KD);
    add_slot(d, p + "self_attn.v_proj.weight", KD, H, ly.Wa + (size_t)(QD + KD) * H * es, H);
    add_slot(d, p + "self_attn.v_proj.bias", 1, KD, ly.ba + (size_t)(QD + KD) * es, KD);
    add_slot(d, p + "self_attn.dense.weight", H, QD, ly.Wb, d->KB);
    add_slot(d, p + "self_attn.dense.bias", 1, H, ly.bd, H);
    add_slot(d, p + "mlp.fc1.weight", I, H, ly.Wa + (size_t)(QD + 2 * KD) * H * es, H);
    add_slot(d, p + "mlp.fc1.bias", 1, I, ly.ba + (size_t)(QD + 2 * KD) * es, I);
    add_slot(d, p + "mlp.fc2.weight", H, I, ly.Wb + (size_t)QD * es, d->KB);
    add_slot(d, p + "mlp.fc2.bias", 1, H, ly.bf, H);
    add_slot(d, p + "input_layernorm.weight", 1, H, ly.ln_w, H);
    add_slot(d, p + "input_layernorm.bias", 1, H, ly.ln_b, H);
  }
  RAI_TRY(dalloc(d, (size_t)H * es, &d->lnf_w));
  RAI_TRY(dalloc(d, (size_t)H * es, &d->lnf_b));
  add_slot(d, "model.final_layernorm.weight", 1, H, d->lnf_w, H);
  add_slot(d, "model.final_layernorm.bias", 1, H, d->lnf_b, H);
  if (d->cfg.tie_word_embeddings) {
    d->head_w = d->embed;
    d->head_b = nullptr;
  } else {
    RAI_TRY(dalloc(d, (size_t)V * H * es, &d->head_w));
    RAI_TRY(dalloc(d, (size_t)V * es, &d->head_b));
    add_slot(d, "lm_head.weight", V, H, d->head_w, H);
    add_slot(d, "lm_head.bias", 1, V, d->head_b, V);
  }
  return RAI_OK;
}

// Qwen2 (rai-models/src/llm/qwen2.rs:276-300) and Gemma (gemma.rs:309-338) parameter slots.
static int create_seq(rai_hip_decoder *d) {
  const size_t es = d->es;
  const int H = d->H, I = d->I, QD = d->QD, KD = d->KD, V = d->V;
  const bool qwen = d->cfg.arch == RAI_ARCH_QWEN2, phi3 = d->cfg.arch == RAI_ARCH_PHI3;
  RAI_TRY(dalloc(d, (size_t)V * H * es, &d->embed));
  add_slot(d, "model.embed_tokens.weight", V, H, d->embed, H);
  d->layers.resize(d->L);
  for (int l = 0; l < d->L; ++l) {
    Layer &ly = d->layers[l];
    memset(&ly, 0, sizeof(ly));
    const int NQ = QD + 2 * KD;
    RAI_TRY(dalloc(d, (size_t)NQ * H * es, &ly.Wqkv));
    RAI_TRY(dalloc(d, (size_t)H * QD * es, &ly.Wo));
    RAI_TRY(dalloc(d, (size_t)2 * I * H * es, &ly.Wgu));
    RAI_TRY(dalloc(d, (size_t)H * I * es, &ly.Wdown));
    RAI_TRY(dalloc(d, (size_t)H * es, &ly.n1_w));
    RAI_TRY(dalloc(d, (size_t)H * es, &ly.n2_w));
    const std::string p = "model.layers." + std::to_string(l) + ".";
    if (phi3) {  // one projection whose rows are q | k | v (phi3.rs:131-132,166-176)
      add_slot(d, p + "self_attn.qkv_proj.weight", NQ, H, ly.Wqkv, H);
    } else {
      add_slot(d, p + "self_attn.q_proj.weight", QD, H, ly.Wqkv, H);
      add_slot(d, p + "self_attn.k_proj.weight", KD, H, ly.Wqkv + (size_t)QD * H * es, H);
      add_slot(d, p + "self_attn.v_proj.weight", KD, H, ly.Wqkv + (size_t)(QD + KD) * H * es, H);
    }
    if (qwen) {  // q/k/v carry a bias, o_proj does not (qwen2.rs:137-140)
      RAI_TRY(dalloc(d, (size_t)NQ * es, &ly.bqkv));
      add_slot(d, p + "self_attn.q_proj.bias", 1, QD, ly.bqkv, QD);
      add_slot(d, p + "self_attn.k_proj.bias", 1, KD, ly.bqkv + (size_t)QD * es, KD);
      add_slot(d, p + "self_attn.v_proj.bias", 1, KD, ly.bqkv + (size_t)(QD + KD) * es, KD);
    }
    add_slot(d, p + "self_attn.o_proj.weight", H, QD, ly.Wo, QD);
    // gate row n -> packed row 2n, up row n -> packed row 2n+1 (pitch of two rows)
    if (phi3) {  // rows [0, I) are the gate, rows [I, 2I) the up projection (phi3.rs:97-101)
      add_split_slot(d, p + "mlp.gate_up_proj.weight", 2 * (int64_t)I, H, ly.Wgu, 2 * (int64_t)H, I, ly.Wgu + (size_t)H * es);
    } else {
      add_slot(d, p + "mlp.gate_proj.weight", I, H, ly.Wgu, 2 * (int64_t)H);
      add_slot(d, p + "mlp.up_proj.weight", I, H, ly.Wgu + (size_t)H * es, 2 * (int64_t)H);
    }
    add_slot(d, p + "mlp.down_proj.weight", H, I, ly.Wdown, I);
    add_slot(d, p + "input_layernorm.weight", 1, H, ly.n1_w, H);
    add_slot(d, p + "post_attention_layernorm.weight", 1, H, ly.n2_w, H);
  }
  RAI_TRY(dalloc(d, (size_t)H * es, &d->lnf_w));
  d->lnf_b = nullptr;
  add_slot(d, "model.norm.weight", 1, H, d->lnf_w, H);
  d->head_b = nullptr;
  if (d->cfg.arch == RAI_ARCH_GEMMA || d->cfg.tie_word_embeddings) {
    d->head_w = d->embed;  // gemma.rs:330 lm_head shares the embedding matrix
  } else {
    RAI_TRY(dalloc(d, (size_t)V * H * es, &d->head_w));
    add_slot(d, "lm_head.weight", V, H, d->head_w, H);
  }
  return RAI_OK;
}

// ------------------------------------------------------------------ forward
template <typename T> static void launch_embed(rai_hip_decoder *d, hipStream_t st, int64_t rows) {
  hipLaunchKernelGGL((k_embed<T>), dim3(grid1d(rows * d->H)), dim3(256), 0, st, (T *)d->x, (const T *)d->embed, d->ids,
                     rows, d->H, d->V, index_error_counter(d->dev), d->embed_scale);
}
template <typename T> static void launch_rope_append(rai_hip_decoder *d, hipStream_t st, int l, int B, int S) {
  const size_t per_layer = (size_t)d->cfg.max_batch * d->Hkv * d->cfg.max_context * d->D;
  int64_t total = (int64_t)B * S * (d->Hq + 2 * d->Hkv) * d->D;
  constexpr int VEC = 16 / sizeof(T);
  const int rot = d->cfg.rotary_dim;
  if (d->D % VEC == 0 && (rot / 2) % VEC == 0 && (d->QD + 2 * d->KD) % VEC == 0 && total / VEC < ((int64_t)1 << 31)) {
    hipLaunchKernelGGL((k_rope_append_vec<T>), dim3(grid1d(total / VEC)), dim3(256), 0, st, (T *)d->qkv,
                       (T *)d->kcache + per_layer * l, (T *)d->vcache + per_layer * l, (const T *)d->cos_t,
                       (const T *)d->sin_t, d->state, B, S, d->Hq, d->Hkv, d->D, rot, d->cfg.max_context);
    return;
  }
  hipLaunchKernelGGL((k_rope_append<T>), dim3(grid1d(total)), dim3(256), 0, st, (T *)d->qkv,
                     (T *)d->kcache + per_layer * l, (T *)d->vcache + per_layer * l, (const T *)d->cos_t,
                     (const T *)d->sin_t, d->state, B, S, d->Hq, d->Hkv, d->D, d->cfg.rotary_dim, d->cfg.max_context);
}

static rai_hip_tensor desc2(void *p, int dtype, int64_t rows, int64_t cols, int64_t row_stride) {
  rai_hip_tensor t;
  memset(&t, 0, sizeof(t));
  t.data = p;
  t.dtype = dtype;
  t.rank = 2;
  t.shape[0] = rows;
  t.shape[1] = cols;
  t.stride[0] = row_stride;
  t.stride[1] = 1;
  return t;
}
static rai_hip_tensor desc1(void *p, int dtype, int64_t n) {
  rai_hip_tensor t;
  memset(&t, 0, sizeof(t));
  t.data = p;
  t.dtype = dtype;
  t.rank = 1;
  t.shape[0] = n;
  t.stride[0] = 1;
  return t;
}

static int linear(rai_hip_decoder *d, hipStream_t st, const LinearArgs &a0) {
  LinearArgs a = a0;
  a.dev = d->dev;
  return d->cfg.dtype == RAI_BF16 ? launch_linear_bf16(st, a) : launch_linear_f32(st, a);
}

static MegaArgs mega_args(rai_hip_decoder *d) {
  MegaArgs m;
  memset(&m, 0, sizeof(m));
  m.layers = d->mega_layers;
  m.Wa0 = (const uint16_t *)d->layers[0].Wa; m.Wb0 = (const uint16_t *)d->layers[0].Wb;
  m.wa_stride = (int64_t)d->NA * d->H; m.wb_stride = (int64_t)d->H * d->KB;
  m.L = d->L; m.H = d->H; m.I = d->I; m.QD = d->QD; m.NA = d->NA; m.n_qkv = d->QD + 2 * d->KD;
  m.Hq = d->Hq; m.Hkv = d->Hkv; m.rot = d->cfg.rotary_dim; m.Tmax = d->cfg.max_context;
  m.x = (uint16_t *)d->x;
  m.xp = d->mega_xchg;
  m.qkvp = m.xp + d->H / 2;
  m.actp = m.qkvp + (d->QD + 2 * d->KD) / 2;
  m.attnp = m.actp + kMegaActPackets;
  m.kcache = (uint16_t *)d->kcache; m.vcache = (uint16_t *)d->vcache;
  m.kv_layer_stride = (int64_t)d->cfg.max_batch * d->Hkv * d->cfg.max_context * d->D;
  m.cos_t = (const uint16_t *)d->cos_t; m.sin_t = (const uint16_t *)d->sin_t;
  m.state = d->state;
  m.ln_eps = (float)d->cfg.norm_eps; m.scale = (float)(1.0 / sqrt((double)d->D));
  m.act = d->cfg.hidden_act;
  static const int rows_attn = getenv("RAI_HIP_MEGA_ROWS_ATTN") ? atoi(getenv("RAI_HIP_MEGA_ROWS_ATTN")) : 0;
  m.rows_attn = rows_attn;
  m.prof = d->mega_prof;
  // Failure-path test hooks (instrumented kernel only), read on every launch that is not replayed from a graph.
  const char *sl = getenv("RAI_HIP_MEGA_SPIN_LIMIT"), *mb = getenv("RAI_HIP_MEGA_TEST_MUTE_BLOCK");
  m.spin_limit = sl && atoi(sl) > 0 ? (unsigned)atoi(sl) : mega_default_spin_limit();
  m.mute_block = mb ? atoi(mb) : -1;
  return m;
}

// Batched decode (9..64 rows) streams every weight matrix once per step through the small-M MFMA kernel; that
// kernel reads 1 KB per load instruction from a copy of the matrix in MFMA-fragment order.  The copies are made on
// the first such step after the parameters changed (never under stream capture: generate runs its first
// single-token step eagerly) and double the weight memory of the decoder.
static bool wants_fragments(const rai_hip_decoder *d, int64_t M) {
  static const bool off = getenv("RAI_HIP_NO_FRAG") != nullptr;
  return !off && d->cfg.dtype == RAI_BF16 && M > 8 && M <= 64;
}
static int ensure_fragments(rai_hip_decoder *d, hipStream_t st) {
  if (d->frag_ready) return RAI_OK;
  auto one = [&](char *W, int64_t ldw, int N, int K, char **dst) -> int {
    if (!W || K % 32) { *dst = nullptr; return RAI_OK; }
    if (!*dst) RAI_TRY(dalloc(d, linear_fragment_elems(N, K) * d->es, dst));
    return launch_linear_fragment_layout(st, W, ldw, N, K, *dst);
  };
  const int NQ = d->QD + 2 * d->KD;
  for (Layer &ly : d->layers) {
    if (d->cfg.arch == RAI_ARCH_PHI2) {
      RAI_TRY(one(ly.Wa, d->H, d->NA, d->H, &ly.Wa_f));
      RAI_TRY(one(ly.Wb, d->KB, d->H, d->KB, &ly.Wb_f));
    } else {
      RAI_TRY(one(ly.Wqkv, d->H, NQ, d->H, &ly.Wqkv_f));
      RAI_TRY(one(ly.Wo, d->QD, d->H, d->QD, &ly.Wo_f));
      RAI_TRY(one(ly.Wgu, d->H, 2 * d->I, d->H, &ly.Wgu_f));
      RAI_TRY(one(ly.Wdown, d->I, d->H, d->I, &ly.Wdown_f));
    }
  }
  RAI_TRY(one(d->head_w, d->H, d->V, d->H, &d->head_f));
  d->frag_ready = true;
  return RAI_OK;
}

constexpr int64_t kSampleMaxVocab = 15 * 1024 * 32;  // the membership bitmap of the penalised choice takes vocab / 8 bytes of LDS

// Chooses the next token of every sequence from d->logits: plain greedy argmax, or the example loop's
// choice when the decoder is in sampling mode.
static int launch_token_choice(rai_hip_decoder *d, hipStream_t st, int B, int S, bool advance_step) {
  const int dt = d->cfg.dtype;
  uint32_t *hist = advance_step ? d->history : nullptr;
  const int dstep = advance_step ? 1 : 0;
  if (d->sample_on) {
    const size_t lds = (size_t)((d->V + 31) / 32) * sizeof(uint32_t);
    if (dt == RAI_BF16)
      hipLaunchKernelGGL((k_sample_token<bf16_raw>), dim3(B), dim3(1024), lds, st, (const bf16_raw *)d->logits,
                         (int64_t)d->V, d->tokens, hist, d->state, B, S, dstep, (const bf16_raw *)d->embed,
                         (bf16_raw *)d->x, d->H, d->embed_scale, d->token_log, d->token_log_cap, d->sample_penalty,
                         d->sample_last_n);
    else
      hipLaunchKernelGGL((k_sample_token<float>), dim3(B), dim3(1024), lds, st, (const float *)d->logits,
                         (int64_t)d->V, d->tokens, hist, d->state, B, S, dstep, (const float *)d->embed, (float *)d->x,
                         d->H, d->embed_scale, d->token_log, d->token_log_cap, d->sample_penalty, d->sample_last_n);
    return launch_check("sample_token");
  }
  // A wide vocabulary is scanned by many blocks first (one block per row would fetch its 100 KB - 500 KB in several
  // dependent rounds of loads: 35 us for 32 rows of 256000); the choice kernel then merges the shares' results.
  int splits = 0;
  if (d->V >= 32768 && !getenv("RAI_HIP_NO_SPLIT_CHOICE")) {
    splits = 1;
    while (B * splits < kNumCU && splits < kChoiceMaxSplits && d->V / (splits * 2) >= 8192) splits *= 2;
    RAI_TRY(launch_argmax_partials(st, dt, d->logits, B, d->V, splits, d->choice_val, d->choice_idx));
  }
  const int threads = splits > 0 ? 256 : 1024;
  if (dt == RAI_BF16)
    hipLaunchKernelGGL((k_select_token<bf16_raw>), dim3(B), dim3(threads), 0, st, (const bf16_raw *)d->logits,
                       (int64_t)d->V, d->tokens, hist, d->state, B, S, dstep, (const bf16_raw *)d->embed,
                       (bf16_raw *)d->x, d->H, d->embed_scale, d->choice_val, d->choice_idx, splits);
  else
    hipLaunchKernelGGL((k_select_token<float>), dim3(B), dim3(threads), 0, st, (const float *)d->logits, (int64_t)d->V,
                       d->tokens, hist, d->state, B, S, dstep, (const float *)d->embed, (float *)d->x, d->H,
                       d->embed_scale, d->choice_val, d->choice_idx, splits);
  return launch_check("select_token");
}

// ids (B*S u32) are already in d->ids; device state holds the context length.
// With from_tokens the input embeddings were already written to d->x by the
// previous step's token selection (single-token steps only).
static int forward_phi2(rai_hip_decoder *d, int B, int S, bool advance_step, bool from_tokens = false) {
  hipStream_t st = stream_of(d->dev);
  if (!st) return RAI_ERR_HIP;
  const int dt = d->cfg.dtype;
  const int H = d->H, QD = d->QD, KD = d->KD, I = d->I;
  const int64_t M = (int64_t)B * S;
  const int ldq = QD + 2 * KD;
  const bool fuse_ln = dt == RAI_BF16 && M <= 8;
  const int T_after = d->ctx_len + S;
  const bool frag = wants_fragments(d, M);
  if (frag) RAI_TRY(ensure_fragments(d, st));

  if (!from_tokens) {
    if (dt == RAI_BF16) launch_embed<bf16_raw>(d, st, M); else launch_embed<float>(d, st, M);
    RAI_TRY(launch_check("embed"));
  }

  char *x = d->x, *xn = d->x2;
  const bool use_mega = S == 1 && B == 1 && d->mega_ok && !d->want_hidden;
  if (use_mega) {
    MegaArgs m = mega_args(d);
    RAI_TRY(launch_phi2_decode_step(st, m, d->D, d->num_cu));
  }
  bool ln_ready = false;   // d->ln already holds this layer's LayerNorm(x): the previous layer's last Linear wrote it
  for (int l = 0; l < (use_mega ? 0 : d->L); ++l) {
    const Layer &ly = d->layers[l];
    LinearArgs a = linear_args_default();
    a.splitk_ws = d->splitk_ws; a.splitk_ws_bytes = d->splitk_ws_bytes;
    if (fuse_ln) {
      a.A = x; a.lda = H;
      a.ln_kind = 0; a.ln_w = ly.ln_w; a.ln_b = ly.ln_b; a.ln_eps = (float)d->cfg.norm_eps;
    } else {
      if (!ln_ready) {
        rai_hip_tensor tx = desc2(x, dt, M, H, H), tw = desc1(ly.ln_w, dt, H), tb = desc1(ly.ln_b, dt, H),
                       to = desc2(d->ln, dt, M, H, H);
        RAI_TRY(rai_hip_layer_norm(d->dev, &tx, &tw, &tb, d->cfg.norm_eps, &to));
      }
      a.A = d->ln; a.lda = H;
    }
    ln_ready = false;
    a.W = ly.Wa; a.ldw = H; a.bias = ly.ba;
    a.Wfrag = frag ? ly.Wa_f : nullptr;
    a.out1 = d->qkv; a.ld1 = ldq;
    a.out2 = d->cat + (size_t)QD * d->es; a.ld2 = d->KB;
    a.M = (int)M; a.N = d->NA; a.K = H; a.n_split = ldq;
    a.act = d->cfg.hidden_act; a.act_from = ldq;
    RAI_TRY(linear(d, st, a));

    const size_t per_layer = (size_t)d->cfg.max_batch * d->Hkv * d->cfg.max_context * d->D;
    if (S == 1) {
      // decode: rotary + cache append + attention in one launch, context length read on the device
      AttnDecodeArgs t;
      memset(&t, 0, sizeof(t));
      t.qkv = d->qkv;
      t.kcache = d->kcache + per_layer * l * d->es;
      t.vcache = d->vcache + per_layer * l * d->es;
      t.out = d->cat;
      t.out_row_stride = d->KB;
      t.cos_t = d->cos_t; t.sin_t = d->sin_t; t.rot = d->cfg.rotary_dim;
      t.pos_dev = &d->state->pos;
      t.B = B; t.Hq = d->Hq; t.Hkv = d->Hkv; t.D = d->D; t.Tmax = d->cfg.max_context;
      t.scale = (float)(1.0 / sqrt((double)d->D));
      t.f32_scores = 1; t.dtype = dt;
      t.ws = (float *)d->attn_ws; t.counters = d->attn_counters;
      RAI_TRY(launch_attention_decode(st, t));
    } else {
      if (dt == RAI_BF16) launch_rope_append<bf16_raw>(d, st, l, B, S); else launch_rope_append<float>(d, st, l, B, S);
      RAI_TRY(launch_check("rope_append"));
      AttnArgs t;
      memset(&t, 0, sizeof(t));
      t.q = d->qkv;
      t.k = d->kcache + per_layer * l * d->es;
      t.v = d->vcache + per_layer * l * d->es;
      t.out = d->cat;
      t.qs[0] = (int64_t)S * ldq; t.qs[1] = d->D; t.qs[2] = ldq;
      t.ks[0] = t.vs[0] = (int64_t)d->Hkv * d->cfg.max_context * d->D;
      t.ks[1] = t.vs[1] = (int64_t)d->cfg.max_context * d->D;
      t.ks[2] = t.vs[2] = d->D;
      t.out_row_stride = d->KB;
      t.B = B; t.Hq = d->Hq; t.Hkv = d->Hkv; t.S = S; t.D = d->D;
      t.scale = (float)(1.0 / sqrt((double)d->D));
      t.causal = 1; t.f32_scores = 1; t.dtype = dt;
      t.T = T_after;
      RAI_TRY(launch_attention(st, t));
    }

    LinearArgs b = linear_args_default();
    b.A = d->cat; b.lda = d->KB;
    b.W = ly.Wb; b.ldw = d->KB;
    b.Wfrag = frag ? ly.Wb_f : nullptr;
    b.bias = ly.bd; b.bias2 = ly.bf;
    b.residual = x; b.ldr = H;
    b.out1 = xn; b.ld1 = H;
    b.M = (int)M; b.N = H; b.K = d->KB; b.n_split = H;
    b.splitk_ws = d->splitk_ws; b.splitk_ws_bytes = d->splitk_ws_bytes;
    if (!fuse_ln && dt == RAI_BF16 && l + 1 < d->L) {
      // the next layer's input LayerNorm rides on the pass that sums this product's split-K partial sums
      const Layer &nx = d->layers[l + 1];
      b.post_ln_out = d->ln; b.post_ln_w = nx.ln_w; b.post_ln_b = nx.ln_b; b.post_ln_eps = (float)d->cfg.norm_eps;
      ln_ready = linear_fuses_post_norm(b);
      if (!ln_ready) b.post_ln_out = nullptr;
    }
    RAI_TRY(linear(d, st, b));
    char *tmp = x; x = xn; xn = tmp;
  }

  if (d->want_hidden) {   // the token choice below writes the next input embedding over the first rows of d->x
    RAI_REQUIRE(!use_mega, RAI_ERR_UNSUPPORTED, "the persistent single-token kernel keeps the residual stream in its packets");
    RAI_HIP_TRY(hipMemcpyAsync(d->hidden_copy, x, (size_t)M * H * d->es, hipMemcpyDeviceToDevice, st));
  }
  // final LayerNorm on the last position of every sequence, then the head
  // (phi2.rs:345-346: narrow(1, S-1, 1) before lm_head).
  LinearArgs h = linear_args_default();
  char *last_rows = x + (size_t)(S - 1) * H * d->es;  // row b*S + S-1, stride S*H
  if (dt == RAI_BF16 && B <= 8) {
    h.A = last_rows; h.lda = (int64_t)S * H;
    h.ln_kind = 0; h.ln_w = d->lnf_w; h.ln_b = d->lnf_b; h.ln_eps = (float)d->cfg.norm_eps;
  } else {
    rai_hip_tensor tx = desc2(last_rows, dt, B, H, (int64_t)S * H), tw = desc1(d->lnf_w, dt, H),
                   tb = desc1(d->lnf_b, dt, H), to = desc2(d->last, dt, B, H, H);
    RAI_TRY(rai_hip_layer_norm(d->dev, &tx, &tw, &tb, d->cfg.norm_eps, &to));
    h.A = d->last; h.lda = H;
  }
  h.W = d->head_w; h.ldw = H; h.bias = d->head_b;
  if (wants_fragments(d, B)) {
    RAI_TRY(ensure_fragments(d, st));
    h.Wfrag = d->head_f;
  }
  h.out1 = d->logits; h.ld1 = d->V;
  h.M = B; h.N = d->V; h.K = H; h.n_split = d->V;
  // One sequence, greedy: final norm, head and token choice as one launch of the step kernel's weight stream
  // (RAI_HIP_NO_HEAD_KERNEL=1 keeps the three launches; read per call: tests compare both forms in one process).
  const char *no_head = getenv("RAI_HIP_NO_HEAD_KERNEL");
  if (B == 1 && dt == RAI_BF16 && !d->sample_on && d->mega_ok && !(no_head && *no_head && *no_head != '0')) {
    HeadArgs ha;
    memset(&ha, 0, sizeof(ha));
    ha.W = (const uint16_t *)d->head_w; ha.bias = (const uint16_t *)d->head_b;
    ha.x = (const uint16_t *)last_rows;
    ha.ln_w = (const uint16_t *)d->lnf_w; ha.ln_b = (const uint16_t *)d->lnf_b; ha.ln_eps = (float)d->cfg.norm_eps;
    ha.V = d->V; ha.H = H;
    ha.logits = (uint16_t *)d->logits;
    ha.best = d->head_best;
    ha.token = d->tokens; ha.history = advance_step ? d->history : nullptr;
    ha.state = d->state; ha.dpos = S; ha.dstep = advance_step ? 1 : 0;
    ha.embed = (const uint16_t *)d->embed; ha.x_next = (uint16_t *)d->x; ha.embed_scale = d->embed_scale;
    if (head_choice_eligible(ha, d->num_cu)) {
      RAI_TRY(launch_phi2_head_choice(st, ha, d->num_cu));
      d->ctx_len = T_after;
      return RAI_OK;
    }
  }
  RAI_TRY(linear(d, st, h));

  RAI_TRY(launch_token_choice(d, st, B, S, advance_step));
  d->ctx_len = T_after;
  return RAI_OK;
}

// Qwen2 / Gemma scale by an f64 1/sqrt(head_dim) cast to the model dtype (qwen2.rs:205, gemma.rs:238); Phi-3
// computes the scalar in f32 (phi3.rs:202).
static float seq_attn_scale(const rai_hip_decoder *d) {
  if (d->cfg.arch == RAI_ARCH_PHI3) return 1.0f / sqrtf((float)d->D);
  return (float)(1.0 / sqrt((double)d->D));
}

// RAI_HIP_CHAIN=1 opts in to the persistent decode chain kernel (read per call: the tests switch it)
static bool chain_wanted() {
  const char *e = getenv("RAI_HIP_CHAIN");
  return e && e[0] == '1';
}

// Sequential pre-norm block of Qwen2 (qwen2.rs:253-266) and Gemma (gemma.rs:286-299):
// x1 = x + o_proj(attn(norm1(x))); x = x1 + down(act(gate(norm2(x1))) * up(norm2(x1))).
static int forward_seq(rai_hip_decoder *d, int B, int S, bool advance_step, bool from_tokens = false) {
  hipStream_t st = stream_of(d->dev);
  if (!st) return RAI_ERR_HIP;
  const int dt = d->cfg.dtype;
  const int H = d->H, QD = d->QD, KD = d->KD, I = d->I;
  const int64_t M = (int64_t)B * S;
  const int ldq = QD + 2 * KD;
  const int kind = d->cfg.arch == RAI_ARCH_GEMMA ? 2 : 1;
  // the norm runs inside the Linear kernel for single rows and for the batched-decode row counts
  const bool fuse_norm = dt == RAI_BF16 && (M <= 8 || linear_mfma_fuses_norm((int)M, H, kind));
  const int T_after = d->ctx_len + S;
  const size_t per_layer = (size_t)d->cfg.max_batch * d->Hkv * d->cfg.max_context * d->D;
  const bool frag = wants_fragments(d, M);
  if (frag) RAI_TRY(ensure_fragments(d, st));

  if (!from_tokens) {
    if (dt == RAI_BF16) launch_embed<bf16_raw>(d, st, M); else launch_embed<float>(d, st, M);
    RAI_TRY(launch_check("embed"));
  }
  auto norm_rows = [&](char *src, char *w, char *dst, int64_t rows, int64_t src_stride) -> int {
    rai_hip_tensor tx = desc2(src, dt, rows, H, src_stride), tw = desc1(w, dt, H), to = desc2(dst, dt, rows, H, H);
    return rai_hip_rms_norm(d->dev, &tx, &tw, d->cfg.norm_eps, kind == 2, &to);
  };
  char *x = d->x, *x1 = d->x2;
  // Batched decode steps (9..32 rows): with RAI_HIP_CHAIN=1 everything between two attention calls -- o_proj,
  // gate|up, down and the next layer's q|k|v -- runs as one persistent launch of the decode chain kernel instead of
  // five launches (four Linears and the sum of the down projection's K splits).  Off by default: on the Gemma-2B
  // widths at batch 32 the chain launch takes 115 us a layer against 85 us for the five launches it replaces (its
  // four grid barriers and the reads past the L2s of what the phase before wrote cost more than the launch
  // boundaries they stand for, and the phase dispatch inside one kernel spills registers).
  const int down_splits = (I + 2047) / 2048;
  bool chain = S == 1 && frag && fuse_norm && M <= 32 && chain_wanted() && decode_chain_serves((int)M, H, QD, false) &&
               decode_chain_serves((int)M, 2 * I, H, false) && decode_chain_serves((int)M, H, I, true) &&
               decode_chain_serves((int)M, ldq, H, false) && ldq % 8 == 0 &&
               (size_t)down_splits * M * H * sizeof(float) <= d->splitk_ws_bytes && !d->want_hidden;
  for (int l = 0; chain && l < d->L; ++l) {
    const Layer &ly = d->layers[l];
    chain = ly.Wo_f && ly.Wgu_f && ly.Wdown_f && ly.Wqkv_f;
  }
  chain = chain && d->num_cu == device_cu_count(d->dev) && d->num_cu <= 512 && d->L <= 512;
  for (int l = 0; l < d->L; ++l) {
    const Layer &ly = d->layers[l];
    LinearArgs a = linear_args_default();
    if (chain && l > 0) {
      // this layer's q|k|v was the last phase of the previous layer's chain
    } else {
    if (fuse_norm) {
      a.A = x; a.lda = H;
      a.ln_kind = kind; a.ln_w = ly.n1_w; a.ln_eps = (float)d->cfg.norm_eps;
    } else {
      RAI_TRY(norm_rows(x, ly.n1_w, d->ln, M, H));
      a.A = d->ln; a.lda = H;
    }
    a.W = ly.Wqkv; a.ldw = H; a.bias = ly.bqkv;
    a.Wfrag = frag ? ly.Wqkv_f : nullptr;
    a.out1 = d->qkv; a.ld1 = ldq;
    a.M = (int)M; a.N = ldq; a.K = H; a.n_split = ldq;
    a.splitk_ws = d->splitk_ws; a.splitk_ws_bytes = d->splitk_ws_bytes;
    RAI_TRY(linear(d, st, a));
    }

    if (S == 1) {
      AttnDecodeArgs t;
      memset(&t, 0, sizeof(t));
      t.qkv = d->qkv;
      t.kcache = d->kcache + per_layer * l * d->es;
      t.vcache = d->vcache + per_layer * l * d->es;
      t.out = d->attn;
      t.out_row_stride = QD;
      t.cos_t = d->cos_t; t.sin_t = d->sin_t; t.rot = d->cfg.rotary_dim;
      t.pos_dev = &d->state->pos;
      t.B = B; t.Hq = d->Hq; t.Hkv = d->Hkv; t.D = d->D; t.Tmax = d->cfg.max_context;
      t.scale = seq_attn_scale(d);
      t.f32_scores = 0; t.dtype = dt;
      t.ws = (float *)d->attn_ws; t.counters = d->attn_counters;
      RAI_TRY(launch_attention_decode(st, t));
    } else {
      if (dt == RAI_BF16) launch_rope_append<bf16_raw>(d, st, l, B, S); else launch_rope_append<float>(d, st, l, B, S);
      RAI_TRY(launch_check("rope_append"));
      AttnArgs t;
      memset(&t, 0, sizeof(t));
      t.q = d->qkv;
      t.k = d->kcache + per_layer * l * d->es;
      t.v = d->vcache + per_layer * l * d->es;
      t.out = d->attn;
      t.qs[0] = (int64_t)S * ldq; t.qs[1] = d->D; t.qs[2] = ldq;
      t.ks[0] = t.vs[0] = (int64_t)d->Hkv * d->cfg.max_context * d->D;
      t.ks[1] = t.vs[1] = (int64_t)d->cfg.max_context * d->D;
      t.ks[2] = t.vs[2] = d->D;
      t.out_row_stride = QD;
      t.B = B; t.Hq = d->Hq; t.Hkv = d->Hkv; t.S = S; t.D = d->D;
      t.scale = seq_attn_scale(d);
      t.causal = 1; t.f32_scores = 0; t.dtype = dt;
      t.T = T_after;
      RAI_TRY(launch_attention(st, t));
    }

    if (chain) {
      ChainArgs c;
      memset(&c, 0, sizeof(c));
      auto lin = [&](ChainPhase &p, const void *A, int64_t lda, bool a_fresh, const void *Wf, int N, int K, void *out, int64_t ldo) {
        p.kind = RAI_CHAIN_LINEAR;
        p.A = A; p.lda = lda; p.a_fresh = a_fresh;
        p.Wfrag = Wf;
        p.out = out; p.ldo = ldo;
        p.M = (int)M; p.N = N; p.K = K;
        p.splits = 1;
        p.KS = K <= 2048 ? K / 256 : 8;
        p.act = -1; p.ln_kind = -1;
        const int tiles = (N + 15) / 16;
        p.G = tiles >= 4 * d->num_cu ? 4 : 1;
      };
      // Every buffer a phase writes is touched with device-scope accesses only for the whole launch (x too, which
      // phase 0 reads as its residual and phase 3 rewrites): an ordinary load would leave a line in this XCD's L2
      // that a later phase could read stale.
      ChainPhase &po = c.ph[0];                       // x1 = x + attn . Wo^T (+ bo)
      lin(po, d->attn, QD, false, ly.Wo_f, H, QD, x1, H);
      po.bias = ly.bo; po.residual = x; po.ldr = H; po.res_fresh = 1;
      ChainPhase &pg = c.ph[1];                       // glu = act(gate(norm2(x1))) * up(norm2(x1))
      lin(pg, x1, H, true, ly.Wgu_f, 2 * I, H, d->glu, I);
      pg.ln_kind = kind; pg.ln_w = ly.n2_w; pg.ln_eps = (float)d->cfg.norm_eps;
      pg.act = d->cfg.hidden_act; pg.glu = 1;
      ChainPhase &pd = c.ph[2];                       // partial products of down over spans of 2048 of K
      lin(pd, d->glu, I, true, ly.Wdown_f, H, I, x, H);
      pd.splits = down_splits; pd.partial = (float *)d->splitk_ws;
      pd.G = (H / 16) >= 4 * (d->num_cu / down_splits) ? 4 : 1;
      ChainPhase &ps = c.ph[3];                       // x = x1 + sum of the partial products
      ps.kind = RAI_CHAIN_SUM;
      ps.partial = (float *)d->splitk_ws; ps.splits = down_splits;
      ps.residual = x1; ps.ldr = H; ps.res_fresh = 1;
      ps.out = x; ps.ldo = H;
      ps.M = (int)M; ps.N = H; ps.act = -1;
      c.n = 4;
      if (l + 1 < d->L) {                             // the next layer's q|k|v behind its input norm
        const Layer &nx = d->layers[l + 1];
        ChainPhase &pq = c.ph[4];
        lin(pq, x, H, true, nx.Wqkv_f, ldq, H, d->qkv, ldq);
        pq.bias = nx.bqkv;
        pq.ln_kind = kind; pq.ln_w = nx.n1_w; pq.ln_eps = (float)d->cfg.norm_eps;
        c.n = 5;
      }
      c.flags = d->state->chain_flags;
      c.epoch = &d->state->epoch;   // advanced by the token choice that ends every step
      c.launch = l;
      c.fault = kernel_fault_word(d->dev);
      c.spin_limit = 1 << 20;
      if (const char *e = getenv("RAI_HIP_CHAIN_SPIN_LIMIT")) {   // failure-path test hook (read per launch)
        const int lim = atoi(e);
        if (lim > 0) c.spin_limit = lim;
      }
      RAI_TRY(launch_decode_chain(st, c, d->dev));
      continue;
    }

    LinearArgs o = linear_args_default();
    o.A = d->attn; o.lda = QD;
    o.W = ly.Wo; o.ldw = QD; o.bias = ly.bo;
    o.Wfrag = frag ? ly.Wo_f : nullptr;
    o.residual = x; o.ldr = H;
    o.out1 = x1; o.ld1 = H;
    o.M = (int)M; o.N = H; o.K = QD; o.n_split = H;
    o.splitk_ws = d->splitk_ws; o.splitk_ws_bytes = d->splitk_ws_bytes;
    RAI_TRY(linear(d, st, o));

    LinearArgs g = linear_args_default();
    g.splitk_ws = d->splitk_ws; g.splitk_ws_bytes = d->splitk_ws_bytes;
    if (fuse_norm) {
      g.A = x1; g.lda = H;
      g.ln_kind = kind; g.ln_w = ly.n2_w; g.ln_eps = (float)d->cfg.norm_eps;
    } else {
      RAI_TRY(norm_rows(x1, ly.n2_w, d->ln, M, H));
      g.A = d->ln; g.lda = H;
    }
    g.W = ly.Wgu; g.ldw = H;
    g.Wfrag = frag ? ly.Wgu_f : nullptr;
    g.out1 = d->glu; g.ld1 = I;
    g.M = (int)M; g.N = 2 * I; g.K = H; g.n_split = 2 * I;
    g.act = d->cfg.hidden_act; g.act_from = 0; g.glu = 1;
    RAI_TRY(linear(d, st, g));

    LinearArgs dn = linear_args_default();
    dn.A = d->glu; dn.lda = I;
    dn.W = ly.Wdown; dn.ldw = I;
    dn.Wfrag = frag ? ly.Wdown_f : nullptr;
    dn.residual = x1; dn.ldr = H;
    dn.out1 = x; dn.ld1 = H;
    dn.M = (int)M; dn.N = H; dn.K = I; dn.n_split = H;
    dn.splitk_ws = d->splitk_ws; dn.splitk_ws_bytes = d->splitk_ws_bytes;
    RAI_TRY(linear(d, st, dn));
  }

  if (d->want_hidden) RAI_HIP_TRY(hipMemcpyAsync(d->hidden_copy, x, (size_t)M * H * d->es, hipMemcpyDeviceToDevice, st));
  // last position -> final norm -> lm_head (qwen2.rs:355-357, gemma.rs:383-385)
  LinearArgs h = linear_args_default();
  char *last_rows = x + (size_t)(S - 1) * H * d->es;
  if (dt == RAI_BF16 && (B <= 8 || linear_mfma_fuses_norm(B, H, kind))) {
    h.A = last_rows; h.lda = (int64_t)S * H;
    h.ln_kind = kind; h.ln_w = d->lnf_w; h.ln_eps = (float)d->cfg.norm_eps;
  } else {
    RAI_TRY(norm_rows(last_rows, d->lnf_w, d->last, B, (int64_t)S * H));
    h.A = d->last; h.lda = H;
  }
  h.W = d->head_w; h.ldw = H;
  if (wants_fragments(d, B)) {
    RAI_TRY(ensure_fragments(d, st));
    h.Wfrag = d->head_f;
  }
  h.out1 = d->logits; h.ld1 = d->V;
  h.M = B; h.N = d->V; h.K = H; h.n_split = d->V;
  RAI_TRY(linear(d, st, h));

  RAI_TRY(launch_token_choice(d, st, B, S, advance_step));
  d->ctx_len = T_after;
  return RAI_OK;
}

static int forward_any(rai_hip_decoder *d, int B, int S, bool advance_step, bool from_tokens = false) {
  return d->cfg.arch == RAI_ARCH_PHI2 ? forward_phi2(d, B, S, advance_step, from_tokens)
                                       : forward_seq(d, B, S, advance_step, from_tokens);
}

// A packet poll of the persistent decode kernel that timed out leaves
// DevState::fault set; the results of that step are not valid.
static int check_fault(rai_hip_decoder *d) {
  RAI_TRY(check_kernel_fault(d->dev));
  if (!d->mega_ok) return RAI_OK;
  DevState hs;
  RAI_TRY(rai_hip_d2h(d->dev, &hs, d->state, sizeof(hs)));
  if (d->mega_prof) {  // phase timings of the last token: mean over layers, for three blocks
    std::vector<unsigned long long> t((size_t)d->num_cu * d->L * 16);
    RAI_HIP_TRY(hipMemcpy(t.data(), d->mega_prof, t.size() * 8, hipMemcpyDeviceToHost));
    const int blocks[4] = {0, d->Hq - 1, d->Hq, d->num_cu - 1};
    auto at = [&](int b, int l, int k) { return (double)t[((size_t)b * d->L + l) * 16 + k] * 0.01; };
    for (int bi = 0; bi < 4; ++bi) {
      double iv[7] = {0, 0, 0, 0, 0, 0, 0};
      const int b = blocks[bi];
      for (int l = 0; l < d->L; ++l)
        for (int k = 0; k < 7; ++k) iv[k] += (at(b, l, k + 1) - at(b, l, k)) / d->L;
      double ex[6] = {0, 0, 0, 0, 0, 0};   // stamps 8, 9 relative to the layer's start, 10..13 to the end of phase A
      for (int l = 0; l < d->L; ++l)
        for (int k = 0; k < 6; ++k) ex[k] += (at(b, l, 8 + k) - at(b, l, k < 2 ? 0 : 1)) / d->L;
      fprintf(stderr, "mega prof block %3d: A %.2f (x arrived +%.2f, q|k|v published +%.2f) | sync %.2f | poll (attention) %.2f | Wb stream %.2f + sync %.2f | publish x %.2f | sync %.2f us\n",
              b, iv[0], ex[0], ex[1], iv[1], iv[2], iv[3], iv[4], iv[5], iv[6]);
      if (b < d->Hq)
        fprintf(stderr, "mega prof block %3d: after A: +%.2f qkv polled | +%.2f k partials | +%.2f softmax | +%.2f attn published\n",
                b, ex[2], ex[3], ex[4], ex[5]);
    }
  }
  if (d->mega_prof) {   // the exchange of the residual stream: from the last block's publication to a block's arrival
    std::vector<unsigned long long> t((size_t)d->num_cu * d->L * 16);
    RAI_HIP_TRY(hipMemcpy(t.data(), d->mega_prof, t.size() * 8, hipMemcpyDeviceToHost));
    auto at = [&](int b, int l, int k) { return (double)t[((size_t)b * d->L + l) * 16 + k] * 0.01; };
    double lat_min = 0, lat_mean = 0, lat_max = 0, spread = 0, behind_median = 0;
    for (int l = 1; l < d->L; ++l) {
      std::vector<double> pub(d->num_cu), arr(d->num_cu);
      for (int b = 0; b < d->num_cu; ++b) { pub[b] = at(b, l - 1, 6); arr[b] = at(b, l, 8); }
      const double last = *std::max_element(pub.begin(), pub.end());
      std::vector<double> sorted = pub;
      std::sort(sorted.begin(), sorted.end());
      spread += (last - sorted.front()) / (d->L - 1);
      behind_median += (last - sorted[sorted.size() / 2]) / (d->L - 1);
      double mn = 1e30, mx = -1e30, sum = 0;
      for (int b = 0; b < d->num_cu; ++b) { const double v = arr[b] - last; mn = v < mn ? v : mn; mx = v > mx ? v : mx; sum += v; }
      lat_min += mn / (d->L - 1); lat_max += mx / (d->L - 1); lat_mean += sum / d->num_cu / (d->L - 1);
    }
    fprintf(stderr, "mega prof x exchange: the last block publishes %.2f us after the first and %.2f us after the median one; "
                    "from that publication to the arrival at a block: min %.2f, mean %.2f, max %.2f us\n",
            spread, behind_median, lat_min, lat_mean, lat_max);
  }
  if (d->mega_prof && getenv("RAI_HIP_MEGA_PROF_SKEW")) {  // how late each block reaches the end of each phase, mean over layers
    std::vector<unsigned long long> t((size_t)d->num_cu * d->L * 16);
    RAI_HIP_TRY(hipMemcpy(t.data(), d->mega_prof, t.size() * 8, hipMemcpyDeviceToHost));
    auto at = [&](int b, int l, int k) { return (double)t[((size_t)b * d->L + l) * 16 + k] * 0.01; };
    const int stamps[3] = {1, 4, 6};
    for (int k = 0; k < 3; ++k) {
      std::vector<double> late(d->num_cu, 0.0);
      for (int l = 0; l < d->L; ++l) {
        double mn = 1e30;
        for (int b = 0; b < d->num_cu; ++b) mn = at(b, l, stamps[k]) < mn ? at(b, l, stamps[k]) : mn;
        for (int b = 0; b < d->num_cu; ++b) late[b] += (at(b, l, stamps[k]) - mn) / d->L;
      }
      fprintf(stderr, "mega skew phase %c:", "ABC"[k]);
      for (int b = 0; b < d->num_cu; ++b) fprintf(stderr, " %.1f", late[b]);
      fprintf(stderr, "\n");
    }
  }
  if (hs.fault == 0) return RAI_OK;
  hs.fault = 0;
  RAI_HIP_TRY(hipMemcpy(&d->state->fault, &hs.fault, sizeof(int), hipMemcpyHostToDevice));
  return fail(RAI_ERR_HIP, "decoder: an exchange of the persistent decode kernel timed out");
}

static int check_call(rai_hip_decoder *d, int B, int S) {
  RAI_REQUIRE(d, RAI_ERR_BAD_ARG, "decoder is null");
  RAI_REQUIRE(B >= 1 && B <= d->cfg.max_batch, RAI_ERR_BAD_SHAPE, "decoder: batch %d outside 1..%d", B, d->cfg.max_batch);
  RAI_REQUIRE(S >= 1, RAI_ERR_BAD_SHAPE, "decoder: empty sequence");
  RAI_REQUIRE(d->ctx_len + S <= d->cfg.max_context, RAI_ERR_BAD_SHAPE, "decoder: context %d + %d exceeds max_context %d",
              d->ctx_len, S, d->cfg.max_context);
  RAI_REQUIRE(d->ctx_len + S <= d->cfg.max_position_embeddings, RAI_ERR_BAD_SHAPE,
              "decoder: position exceeds max_position_embeddings");
  for (const ParamSlot &s : d->slots)
    RAI_REQUIRE(s.loaded, RAI_ERR_BAD_ARG, "decoder: parameter %s was never loaded", s.name.c_str());
  return RAI_OK;
}

}  // namespace rai

extern "C" {

int rai_hip_decoder_create(int dev, const rai_hip_decoder_config *cfg, rai_hip_decoder **out) {
  RAI_REQUIRE(cfg && out, RAI_ERR_BAD_ARG, "decoder_create: null argument");
  RAI_REQUIRE(cfg->arch == RAI_ARCH_PHI2 || cfg->arch == RAI_ARCH_QWEN2 || cfg->arch == RAI_ARCH_GEMMA ||
                  cfg->arch == RAI_ARCH_PHI3,
              RAI_ERR_UNSUPPORTED, "decoder_create: architecture %d not available", cfg->arch);
  RAI_REQUIRE(cfg->dtype == RAI_BF16 || cfg->dtype == RAI_F32, RAI_ERR_BAD_DTYPE, "decoder_create: bf16 or f32");
  RAI_REQUIRE(cfg->hidden_size > 0 && cfg->num_attention_heads > 0 && cfg->num_key_value_heads > 0 &&
                  cfg->num_attention_heads % cfg->num_key_value_heads == 0 && cfg->head_dim > 0 &&
                  cfg->vocab_size > 0 && cfg->intermediate_size > 0 && cfg->num_hidden_layers > 0 &&
                  cfg->max_batch > 0 && cfg->max_context > 0 && cfg->max_position_embeddings > 0,
              RAI_ERR_BAD_ARG, "decoder_create: bad config");
  RAI_REQUIRE(cfg->rotary_dim > 0 && cfg->rotary_dim % 2 == 0 && cfg->rotary_dim <= cfg->head_dim, RAI_ERR_BAD_ARG,
              "decoder_create: rotary_dim %d", cfg->rotary_dim);
  RAI_REQUIRE(cfg->hidden_act == RAI_UN_NEW_GELU || cfg->hidden_act == RAI_UN_GELU || cfg->hidden_act == RAI_UN_SILU ||
                  cfg->hidden_act == RAI_UN_RELU,
              RAI_ERR_BAD_ARG, "decoder_create: hidden_act %d", cfg->hidden_act);
  RAI_REQUIRE(!cfg->qk_layernorm, RAI_ERR_UNSUPPORTED,
              "decoder_create: qk_layernorm (rai-models/src/llm/phi2.rs:207-216) is not implemented by the decoder drivers");
  if (!ctx(dev)) return RAI_ERR_HIP;
  rai_hip_decoder *d = new rai_hip_decoder();
  d->dev = dev;
  d->cfg = *cfg;
  d->es = dtype_size(cfg->dtype);
  d->H = cfg->hidden_size; d->I = cfg->intermediate_size; d->D = cfg->head_dim;
  d->Hq = cfg->num_attention_heads; d->Hkv = cfg->num_key_value_heads;
  d->QD = d->Hq * d->D; d->KD = d->Hkv * d->D; d->V = cfg->vocab_size; d->L = cfg->num_hidden_layers;
  d->NA = d->QD + 2 * d->KD + d->I;
  d->KB = d->QD + d->I;
  d->ctx_len = 0;
  d->step_graph = nullptr;
  d->step_graph_n = nullptr;
  d->step_graph_batch = 0;
  d->x_holds_next = false;
  d->sample_on = false; d->sample_penalty = 0.f; d->sample_last_n = 0;
  d->token_log = nullptr; d->token_log_cap = 0;
  d->graph_sampled = false; d->graph_penalty = 0.f; d->graph_last_n = 0;
  d->head_f = nullptr; d->frag_ready = false;
  d->hidden_copy = nullptr; d->want_hidden = false;
  d->choice_val = nullptr; d->choice_idx = nullptr; d->head_best = nullptr;
  const int vec = (int)(16 / d->es);
  int st = RAI_OK;
  auto bail = [&](int code) {
    rai_hip_decoder_destroy(d);
    return code;
  };
  if (d->H % vec || d->QD % vec || d->KD % vec || d->I % vec || d->D % vec)
    return bail(fail(RAI_ERR_BAD_SHAPE, "decoder_create: sizes must be multiples of %d elements", vec));
  d->embed_scale = 1.0f;
  if (cfg->arch == RAI_ARCH_GEMMA) d->embed_scale = round_dt((float)sqrt((double)d->H), cfg->dtype);
  if ((st = (cfg->arch == RAI_ARCH_PHI2 ? create_phi2(d) : create_seq(d))) != RAI_OK) return bail(st);
  const size_t es = d->es;
  d->max_rows = (int64_t)cfg->max_batch * cfg->max_context;
  const size_t kv = (size_t)d->L * cfg->max_batch * d->Hkv * cfg->max_context * d->D * es;
  const size_t rope = (size_t)cfg->max_position_embeddings * cfg->rotary_dim * es;
  d->history_cap = cfg->max_context;
  char *tmp = nullptr;
  if ((st = dalloc(d, kv, &d->kcache)) || (st = dalloc(d, kv, &d->vcache)) || (st = dalloc(d, rope, &d->cos_t)) ||
      (st = dalloc(d, rope, &d->sin_t)) || (st = dalloc(d, d->max_rows * d->H * es, &d->x)) ||
      (st = dalloc(d, d->max_rows * d->H * es, &d->x2)) || (st = dalloc(d, d->max_rows * d->H * es, &d->ln)) ||
      (st = dalloc(d, d->max_rows * (d->QD + 2 * d->KD) * es, &d->qkv)) ||
      (st = dalloc(d, cfg->arch == RAI_ARCH_PHI2 ? d->max_rows * d->KB * es : 16, &d->cat)) ||
      (st = dalloc(d, cfg->arch == RAI_ARCH_PHI2 ? 16 : d->max_rows * d->QD * es, &d->attn)) ||
      (st = dalloc(d, cfg->arch == RAI_ARCH_PHI2 ? 16 : d->max_rows * d->I * es, &d->glu)) || (st = dalloc(d, (size_t)cfg->max_batch * d->H * es, &d->last)) ||
      (st = dalloc(d, (size_t)cfg->max_batch * d->V * es, &d->logits)))
    return bail(st);
  if ((st = dalloc(d, d->max_rows * sizeof(uint32_t), &tmp))) return bail(st);
  d->ids = (uint32_t *)tmp;
  if ((st = dalloc(d, (size_t)cfg->max_batch * sizeof(uint32_t), &tmp))) return bail(st);
  d->tokens = (uint32_t *)tmp;
  if ((st = dalloc(d, (size_t)d->history_cap * cfg->max_batch * sizeof(uint32_t), &tmp))) return bail(st);
  d->history = (uint32_t *)tmp;
  d->token_log_cap = cfg->max_context + 1;
  if ((st = dalloc(d, (size_t)d->token_log_cap * cfg->max_batch * sizeof(uint32_t), &tmp))) return bail(st);
  d->token_log = (uint32_t *)tmp;
  if ((st = dalloc(d, sizeof(DevState), &tmp))) return bail(st);
  d->state = (DevState *)tmp;
  d->splitk_ws_bytes = (size_t)12 * d->max_rows * d->H * sizeof(float);
  if (d->splitk_ws_bytes > ((size_t)256 << 20)) d->splitk_ws_bytes = (size_t)256 << 20;
  // the stream-K form of the tile kernel (prefill products of 136 tiles and more) parks partial tiles here
  if (cfg->dtype == RAI_BF16 && d->max_rows >= 256 && d->splitk_ws_bytes < ((size_t)192 << 20))
    d->splitk_ws_bytes = (size_t)192 << 20;
  if ((st = dalloc(d, d->splitk_ws_bytes, &d->splitk_ws))) return bail(st);
  if ((st = dalloc(d, attention_decode_ws_bytes(cfg->max_batch, d->Hq, d->D), &d->attn_ws))) return bail(st);
  if ((st = dalloc(d, attention_decode_counter_bytes(cfg->max_batch, d->Hq), &tmp))) return bail(st);
  d->attn_counters = (int *)tmp;
  if ((st = dalloc(d, (size_t)cfg->max_batch * kChoiceMaxSplits * sizeof(float), &tmp))) return bail(st);
  d->choice_val = (float *)tmp;
  if ((st = dalloc(d, (size_t)cfg->max_batch * kChoiceMaxSplits * sizeof(uint32_t), &tmp))) return bail(st);
  d->choice_idx = (uint32_t *)tmp;
  if ((st = dalloc(d, 256 * sizeof(unsigned long long), &tmp))) return bail(st);
  d->head_best = (unsigned long long *)tmp;
  if (hipMemset(d->attn_counters, 0, attention_decode_counter_bytes(cfg->max_batch, d->Hq)) != hipSuccess)
    return bail(fail(RAI_ERR_HIP, "decoder_create: memset failed"));

  d->mega_layers = nullptr;
  d->mega_ok = false;
  d->mega_prof = nullptr;
  {
    hipDeviceProp_t prop;
    d->num_cu = hipGetDeviceProperties(&prop, dev) == hipSuccess ? prop.multiProcessorCount : kNumCU;
  }
  d->mega_xchg = nullptr;
  if (cfg->arch == RAI_ARCH_PHI2 && cfg->dtype == RAI_BF16 && getenv("RAI_HIP_NO_MEGA") == nullptr) {
    {  // zeroed: tag 0 is never a valid exchange tag
      // x and q|k|v: two values to a packet; activations: 16 packets for each of up to 256 producers;
      // attention output: ceil(D / 3) packets per head
      const size_t packets = (size_t)(d->H + d->QD + 2 * d->KD) / 2 + kMegaActPackets + (size_t)d->Hq * ((d->D + 2) / 3) + 8;
      if ((st = dalloc(d, packets * sizeof(uint64_t), &tmp))) return bail(st);
      d->mega_xchg = (uint64_t *)tmp;
      if (hipMemset(d->mega_xchg, 0, packets * sizeof(uint64_t)) != hipSuccess)
        return bail(fail(RAI_ERR_HIP, "decoder_create: memset failed"));
    }
    std::vector<MegaLayer> ml(d->L);
    for (int l = 0; l < d->L; ++l) {
      const Layer &ly = d->layers[l];
      ml[l] = MegaLayer{(const uint16_t *)ly.Wa, (const uint16_t *)ly.ba, (const uint16_t *)ly.Wb, (const uint16_t *)ly.bd,
                        (const uint16_t *)ly.bf, (const uint16_t *)ly.ln_w, (const uint16_t *)ly.ln_b};
    }
    if ((st = dalloc(d, ml.size() * sizeof(MegaLayer), &tmp))) return bail(st);
    d->mega_layers = (MegaLayer *)tmp;
    if (hipMemcpy(d->mega_layers, ml.data(), ml.size() * sizeof(MegaLayer), hipMemcpyHostToDevice) != hipSuccess)
      return bail(fail(RAI_ERR_HIP, "decoder_create: layer table upload failed"));
    if (getenv("RAI_HIP_MEGA_PROF")) {
      if ((st = dalloc(d, (size_t)d->num_cu * d->L * 16 * sizeof(unsigned long long), &tmp))) return bail(st);
      d->mega_prof = (unsigned long long *)tmp;
    }
    MegaArgs m = mega_args(d);
    d->mega_ok = mega_eligible(m, d->D, d->num_cu, nullptr);
  }
  if (hipMemset(d->state, 0, sizeof(DevState)) != hipSuccess || hipMemset(d->kcache, 0, kv) != hipSuccess ||
      hipMemset(d->vcache, 0, kv) != hipSuccess)
    return bail(fail(RAI_ERR_HIP, "decoder_create: memset failed"));
  if ((st = build_rope_tables(d)) != RAI_OK) return bail(st);
  *out = d;
  return RAI_OK;
}

int rai_hip_decoder_destroy(rai_hip_decoder *d) {
  if (!d) return RAI_OK;
  (void)hipSetDevice(d->dev);
  (void)hipStreamSynchronize(stream_of(d->dev));
  if (d->step_graph) (void)hipGraphExecDestroy(d->step_graph);
  if (d->step_graph_n) (void)hipGraphExecDestroy(d->step_graph_n);
  for (void *p : d->allocs) (void)hipFree(p);
  delete d;
  return RAI_OK;
}

int rai_hip_decoder_param_count(rai_hip_decoder *d, int32_t *count) {
  RAI_REQUIRE(d && count, RAI_ERR_BAD_ARG, "null argument");
  *count = (int32_t)d->slots.size();
  return RAI_OK;
}

int rai_hip_decoder_param_name(rai_hip_decoder *d, int32_t i, char *buf, size_t buflen, int64_t *numel) {
  RAI_REQUIRE(d && buf && buflen > 0, RAI_ERR_BAD_ARG, "null argument");
  RAI_REQUIRE(i >= 0 && i < (int32_t)d->slots.size(), RAI_ERR_BAD_ARG, "parameter index %d out of range", i);
  snprintf(buf, buflen, "%s", d->slots[i].name.c_str());
  if (numel) *numel = d->slots[i].rows * d->slots[i].cols;
  return RAI_OK;
}

int rai_hip_decoder_param_shape(rai_hip_decoder *d, int32_t i, int64_t *rows, int64_t *cols) {
  RAI_REQUIRE(d && rows && cols, RAI_ERR_BAD_ARG, "null argument");
  RAI_REQUIRE(i >= 0 && i < (int32_t)d->slots.size(), RAI_ERR_BAD_ARG, "parameter index %d out of range", i);
  *rows = d->slots[i].rows;
  *cols = d->slots[i].cols;
  return RAI_OK;
}

int rai_hip_decoder_load_param(rai_hip_decoder *d, const char *name, const void *host_data, size_t bytes) {
  RAI_REQUIRE(d && name && host_data, RAI_ERR_BAD_ARG, "null argument");
  auto it = d->slot_by_name.find(name);
  RAI_REQUIRE(it != d->slot_by_name.end(), RAI_ERR_BAD_ARG, "decoder: unknown parameter '%s'", name);
  ParamSlot &s = d->slots[it->second];
  const size_t want = (size_t)s.rows * s.cols * d->es;
  RAI_REQUIRE(bytes == want, RAI_ERR_BAD_SHAPE, "decoder: parameter '%s' needs %zu bytes, got %zu", name, want, bytes);
  RAI_HIP_TRY(hipSetDevice(d->dev));
  RAI_HIP_TRY(hipStreamSynchronize(stream_of(d->dev)));
  const size_t row_bytes = (size_t)s.cols * d->es, rows1 = (size_t)(s.rows - s.rows2);
  RAI_HIP_TRY(hipMemcpy2D(s.dst, (size_t)s.pitch * d->es, host_data, row_bytes, row_bytes, rows1, hipMemcpyHostToDevice));
  if (s.rows2 > 0)
    RAI_HIP_TRY(hipMemcpy2D(s.dst2, (size_t)s.pitch * d->es, (const char *)host_data + rows1 * row_bytes, row_bytes, row_bytes,
                            (size_t)s.rows2, hipMemcpyHostToDevice));
  s.loaded = true;
  d->frag_ready = false;   // the fragment-order copies are rebuilt on the next batched decode step
  return RAI_OK;
}

int rai_hip_decoder_dtype(rai_hip_decoder *d, int32_t *dtype) {
  RAI_REQUIRE(d && dtype, RAI_ERR_BAD_ARG, "null argument");
  *dtype = d->cfg.dtype;
  return RAI_OK;
}

int rai_hip_decoder_clear_kv_cache(rai_hip_decoder *d) {
  RAI_REQUIRE(d, RAI_ERR_BAD_ARG, "decoder is null");
  hipStream_t st = stream_of(d->dev);
  hipLaunchKernelGGL(k_set_state, dim3(1), dim3(1), 0, st, d->state, 0, 0);
  RAI_TRY(launch_check("set_state"));
  d->ctx_len = 0;
  return RAI_OK;
}

int rai_hip_decoder_context_len(rai_hip_decoder *d, int32_t *len) {
  RAI_REQUIRE(d && len, RAI_ERR_BAD_ARG, "null argument");
  *len = d->ctx_len;
  return RAI_OK;
}

static int widen_to_host(rai_hip_decoder *d, hipStream_t st, const char *src, int64_t n, float *dst_host) {
  void *ws = nullptr;
  RAI_TRY(workspace(d->dev, (size_t)n * sizeof(float), &ws));
  if (d->cfg.dtype == RAI_BF16)
    hipLaunchKernelGGL((k_to_f32<bf16_raw>), dim3(grid1d(n)), dim3(256), 0, st, (float *)ws, (const bf16_raw *)src, n);
  else
    hipLaunchKernelGGL((k_to_f32<float>), dim3(grid1d(n)), dim3(256), 0, st, (float *)ws, (const float *)src, n);
  RAI_TRY(launch_check("to_f32"));
  return rai_hip_d2h(d->dev, dst_host, ws, (size_t)n * sizeof(float));
}

int rai_hip_decoder_forward_hidden(rai_hip_decoder *d, const uint32_t *ids_host, const void *hidden_in_host, int32_t batch,
                                   int32_t seq, float *hidden_out_host, float *logits_host, uint32_t *tokens_host) {
  RAI_REQUIRE((ids_host != nullptr) != (hidden_in_host != nullptr), RAI_ERR_BAD_ARG,
              "forward_hidden: give either token ids or input rows");
  RAI_TRY(check_call(d, batch, seq));
  hipStream_t st = stream_of(d->dev);
  const size_t rows_bytes = (size_t)batch * seq * d->H * d->es;
  if (hidden_out_host && !d->hidden_copy) RAI_TRY(dalloc(d, (size_t)d->max_rows * d->H * d->es, &d->hidden_copy));
  if (ids_host) {
    RAI_HIP_TRY(hipMemcpyAsync(d->ids, ids_host, (size_t)batch * seq * sizeof(uint32_t), hipMemcpyHostToDevice, st));
  } else {
    RAI_HIP_TRY(hipMemcpyAsync(d->x, hidden_in_host, rows_bytes, hipMemcpyHostToDevice, st));
    RAI_HIP_TRY(hipStreamSynchronize(st));   // the caller's buffer is free again when this returns
  }
  d->want_hidden = hidden_out_host != nullptr;
  const int rc = forward_any(d, batch, seq, false, hidden_in_host != nullptr);
  d->want_hidden = false;
  d->x_holds_next = false;
  RAI_TRY(rc);
  if (hidden_out_host) RAI_TRY(widen_to_host(d, st, d->hidden_copy, (int64_t)batch * seq * d->H, hidden_out_host));
  if (logits_host) RAI_TRY(widen_to_host(d, st, d->logits, (int64_t)batch * d->V, logits_host));
  if (tokens_host) RAI_TRY(rai_hip_d2h(d->dev, tokens_host, d->tokens, (size_t)batch * sizeof(uint32_t)));
  if (hidden_out_host || logits_host || tokens_host) {
    RAI_TRY(check_fault(d));
    uint64_t bad = 0;
    RAI_TRY(rai_hip_index_errors(d->dev, &bad));
    RAI_REQUIRE(bad == 0, RAI_ERR_INDEX, "decoder: %llu token ids outside the vocabulary", (unsigned long long)bad);
  }
  return RAI_OK;
}

int rai_hip_decoder_forward(rai_hip_decoder *d, const uint32_t *ids_host, int32_t batch, int32_t seq, float *logits_host,
                            uint32_t *tokens_host) {
  RAI_REQUIRE(ids_host, RAI_ERR_BAD_ARG, "ids is null");
  RAI_TRY(check_call(d, batch, seq));
  hipStream_t st = stream_of(d->dev);
  RAI_HIP_TRY(hipMemcpyAsync(d->ids, ids_host, (size_t)batch * seq * sizeof(uint32_t), hipMemcpyHostToDevice, st));
  RAI_TRY(forward_any(d, batch, seq, false));
  if (logits_host) {
    // widen on device, then one synchronous copy
    void *ws = nullptr;
    const int64_t n = (int64_t)batch * d->V;
    RAI_TRY(workspace(d->dev, (size_t)n * sizeof(float), &ws));
    if (d->cfg.dtype == RAI_BF16)
      hipLaunchKernelGGL((k_to_f32<bf16_raw>), dim3(grid1d(n)), dim3(256), 0, st, (float *)ws, (const bf16_raw *)d->logits, n);
    else
      hipLaunchKernelGGL((k_to_f32<float>), dim3(grid1d(n)), dim3(256), 0, st, (float *)ws, (const float *)d->logits, n);
    RAI_TRY(launch_check("to_f32"));
    RAI_TRY(rai_hip_d2h(d->dev, logits_host, ws, (size_t)n * sizeof(float)));
  }
  if (tokens_host) RAI_TRY(rai_hip_d2h(d->dev, tokens_host, d->tokens, (size_t)batch * sizeof(uint32_t)));
  if (logits_host || tokens_host) {
    RAI_TRY(check_fault(d));
    uint64_t bad = 0;
    RAI_TRY(rai_hip_index_errors(d->dev, &bad));
    RAI_REQUIRE(bad == 0, RAI_ERR_INDEX, "decoder: %llu token ids outside the vocabulary", (unsigned long long)bad);
  }
  return RAI_OK;
}

// The loop of both generate entry points; d->sample_on selects the token choice.
static int generate_impl(rai_hip_decoder *d, const uint32_t *prompt_host, int32_t batch, int32_t prompt_len,
                         int32_t n_new, uint32_t *tokens_host, float *prefill_ms, float *decode_ms) {
  RAI_REQUIRE(prompt_host && tokens_host, RAI_ERR_BAD_ARG, "null argument");
  RAI_REQUIRE(n_new >= 1, RAI_ERR_BAD_ARG, "generate: n_new must be >= 1");
  RAI_TRY(rai_hip_decoder_clear_kv_cache(d));
  RAI_TRY(check_call(d, batch, prompt_len));
  RAI_REQUIRE(prompt_len + n_new - 1 <= d->cfg.max_context && n_new <= d->history_cap, RAI_ERR_BAD_SHAPE,
              "generate: %d + %d tokens exceed max_context %d", prompt_len, n_new, d->cfg.max_context);
  hipStream_t st = stream_of(d->dev);
  if (d->sample_on)   // the token log starts as the prompt, one row per sequence
    RAI_HIP_TRY(hipMemcpy2DAsync(d->token_log, (size_t)d->token_log_cap * sizeof(uint32_t), prompt_host,
                                 (size_t)prompt_len * sizeof(uint32_t), (size_t)prompt_len * sizeof(uint32_t), batch,
                                 hipMemcpyHostToDevice, st));
  hipEvent_t e0, e1, e2;
  RAI_HIP_TRY(hipEventCreate(&e0));
  RAI_HIP_TRY(hipEventCreate(&e1));
  RAI_HIP_TRY(hipEventCreate(&e2));
  RAI_HIP_TRY(hipMemcpyAsync(d->ids, prompt_host, (size_t)batch * prompt_len * sizeof(uint32_t), hipMemcpyHostToDevice, st));
  RAI_HIP_TRY(hipStreamSynchronize(st));
  RAI_HIP_TRY(hipEventRecord(e0, st));
  int rc = forward_any(d, batch, prompt_len, true);
  if (rc == RAI_OK) rc = hipEventRecord(e1, st) == hipSuccess ? RAI_OK : fail(RAI_ERR_HIP, "event record");
  // Single-token steps: the previous step left the next input embedding, the
  // token and the advanced context length on the device, so every step is the
  // same sequence of launches.  The first step runs eagerly (it also performs
  // any one-time kernel attribute set-up); the rest replay captured hipGraphs,
  // kGraphSteps steps per launch while that many remain, then one step per launch.
  const bool use_graph = d->cfg.dtype == RAI_BF16 && getenv("RAI_HIP_NO_GRAPH") == nullptr;
  // Captures `steps` consecutive single-token steps (they read their inputs from device state, so the
  // recorded launches are identical for every step) into an executable graph.
  auto capture = [&](int steps, hipGraphExec_t *exec) -> int {
    hipGraph_t g = nullptr;
    const int ctx0 = d->ctx_len;
    if (hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal) != hipSuccess)
      return fail(RAI_ERR_HIP, "generate: begin capture failed");
    int frc = RAI_OK;
    for (int i = 0; i < steps && frc == RAI_OK; ++i) frc = forward_any(d, batch, 1, true, true);
    hipError_t ce = hipStreamEndCapture(st, &g);
    d->ctx_len = ctx0;  // capture only recorded the steps; they have not run
    if (frc != RAI_OK) { if (g) (void)hipGraphDestroy(g); return frc; }
    if (ce != hipSuccess || !g) return fail(RAI_ERR_HIP, "generate: end capture failed: %s", hipGetErrorString(ce));
    hipError_t ie = hipGraphInstantiate(exec, g, nullptr, nullptr, 0);
    (void)hipGraphDestroy(g);
    if (ie != hipSuccess) { *exec = nullptr; return fail(RAI_ERR_HIP, "generate: graph instantiate: %s", hipGetErrorString(ie)); }
    return RAI_OK;
  };
  int step = 1;
  if (rc == RAI_OK && step < n_new) {  // first step eagerly: one-time kernel attribute set-up happens outside capture
    rc = forward_any(d, batch, 1, true, true);
    ++step;
  }
  // the recorded launches bake in the batch and the token choice with its parameters
  const bool same_choice = d->graph_sampled == d->sample_on &&
                           (!d->sample_on || (d->graph_penalty == d->sample_penalty && d->graph_last_n == d->sample_last_n));
  if (rc == RAI_OK && use_graph && (d->step_graph_batch != batch || !same_choice)) {
    if (d->step_graph) { (void)hipGraphExecDestroy(d->step_graph); d->step_graph = nullptr; }
    if (d->step_graph_n) { (void)hipGraphExecDestroy(d->step_graph_n); d->step_graph_n = nullptr; }
    d->step_graph_batch = batch;
    d->graph_sampled = d->sample_on; d->graph_penalty = d->sample_penalty; d->graph_last_n = d->sample_last_n;
  }
  while (rc == RAI_OK && step < n_new) {
    const int left = n_new - step;
    if (!use_graph) {
      rc = forward_any(d, batch, 1, true, true);
      ++step;
      continue;
    }
    if (left >= kGraphSteps) {   // the gap between two graph launches is paid once per kGraphSteps tokens
      if (!d->step_graph_n) { rc = capture(kGraphSteps, &d->step_graph_n); if (rc != RAI_OK) break; }
      if (hipGraphLaunch(d->step_graph_n, st) != hipSuccess) { rc = fail(RAI_ERR_HIP, "generate: graph launch failed"); break; }
      d->ctx_len += kGraphSteps;
      step += kGraphSteps;
    } else {
      if (!d->step_graph) { rc = capture(1, &d->step_graph); if (rc != RAI_OK) break; }
      if (hipGraphLaunch(d->step_graph, st) != hipSuccess) { rc = fail(RAI_ERR_HIP, "generate: graph launch failed"); break; }
      d->ctx_len += 1;
      ++step;
    }
  }
  if (rc == RAI_OK && hipEventRecord(e2, st) != hipSuccess) rc = fail(RAI_ERR_HIP, "event record");
  if (rc == RAI_OK && hipStreamSynchronize(st) != hipSuccess) rc = fail(RAI_ERR_HIP, "generate: stream sync failed");
  if (rc == RAI_OK) {
    float ms = 0.f;
    if (prefill_ms) { (void)hipEventElapsedTime(&ms, e0, e1); *prefill_ms = ms; }
    if (decode_ms) { (void)hipEventElapsedTime(&ms, e1, e2); *decode_ms = ms; }
    // history is [step][batch]; hand back [batch][step]
    std::vector<uint32_t> h((size_t)n_new * batch);
    rc = rai_hip_d2h(d->dev, h.data(), d->history, h.size() * sizeof(uint32_t));
    for (int s = 0; rc == RAI_OK && s < n_new; ++s)
      for (int b = 0; b < batch; ++b) tokens_host[(size_t)b * n_new + s] = h[(size_t)s * batch + b];
  }
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  (void)hipEventDestroy(e2);
  if (rc == RAI_OK) {
    RAI_TRY(check_fault(d));
    uint64_t bad = 0;
    RAI_TRY(rai_hip_index_errors(d->dev, &bad));
    RAI_REQUIRE(bad == 0, RAI_ERR_INDEX, "decoder: %llu token ids outside the vocabulary", (unsigned long long)bad);
  }
  return rc;
}

int rai_hip_sample_argmax(int dev, const rai_hip_tensor *logits, const rai_hip_tensor *context, float repeat_penalty,
                          const rai_hip_tensor *out) {
  RAI_TRY(validate(logits, "logits"));
  RAI_TRY(validate(out, "out"));
  RAI_REQUIRE(logits->rank == 2 && is_contiguous(logits), RAI_ERR_BAD_SHAPE, "sample_argmax: logits must be contiguous [rows, vocab]");
  RAI_REQUIRE(logits->dtype == RAI_F32 || logits->dtype == RAI_BF16, RAI_ERR_BAD_DTYPE, "sample_argmax: logits dtype %s",
              dtype_name(logits->dtype));
  const int64_t rows = logits->shape[0], V = logits->shape[1];
  RAI_REQUIRE(V >= 1 && V <= kSampleMaxVocab, RAI_ERR_BAD_SHAPE, "sample_argmax: vocabulary %lld outside 1..%lld", (long long)V,
              (long long)kSampleMaxVocab);
  RAI_REQUIRE(out->dtype == RAI_U32 && out->rank == 1 && out->shape[0] == rows && is_contiguous(out), RAI_ERR_BAD_SHAPE,
              "sample_argmax: out must be contiguous u32 [rows]");
  RAI_REQUIRE(repeat_penalty == repeat_penalty, RAI_ERR_BAD_ARG, "sample_argmax: repeat_penalty is NaN");
  int n_ctx = 0;
  const uint32_t *ctx = nullptr;
  if (context) {
    RAI_TRY(validate(context, "context"));
    RAI_REQUIRE(context->dtype == RAI_U32 && context->rank == 2 && context->shape[0] == rows && is_contiguous(context),
                RAI_ERR_BAD_SHAPE, "sample_argmax: context must be contiguous u32 [rows, n]");
    RAI_REQUIRE(context->shape[1] <= (1 << 20), RAI_ERR_BAD_SHAPE, "sample_argmax: context too long");
    n_ctx = (int)context->shape[1];
    ctx = (const uint32_t *)base_ptr(context);
  }
  if (rows == 0) return RAI_OK;
  hipStream_t st = stream_of(dev);
  if (!st) return RAI_ERR_HIP;
  const size_t lds = (size_t)((V + 31) / 32) * sizeof(uint32_t);
  if (logits->dtype == RAI_BF16)
    hipLaunchKernelGGL((k_sample_rows<bf16_raw>), dim3((unsigned)rows), dim3(1024), lds, st, (const bf16_raw *)base_ptr(logits),
                       V, ctx, n_ctx, repeat_penalty, (uint32_t *)base_ptr(out));
  else
    hipLaunchKernelGGL((k_sample_rows<float>), dim3((unsigned)rows), dim3(1024), lds, st, (const float *)base_ptr(logits), V,
                       ctx, n_ctx, repeat_penalty, (uint32_t *)base_ptr(out));
  return launch_check("sample_rows");
}

int rai_hip_decoder_generate(rai_hip_decoder *d, const uint32_t *prompt_host, int32_t batch, int32_t prompt_len,
                             int32_t n_new, uint32_t *tokens_host, float *prefill_ms, float *decode_ms) {
  RAI_REQUIRE(d, RAI_ERR_BAD_ARG, "decoder is null");
  d->sample_on = false;
  return generate_impl(d, prompt_host, batch, prompt_len, n_new, tokens_host, prefill_ms, decode_ms);
}

int rai_hip_decoder_generate_sampled(rai_hip_decoder *d, const uint32_t *prompt_host, int32_t batch, int32_t prompt_len,
                                     int32_t n_new, float repeat_penalty, int32_t repeat_last_n, int64_t eos_token,
                                     uint32_t *tokens_host, int32_t *n_generated, float *prefill_ms, float *decode_ms) {
  RAI_REQUIRE(d, RAI_ERR_BAD_ARG, "decoder is null");
  RAI_REQUIRE(repeat_last_n >= 0, RAI_ERR_BAD_ARG, "generate_sampled: repeat_last_n must be >= 0");
  RAI_REQUIRE(repeat_penalty == repeat_penalty, RAI_ERR_BAD_ARG, "generate_sampled: repeat_penalty is NaN");
  RAI_REQUIRE(d->V <= kSampleMaxVocab, RAI_ERR_UNSUPPORTED, "generate_sampled: vocabulary %d above %lld", d->V,
              (long long)kSampleMaxVocab);
  d->sample_on = true;
  d->sample_penalty = repeat_penalty;
  d->sample_last_n = repeat_last_n;
  const int rc = generate_impl(d, prompt_host, batch, prompt_len, n_new, tokens_host, prefill_ms, decode_ms);
  d->sample_on = false;
  RAI_TRY(rc);
  // the example loop stops after it has pushed the end-of-text token (main.rs:83-86): report how many tokens
  // of each row it would have produced; the entries behind them are what a loop without the stop generates
  for (int b = 0; n_generated && b < batch; ++b) {
    int n = n_new;
    for (int s = 0; eos_token >= 0 && s < n_new; ++s)
      if ((int64_t)tokens_host[(size_t)b * n_new + s] == eos_token) { n = s + 1; break; }
    n_generated[b] = n;
  }
  return RAI_OK;
}

int rai_hip_decoder_time_decode_step(rai_hip_decoder *d, int32_t sweeps, float *us_per_launch,
                                     double *bytes_per_launch) {
  RAI_REQUIRE(d && us_per_launch && bytes_per_launch && sweeps > 0, RAI_ERR_BAD_ARG, "bad argument");
  RAI_REQUIRE(d->mega_ok, RAI_ERR_UNSUPPORTED, "time_decode_step: the persistent decode kernel does not serve this model");
  RAI_REQUIRE(d->ctx_len >= 1 && d->ctx_len < d->cfg.max_context, RAI_ERR_BAD_SHAPE,
              "time_decode_step: needs a context of 1..%d tokens", d->cfg.max_context - 1);
  hipStream_t st = stream_of(d->dev);
  hipEvent_t e0, e1;
  RAI_HIP_TRY(hipEventCreate(&e0));
  RAI_HIP_TRY(hipEventCreate(&e1));
  const MegaArgs m = mega_args(d);
  double total_ms = 0.0;
  int rc = RAI_OK;
  for (int s = 0; s < sweeps + 2 && rc == RAI_OK; ++s) {  // two warm-up launches
    if (hipEventRecord(e0, st) != hipSuccess) { rc = fail(RAI_ERR_HIP, "event record"); break; }
    rc = launch_phi2_decode_step(st, m, d->D, d->num_cu);
    if (rc != RAI_OK) break;
    if (hipEventRecord(e1, st) != hipSuccess) { rc = fail(RAI_ERR_HIP, "time_decode_step: launch failed"); break; }
    hipLaunchKernelGGL(k_next_epoch, dim3(1), dim3(1), 0, st, d->state);
    if (hipEventSynchronize(e1) != hipSuccess) { rc = fail(RAI_ERR_HIP, "time_decode_step: launch failed"); break; }
    float ms = 0.f;
    (void)hipEventElapsedTime(&ms, e0, e1);
    if (s >= 2) total_ms += ms;
  }
  (void)hipStreamSynchronize(st);
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  RAI_TRY(rc);
  RAI_TRY(check_fault(d));
  *us_per_launch = (float)(total_ms * 1000.0 / sweeps);
  // algorithmic bytes of one launch: every layer's weights, biases and LayerNorm parameters once, plus the
  // cached keys and values of the current context
  const double es = (double)d->es;
  const double per_layer = (double)d->NA * d->H + d->NA + (double)d->H * d->KB + 2.0 * d->H + 2.0 * d->H;
  const double kv = 2.0 * d->Hkv * d->D * (double)d->ctx_len;
  *bytes_per_launch = es * d->L * (per_layer + kv);
  return RAI_OK;
}

int rai_hip_decoder_time_decode_linear(rai_hip_decoder *d, int32_t sweeps, float *us_per_launch,
                                       double *bytes_per_launch) {
  RAI_REQUIRE(d && us_per_launch && bytes_per_launch && sweeps > 0, RAI_ERR_BAD_ARG, "bad argument");
  RAI_REQUIRE(d->cfg.dtype == RAI_BF16 && d->cfg.arch == RAI_ARCH_PHI2, RAI_ERR_UNSUPPORTED,
              "time_decode_linear: bf16 Phi-2 models only");
  hipStream_t st = stream_of(d->dev);
  hipEvent_t e0, e1;
  RAI_HIP_TRY(hipEventCreate(&e0));
  RAI_HIP_TRY(hipEventCreate(&e1));
  const int H = d->H, ldq = d->QD + 2 * d->KD;
  auto sweep = [&]() -> int {
    for (int l = 0; l < d->L; ++l) {
      const Layer &ly = d->layers[l];
      LinearArgs a = linear_args_default();
      a.A = d->x; a.lda = H;
      a.ln_kind = 0; a.ln_w = ly.ln_w; a.ln_b = ly.ln_b; a.ln_eps = (float)d->cfg.norm_eps;
      a.W = ly.Wa; a.ldw = H; a.bias = ly.ba;
      a.out1 = d->qkv; a.ld1 = ldq;
      a.out2 = d->cat + (size_t)d->QD * d->es; a.ld2 = d->KB;
      a.M = 1; a.N = d->NA; a.K = H; a.n_split = ldq;
      a.act = d->cfg.hidden_act; a.act_from = ldq;
      RAI_TRY(launch_linear_bf16(st, a));
      LinearArgs b = linear_args_default();
      b.A = d->cat; b.lda = d->KB;
      b.W = ly.Wb; b.ldw = d->KB;
      b.bias = ly.bd; b.bias2 = ly.bf;
      b.residual = d->x; b.ldr = H;
      b.out1 = d->x2; b.ld1 = H;
      b.M = 1; b.N = H; b.K = d->KB; b.n_split = H;
      RAI_TRY(launch_linear_bf16(st, b));
    }
    return RAI_OK;
  };
  RAI_TRY(sweep());  // warm-up
  RAI_HIP_TRY(hipEventRecord(e0, st));
  for (int s = 0; s < sweeps; ++s) RAI_TRY(sweep());
  RAI_HIP_TRY(hipEventRecord(e1, st));
  RAI_HIP_TRY(hipEventSynchronize(e1));
  float ms = 0.f;
  RAI_HIP_TRY(hipEventElapsedTime(&ms, e0, e1));
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  *us_per_launch = ms * 1000.0f / (float)(2 * d->L * sweeps);
  const double es = (double)d->es;
  const double bytes_a = ((double)d->NA * H + d->NA + 3.0 * H + d->NA) * es;          // W, bias, x + ln w/b, out
  const double bytes_b = ((double)H * d->KB + 2.0 * H + d->KB + H + H) * es;          // W, 2 biases, in, residual, out
  *bytes_per_launch = 0.5 * (bytes_a + bytes_b);
  return RAI_OK;
}

}  // extern "C"
