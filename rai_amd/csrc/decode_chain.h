// A chain of small-M Linears as one persistent launch: the part of a batched decode step (9..32 rows) of a
// sequential-block decoder (rai-models/src/llm/qwen2.rs:253-266, gemma.rs:286-299) that lies between two attention
// calls.  Internal launcher, shared with the decoder drivers.
#pragma once
#include "common.h"

namespace rai {

enum { RAI_CHAIN_LINEAR = 0, RAI_CHAIN_SUM = 1 };

// One phase.  RAI_CHAIN_LINEAR: out[m, n] = epilogue(sum_k norm(A)[m, k] * W[n, k]) as LinearArgs describes it, with
// the weights in fragment order (linear_fragment_elems) and K either whole (splits == 1) or cut into `splits` spans
// of 256 * KS columns whose f32 products go to partial[split][M][N].  RAI_CHAIN_SUM: out = residual + the sum of
// `splits` partial products, in split order.  The `*_fresh` flags say that the operand was written by an earlier
// phase of the same launch: it is then read past the (per-XCD, mutually incoherent) L2s.
struct ChainPhase {
  int kind;
  const void *A;
  int64_t lda;
  int a_fresh;
  const void *Wfrag;
  const void *bias;
  const void *residual;
  int64_t ldr;
  int res_fresh;
  void *out;
  int64_t ldo;
  float *partial;
  int M, N, K;
  int splits, G, KS;   // G: 16-row weight tiles per group (1 or 4); KS: 32-column steps per wave (6 or 8)
  int act, glu;
  const void *ln_w;
  float ln_eps;
  int ln_kind;         // -1 none, 1 rmsnorm, 2 rmsnorm (1 + w)
};

constexpr int kChainMaxPhases = 6;
struct ChainArgs {
  ChainPhase ph[kChainMaxPhases];
  int n;
  // Grid barrier between phases without read-modify-write traffic: block b announces that it has finished phase i by
  // storing the barrier's number, (*epoch << 12) + launch * 8 + i + 1, to flags[b], and waits until all of flags[0 ..
  // grid) have reached that number (every thread polls one flag).  *epoch grows by one per decode step (the token
  // choice advances it) and `launch` numbers the chain launches of a step, so the numbers only ever grow and nothing
  // needs resetting.  A wait is bounded (spin_limit polls): on expiry RAI_FAULT_CHAIN goes to the device's fault
  // word and every later wait falls through, so that all waves still exit.
  unsigned long long *flags;
  const unsigned *epoch;
  int launch;
  int *fault;
  int spin_limit;
};

// Whether the chain kernel serves a Linear of this shape (bf16, fragment-order weights present).
bool decode_chain_serves(int M, int N, int K, bool k_split);
int launch_decode_chain(hipStream_t st, const ChainArgs &a, int dev);

}  // namespace rai
