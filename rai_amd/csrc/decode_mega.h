// Launcher of the persistent per-token decode kernel (Phi-2 architecture,
// batch 1, bf16) and the device-side decode state shared with the decoder
// drivers.
#pragma once
#include "common.h"

namespace rai {

constexpr int kMegaActPackets = 256 * 16;   // slots of the activation packets: 16 for each of up to 256 producer blocks

struct DevState {
  int pos;    // tokens already in the KV cache
  int step;   // greedy steps taken by the current generate call
  int done;   // blocks of the token-selection kernel that have finished (reset by the last one)
  int fault;  // set by a packet poll that timed out; checked by the host after a generate call
  unsigned epoch;  // launches of the persistent decode kernel so far: makes its exchange tags unique
  // Arrival flags of the decode chain kernel's barriers (decode_chain.h), one per block: a block announces barrier
  // number n of the decoder's life by storing n, and n only grows (epoch * 4096 + launch * 8 + phase), so nothing is
  // ever reset.
  unsigned long long chain_flags[512];
};

struct MegaLayer {
  const uint16_t *Wa, *ba;            // [NA, H] rows q | k | v | fc1, and their biases
  const uint16_t *Wb, *bd, *bf;       // [H, QD + I] row n = dense[n, :] | fc2[n, :], and both biases
  const uint16_t *ln_w, *ln_b;
};

struct MegaArgs {
  const MegaLayer *layers;  // device array [L]
  const uint16_t *Wa0, *Wb0;      // layer 0; layer l sits wa_stride / wb_stride elements further
  int64_t wa_stride, wb_stride;
  int L, H, I, QD, NA, n_qkv, Hq, Hkv, rot, Tmax;   // Hkv < Hq: Hq / Hkv query heads share a key/value head
  uint16_t *x;              // [H] residual stream, updated in place
  // Vectors exchanged between blocks inside the launch, as 8-byte packets: {two bf16 values, 32-bit tag} for xp and
  // qkvp, {three bf16 values, 16-bit tag in the top bits} for actp and attnp.  A packet is valid for an exchange when
  // its tag is (the low bits of) epoch * 1024 + exchange index + 1.
  uint64_t *xp;             // [H / 2]      residual stream after a layer
  uint64_t *qkvp;           // [(QD + 2 * Hkv * D) / 2]
  uint64_t *actp;           // [kMegaActPackets] gelu(fc1), three values to a packet, 16 packets per producer block
  uint64_t *attnp;          // [Hq * ceil(D / 3)] attention output, three values to a packet
  uint16_t *kcache, *vcache;
  int64_t kv_layer_stride;  // elements between consecutive layers of the cache
  const uint16_t *cos_t, *sin_t;
  DevState *state;
  float ln_eps, scale;
  int act;
  int rows_attn;            // rows of phases B/C given to each attention block
  int stage_off;            // byte offset in LDS of the weight staging area (set by the launcher; 0 = none fits)
  unsigned long long *prof; // optional [blocks][L][16] time stamps (debugging aid), or null
  // Failure-path test hooks, honoured only by the instrumented build of the kernel (prof != null):
  unsigned spin_limit;      // polling rounds after which a wait gives up and raises DevState::fault
  int mute_block;           // this block sends no phase-A packets, so its consumers time out; -1 = none
};

// The head of the same decoder behind the persistent step: final LayerNorm, the vocabulary product and the greedy
// choice in one launch (k_phi2_head_choice, one block per CU, the weight stream of the step kernel).
struct HeadArgs {
  const uint16_t *W, *bias;       // [V, H] and [V] (bias may be null)
  const uint16_t *x;              // [H] residual stream after the last layer
  const uint16_t *ln_w, *ln_b;
  float ln_eps;
  int V, H;
  uint16_t *logits;               // [V], written as the product is rounded
  unsigned long long *best;       // one (value bits << 32 | row) per block, exchanged inside the launch
  uint32_t *token, *history;      // history may be null; history[state->step] otherwise
  DevState *state;                // done is the arrival counter (zero between launches); pos, step, epoch are advanced
  int dpos, dstep;
  const uint16_t *embed;          // [V, H]: row `token` times embed_scale becomes x_next (the next step's input)
  uint16_t *x_next;
  float embed_scale;
};
bool head_choice_eligible(const HeadArgs &a, int num_cu);
int launch_phi2_head_choice(hipStream_t st, const HeadArgs &a, int num_cu);

unsigned mega_default_spin_limit();
bool mega_eligible(const MegaArgs &a, int D, int num_cu, const char **why);
int launch_phi2_decode_step(hipStream_t st, const MegaArgs &a, int D, int num_cu);

}  // namespace rai
