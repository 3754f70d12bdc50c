// Internal launcher of the attention kernels (shared by the C ABI and the
// decoder drivers).
#pragma once
#include "common.h"

namespace rai {

// q[B, Hq, S, D], k/v[B, Hkv, T, D] with unit stride on D; out[B, S, Hq*D].
// Query row s of a length-S block sits at absolute position T - S + s, so with
// causal != 0 it sees keys 0 .. T - S + s.
struct AttnArgs {
  const void *q, *k, *v;
  void *out;
  int64_t qs[3], ks[3], vs[3];  // element strides of dims B, H, S/T
  int64_t out_row_stride;       // elements between consecutive (b, s) rows of out
  int B, Hq, Hkv, S, T, D;
  float scale;
  int causal;
  int f32_scores;  // 1: phi2.rs:244-260 numerics; 0: qwen2.rs:205-216 / gemma.rs:238-254
  int dtype;       // RAI_BF16 / RAI_F16 / RAI_F32
  // When t_dev is non-null the key count is read on the device (*t_dev + t_add)
  // instead of T, so one captured launch serves every decode step; T is then
  // the capacity bound.
  const int *t_dev;
  int t_add;
};

int launch_attention(hipStream_t st, const AttnArgs &a);

// One new token per sequence (decode): rotary embedding of q and of the new k,
// append of k/v to the cache, and attention over the cache plus the new token,
// in one launch.  qkv rows are [q (Hq*D) | k (Hkv*D) | v (Hkv*D)], not yet rotated.
struct AttnDecodeArgs {
  const void *qkv;
  void *kcache, *vcache;  // this layer's [B][Hkv][Tmax][D]
  void *out;
  int64_t out_row_stride;
  const void *cos_t, *sin_t;  // [max_pos, rot] in the model dtype
  const int *pos_dev;         // tokens already in the cache (device memory); null: pos_host
  int pos_host;
  // The new token's key and value rows as tensors of their own ([B][Hkv*D], element strides between sequences
  // below) instead of behind the queries in one packed row; qkv then holds the queries alone.  Null: packed.
  const void *k_new, *v_new;
  int64_t q_row_stride, k_row_stride, v_row_stride;
  int rot;
  int B, Hq, Hkv, D, Tmax;
  float scale;
  int f32_scores;
  int dtype;
  // Partial results of the context splits: ws holds attention_decode_ws_bytes()
  // bytes, counters attention_decode_counter_bytes() bytes that are zero between launches.
  float *ws;
  int *counters;
  int ns, chunk_cap;  // filled in by the launcher
};
size_t attention_decode_ws_bytes(int B, int Hq, int D);
size_t attention_decode_counter_bytes(int B, int Hq);
int launch_attention_decode(hipStream_t st, const AttnDecodeArgs &a);

}  // namespace rai
