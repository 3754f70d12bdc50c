// Scaled-dot-product attention.
//   k_attn_row: one 256-thread block per (query row, head, batch).  K and V of the
//   head are streamed once per block with 16-byte loads; scores live in LDS as
//   f32.  This is the decode kernel (S == 1: HBM-bound on the KV cache) and the
//   dtype-generic fallback for short prefills.
//
// Reference semantics: rai-models/src/llm/phi2.rs:244-262 (f32 scores, -inf mask,
// f32 softmax, P cast to V's dtype), qwen2.rs:205-221 and gemma.rs:238-254
// (scores, scale and softmax rounded to the model dtype), repeat_kv
// gemma.rs:191-201 (query head h reads kv head h / (Hq/Hkv)).
#include <cstdlib>

#include "attention.h"

namespace rai {

template <typename T> struct AttnVec;
template <> struct AttnVec<float> { static constexpr int V = 4; };
template <> struct AttnVec<bf16_raw> { static constexpr int V = 8; };
template <> struct AttnVec<f16_raw> { static constexpr int V = 8; };
template <typename T, int V> struct alignas(sizeof(T) * V) APack { T v[V]; };

template <typename T> __device__ __forceinline__ float round_to(float x) {
  T t;
  Scalar<T>::store(&t, x);
  return (float)Scalar<T>::load(&t);
}
template <> __device__ __forceinline__ float round_to<float>(float x) { return x; }

template <typename T>
__global__ void __launch_bounds__(256) k_attn_row(AttnArgs a) {
  constexpr int V = AttnVec<T>::V;
  extern __shared__ __attribute__((aligned(16))) float smem[];
  // layout: q[D] | red[groups*D] | scores[T]
  const int D = a.D, ncol = D / V;
  const int groups = 256 / ncol;
  float *qf = smem;
  float *red = qf + D;
  float *scores = red + groups * D;
  __shared__ float sh[8];

  const int s = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int hk = h / (a.Hq / a.Hkv);
  int n_keys = a.T;
  if (a.t_dev) {
    n_keys = *a.t_dev + a.t_add;
    if (n_keys > a.T) n_keys = a.T;
  }
  int t_end = a.causal ? (n_keys - a.S + s + 1) : n_keys;
  if (t_end > n_keys) t_end = n_keys;
  if (t_end < 0) t_end = 0;

  const T *q = (const T *)a.q + b * a.qs[0] + h * a.qs[1] + s * a.qs[2];
  const T *K = (const T *)a.k + b * a.ks[0] + hk * a.ks[1];
  const T *Vp = (const T *)a.v + b * a.vs[0] + hk * a.vs[1];
  for (int d = tid; d < D; d += 256) qf[d] = (float)Scalar<T>::load(q + d);
  __syncthreads();

  // ---- scores: 16 lanes cooperate on one key row
  {
    const int g = tid >> 4, gl = tid & 15;
    for (int t = g; t < t_end; t += 16) {
      const T *kr = K + (int64_t)t * a.ks[2];
      float acc = 0.f;
      for (int c = gl; c < ncol; c += 16) {
        APack<T, V> pk = *reinterpret_cast<const APack<T, V> *>(kr + c * V);
#pragma unroll
        for (int j = 0; j < V; ++j) acc = fmaf(qf[c * V + j], (float)Scalar<T>::load(&pk.v[j]), acc);
      }
      acc += __shfl_xor(acc, 8, 64);
      acc += __shfl_xor(acc, 4, 64);
      acc += __shfl_xor(acc, 2, 64);
      acc += __shfl_xor(acc, 1, 64);
      if (gl == 0) {
        float sc;
        if (a.f32_scores) sc = acc * a.scale;
        else sc = round_to<T>(round_to<T>(acc) * round_to<T>(a.scale));
        scores[t] = sc;
      }
    }
  }
  __syncthreads();

  // ---- softmax over scores[0..t_end)
  float m = -INFINITY;
  for (int t = tid; t < t_end; t += 256) m = fmaxf(m, scores[t]);
  m = wave_max(m);
  if (lane == 0) sh[wave] = m;
  __syncthreads();
  m = fmaxf(fmaxf(sh[0], sh[1]), fmaxf(sh[2], sh[3]));
  float sum = 0.f;
  for (int t = tid; t < t_end; t += 256) {
    float e = expf(scores[t] - m);
    if (!a.f32_scores) e = round_to<T>(e);
    scores[t] = e;
    sum += e;
  }
  sum = wave_sum(sum);
  if (lane == 0) sh[4 + wave] = sum;
  __syncthreads();
  sum = sh[4] + sh[5] + sh[6] + sh[7];
  if (!a.f32_scores) sum = round_to<T>(sum);
  const float inv = 1.0f / sum;

  // ---- P.V: thread (grp, col) accumulates keys grp, grp+groups, ... for V
  //      consecutive output features
  {
    const int col = tid % ncol, grp = tid / ncol;
    float acc[V];
#pragma unroll
    for (int j = 0; j < V; ++j) acc[j] = 0.f;
    if (grp < groups) {
      for (int t = grp; t < t_end; t += groups) {
        // the reference rounds the normalised probabilities to V's dtype
        const float p = a.f32_scores ? round_to<T>(scores[t] * inv) : round_to<T>(scores[t] / sum);
        APack<T, V> pk = *reinterpret_cast<const APack<T, V> *>(Vp + (int64_t)t * a.vs[2] + col * V);
#pragma unroll
        for (int j = 0; j < V; ++j) acc[j] = fmaf(p, (float)Scalar<T>::load(&pk.v[j]), acc[j]);
      }
#pragma unroll
      for (int j = 0; j < V; ++j) red[grp * D + col * V + j] = acc[j];
    }
  }
  __syncthreads();
  T *o = (T *)a.out + ((int64_t)b * a.S + s) * a.out_row_stride + (int64_t)h * D;
  for (int d = tid; d < D; d += 256) {
    float r = 0.f;
    for (int g = 0; g < groups; ++g) r += red[g * D + d];
    Scalar<T>::store(o + d, (typename Scalar<T>::compute)r);
  }
}

// Rotary embedding of feature d of one head for position pos, with the
// reference's three roundings (x*cos, rotate_half(x)*sin, their sum:
// rai-models/src/llm/phi2.rs:75).
template <typename T>
__device__ __forceinline__ float rope_feature(const T *head, int d, int rot, const T *cos_t, const T *sin_t, int pos) {
  float v = (float)Scalar<T>::load(head + d);
  if (d >= rot) return v;
  const int half = rot >> 1;
  float other = d < half ? -(float)Scalar<T>::load(head + d + half) : (float)Scalar<T>::load(head + d - half);
  float c = (float)Scalar<T>::load(cos_t + (int64_t)pos * rot + d);
  float s = (float)Scalar<T>::load(sin_t + (int64_t)pos * rot + d);
  return round_to<T>(round_to<T>(v * c) + round_to<T>(other * s));
}

// Decode attention, split over the context ("flash decoding"): block
// (split, kv-head group, batch) handles ceil((pos+1)/NS) consecutive keys for
// the R query heads that share one KV head, so the cached K and V are read once
// per KV head (repeat_kv is never materialised) and NS * Hkv * B blocks keep
// every CU busy even at batch 1.  All of a block's first K and V loads are
// issued before anything is computed: a short context costs one HBM round trip.
// Each block writes an unnormalised partial (running max m, sum l, o[D]) per
// query head; the last block of a head group to finish (device-scope counter)
// merges the NS partials and writes the output row.  The new token's rotated
// key and value are appended to the cache by the block that owns position pos
// and are used from LDS.  Probabilities stay in f32 until the product with V.
constexpr int kDecodeThreads = 256;
constexpr int kDecodeMaxSplits = 64;
constexpr int kDecodeCounterStride = 32;

// Device-scope accesses for data handed from one block to another inside a
// kernel.  The L2 of each XCD is not coherent with the others for ordinary
// accesses, and a device-scope fence writes back and invalidates a whole L2;
// relaxed device-scope atomics instead write through / read around the L2 for
// just the words involved.
__device__ __forceinline__ void store_device(float *p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_device(const float *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Tail of a decode-attention block: once its partials are written, the block
// counts itself in; the last block of the head group to arrive merges the NS
// partials of the R query heads starting at hq0 and writes their output rows.
// wbuf is block-shared scratch of 2 * R * NS floats that no wave uses any more.
// The merge is a chain of dependent memory round trips, so it is kept short: one
// for all (m, l) statistics, then the per-split weights exp(m_s - M) / L are
// computed once per head, and every thread has 64 partial-output loads in flight.
template <typename T>
__device__ __forceinline__ void decode_merge_last(const AttnDecodeArgs &a, int b, int hq0, int R, int *sh_last,
                                                  float *wbuf) {
  constexpr int NT = kDecodeThreads;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, NS = a.ns, D = a.D, PW = D + 2;
  // every thread's write-through stores have completed before the block's arrival is counted
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  int *counter = a.counters + ((int64_t)b * a.Hq + hq0) * kDecodeCounterStride;  // one 128-byte line each
  if (tid == 0) *sh_last = atomicAdd(counter, 1) == NS - 1;
  __syncthreads();
  if (!*sh_last) return;
  const float *all = a.ws + ((int64_t)b * a.Hq + hq0) * NS * PW;
  float *wm = wbuf, *wl = wbuf + R * NS;
  for (int i = tid; i < R * NS; i += NT) {
    const float *st = all + (int64_t)i * PW;   // (head r, split s) at index r*NS + s
    wm[i] = load_device(st);
    wl[i] = load_device(st + 1);
  }
  __syncthreads();
  for (int r = wave; r < R; r += NT / 64) {      // NS <= 64: one split per lane
    const float m = lane < NS ? wm[r * NS + lane] : -INFINITY;
    const float M = wave_max(m);                 // split 0 always holds a key, so M is finite
    const float e = lane < NS ? expf(m - M) : 0.f;  // an empty split has m = -inf: weight 0
    const float L = wave_sum(lane < NS ? e * wl[r * NS + lane] : 0.f);
    if (lane < NS) wm[r * NS + lane] = e / L;
  }
  __syncthreads();
  constexpr int EU = 8, SB = 8;
  for (int e0 = tid; e0 < R * D; e0 += NT * EU) {
    const float *po[EU];
    int hr[EU], hd[EU];
    float O[EU];
#pragma unroll
    for (int i = 0; i < EU; ++i) {
      const int e = e0 + i * NT < R * D ? e0 + i * NT : e0;
      hr[i] = e / D;
      hd[i] = e - hr[i] * D;
      po[i] = all + (int64_t)hr[i] * NS * PW + 2 + hd[i];
      O[i] = 0.f;
    }
    for (int s0 = 0; s0 < NS; s0 += SB) {
      float ov[EU][SB];
#pragma unroll
      for (int i = 0; i < EU; ++i)
#pragma unroll
        for (int j = 0; j < SB; ++j) ov[i][j] = load_device(po[i] + (s0 + j < NS ? s0 + j : NS - 1) * PW);
#pragma unroll
      for (int i = 0; i < EU; ++i)
#pragma unroll
        for (int j = 0; j < SB; ++j)
          if (s0 + j < NS) O[i] = fmaf(wm[hr[i] * NS + s0 + j], ov[i][j], O[i]);
    }
#pragma unroll
    for (int i = 0; i < EU; ++i)
      if (e0 + i * NT < R * D)
        Scalar<T>::store((T *)a.out + (int64_t)b * a.out_row_stride + (int64_t)(hq0 + hr[i]) * D + hd[i],
                         (typename Scalar<T>::compute)O[i]);
  }
  if (tid == 0) *counter = 0;  // ready for the next launch (stream order)
}

template <typename T, int R, int CC, int UK, int UV>
__global__ void __launch_bounds__(kDecodeThreads) k_attn_decode_split(AttnDecodeArgs a) {
  constexpr int V = AttnVec<T>::V;
  constexpr int NT = kDecodeThreads, NW = NT / 64;
  extern __shared__ __attribute__((aligned(16))) float smem[];
  const int D = a.D, ncol = D / V, groups = NT / ncol;
  const int NS = a.ns, CH = a.chunk_cap;
  // layout: q[R*D] | knew[D] | vnew[D] | scores[R*CH] | red[groups*R*D]
  float *qf = smem;
  float *knew = qf + R * D;
  float *vnew = knew + D;
  float *scores = vnew + D;
  float *red = scores + R * CH;
  __shared__ float sh_m[R], sh_l[R];
  __shared__ int sh_last;

  const int s = blockIdx.x, b = blockIdx.z;
  const int hq0 = blockIdx.y * R;           // first query head of this block
  const int n_rep = a.Hq / a.Hkv, hk = hq0 / n_rep;
  const bool writer = hq0 % n_rep == 0;     // one block per KV head appends the new token
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int pos = a.pos_dev ? *a.pos_dev : a.pos_host;
  if (pos > a.Tmax - 1) pos = a.Tmax - 1;   // capacity is checked on the host; never write past the cache
  const int cnt = pos + 1;
  int chunk = (cnt + NS - 1) / NS;
  if (chunk > CH) chunk = CH;
  const int t0 = s * chunk;
  const int t1 = t0 + chunk < cnt ? t0 + chunk : cnt;
  const int n = t1 > t0 ? t1 - t0 : 0;      // keys of this split (the new token included when it falls inside)
  const bool has_new = pos >= t0 && pos < t1;
  const int t1c = has_new ? pos : t1;       // cached keys are [t0, t1c)

  const int QD = a.Hq * D, KD = a.Hkv * D;
  // the new token's rows: one packed [q | k | v] row per sequence, or three separate ones
  const T *qrow = (const T *)a.qkv + (int64_t)b * (a.k_new ? a.q_row_stride : (int64_t)(QD + 2 * KD));
  const T *krow = a.k_new ? (const T *)a.k_new + (int64_t)b * a.k_row_stride : qrow + QD;
  const T *vrow = a.k_new ? (const T *)a.v_new + (int64_t)b * a.v_row_stride : qrow + QD + KD;
  T *Kc = (T *)a.kcache + ((int64_t)b * a.Hkv + hk) * a.Tmax * D;
  T *Vc = (T *)a.vcache + ((int64_t)b * a.Hkv + hk) * a.Tmax * D;
  const T *cos_t = (const T *)a.cos_t, *sin_t = (const T *)a.sin_t;
  const int g = tid >> 4, gl = tid & 15;
  const int col = tid % ncol, grp = tid / ncol;

  // ---- first round of K and V loads
  APack<T, V> kreg[UK][CC], vreg[UV];
#pragma unroll
  for (int u = 0; u < UK; ++u) {
    const int t = t0 + g + 16 * u;
#pragma unroll
    for (int cc = 0; cc < CC; ++cc) {
      const int c = gl + 16 * cc;
      if (t < t1c && c < ncol) kreg[u][cc] = *reinterpret_cast<const APack<T, V> *>(Kc + (int64_t)t * D + c * V);
    }
  }
#pragma unroll
  for (int u = 0; u < UV; ++u) {
    const int t = t0 + grp + u * groups;
    if (grp < groups && t < t1c) vreg[u] = *reinterpret_cast<const APack<T, V> *>(Vc + (int64_t)t * D + col * V);
  }
  // ---- rotary embedding of the R query rows (and of the new key where it is needed)
  for (int e = tid; e < R * D; e += NT) {
    const int r = e / D, d = e - r * D;
    qf[e] = rope_feature<T>(qrow + (hq0 + r) * D, d, a.rot, cos_t, sin_t, pos);
  }
  if (has_new) {
    for (int d = tid; d < D; d += NT) {
      const float kr = rope_feature<T>(krow + hk * D, d, a.rot, cos_t, sin_t, pos);
      const float vr = (float)Scalar<T>::load(vrow + hk * D + d);
      knew[d] = kr;
      vnew[d] = vr;
      if (writer) {
        Scalar<T>::store(Kc + (int64_t)pos * D + d, (typename Scalar<T>::compute)kr);
        Scalar<T>::store(Vc + (int64_t)pos * D + d, (typename Scalar<T>::compute)vr);
      }
    }
  }
  __syncthreads();

  auto finish_score = [&](float acc) -> float {
    if (a.f32_scores) return acc * a.scale;
    return round_to<T>(round_to<T>(acc) * round_to<T>(a.scale));
  };
  // ---- scores against the cached keys: 16 lanes per key row, round 0 from the prefetched registers
  for (int tb = t0 + g; tb < t1c; tb += 16 * UK) {
    if (tb != t0 + g) {
#pragma unroll
      for (int u = 0; u < UK; ++u) {
        const int t = tb + 16 * u;
#pragma unroll
        for (int cc = 0; cc < CC; ++cc) {
          const int c = gl + 16 * cc;
          if (t < t1c && c < ncol) kreg[u][cc] = *reinterpret_cast<const APack<T, V> *>(Kc + (int64_t)t * D + c * V);
        }
      }
    }
#pragma unroll
    for (int u = 0; u < UK; ++u) {
      const int t = tb + 16 * u;
      float kf[CC][V];
#pragma unroll
      for (int cc = 0; cc < CC; ++cc)
#pragma unroll
        for (int j = 0; j < V; ++j) kf[cc][j] = (float)Scalar<T>::load(&kreg[u][cc].v[j]);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        float acc = 0.f;
#pragma unroll
        for (int cc = 0; cc < CC; ++cc) {
          const int c = gl + 16 * cc;
          if (t < t1c && c < ncol) {
#pragma unroll
            for (int j = 0; j < V; ++j) acc = fmaf(qf[r * D + c * V + j], kf[cc][j], acc);
          }
        }
        acc += __shfl_xor(acc, 8, 64);
        acc += __shfl_xor(acc, 4, 64);
        acc += __shfl_xor(acc, 2, 64);
        acc += __shfl_xor(acc, 1, 64);
        if (gl == 0 && t < t1c) scores[r * CH + (t - t0)] = finish_score(acc);
      }
    }
  }
  if (has_new && wave == NW - 1) {  // the new token's own key, still in LDS
    for (int r = 0; r < R; ++r) {
      float acc = 0.f;
      for (int d = lane; d < D; d += 64) acc = fmaf(qf[r * D + d], knew[d], acc);
      acc = wave_sum(acc);
      if (lane == 0) scores[r * CH + (pos - t0)] = finish_score(acc);
    }
  }
  __syncthreads();
  // ---- partial softmax statistics, one wave per query head
  for (int r = wave; r < R; r += NW) {
    float m = -INFINITY;
    for (int t = lane; t < n; t += 64) m = fmaxf(m, scores[r * CH + t]);
    m = wave_max(m);
    float l = 0.f;
    for (int t = lane; t < n; t += 64) {
      const float e = expf(scores[r * CH + t] - m);
      scores[r * CH + t] = e;
      l += e;
    }
    l = wave_sum(l);
    if (lane == 0) { sh_m[r] = m; sh_l[r] = l; }
  }
  __syncthreads();
  // ---- unnormalised P.V over the cached values: round 0 from the prefetched registers
  {
    float acc[R][V];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int j = 0; j < V; ++j) acc[r][j] = 0.f;
    if (grp < groups) {
      for (int tb = t0 + grp; tb < t1c; tb += UV * groups) {
        if (tb != t0 + grp) {
#pragma unroll
          for (int u = 0; u < UV; ++u) {
            const int t = tb + u * groups;
            if (t < t1c) vreg[u] = *reinterpret_cast<const APack<T, V> *>(Vc + (int64_t)t * D + col * V);
          }
        }
#pragma unroll
        for (int u = 0; u < UV; ++u) {
          const int t = tb + u * groups;
          if (t < t1c) {
            float vf[V];
#pragma unroll
            for (int j = 0; j < V; ++j) vf[j] = (float)Scalar<T>::load(&vreg[u].v[j]);
#pragma unroll
            for (int r = 0; r < R; ++r) {
              const float p = scores[r * CH + (t - t0)];
#pragma unroll
              for (int j = 0; j < V; ++j) acc[r][j] = fmaf(p, vf[j], acc[r][j]);
            }
          }
        }
      }
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int j = 0; j < V; ++j) red[(grp * R + r) * D + col * V + j] = acc[r][j];
    }
  }
  __syncthreads();
  // ---- partial (m, l, o[D]) of every query head of the block
  const int PW = D + 2;
  float *part = a.ws + (((int64_t)b * a.Hq + hq0) * NS + s) * PW;  // head r at part + r*NS*PW
  for (int e = tid; e < R * D; e += NT) {
    const int r = e / D, d = e - r * D;
    float o = has_new ? scores[r * CH + (pos - t0)] * vnew[d] : 0.f;
    for (int gg = 0; gg < groups; ++gg) o += red[(gg * R + r) * D + d];
    store_device(part + (int64_t)r * NS * PW + 2 + d, o);
  }
  if (tid < R) {
    store_device(part + (int64_t)tid * NS * PW, sh_m[tid]);
    store_device(part + (int64_t)tid * NS * PW + 1, sh_l[tid]);
  }
  decode_merge_last<T>(a, b, hq0, R, &sh_last, smem);
}

// Number of context splits: enough blocks to fill the chip, bounded so that a
// block's share of the longest context fits the LDS score buffer.
static int decode_splits(const AttnDecodeArgs &a, int head_groups) {
  const char *knob = getenv("RAI_HIP_ATTN_SPLITS");  // tuning and test aid, read at every launch
  const int forced = knob ? atoi(knob) : 0;
  int ns = forced > 0 ? forced : (2 * kNumCU + head_groups * a.B - 1) / (head_groups * a.B);
  // not more blocks than there are runs of 64 keys: below that a block's share no longer pays for its part of the
  // merge (a 530-key context of 32 heads: 8 splits 1.89 ms per Phi-2 token through the graph path, 16 splits 1.96,
  // 32 splits 2.34).  The length is the host's when it knows it, the cache's capacity otherwise.
  const int len = a.pos_dev ? a.Tmax : a.pos_host + 1;
  if (forced <= 0 && ns > (len + 63) / 64) ns = (len + 63) / 64;
  const int need = (a.Tmax + 1023) / 1024;
  if (ns < need) ns = need;
  if (ns > kDecodeMaxSplits) ns = kDecodeMaxSplits;
  if (ns > a.Tmax) ns = a.Tmax;
  return ns < 1 ? 1 : ns;
}

size_t attention_decode_ws_bytes(int B, int Hq, int D) {
  return sizeof(float) * (size_t)B * Hq * kDecodeMaxSplits * (D + 2);
}
size_t attention_decode_counter_bytes(int B, int Hq) { return sizeof(int) * (size_t)B * Hq * kDecodeCounterStride; }

// Decode attention for grouped-query models in bf16, both products on
// v_mfma_f32_16x16x32_bf16.  Block (split, kv head, batch) serves all R <= 16 query
// heads of one KV head over at most CH (64 or 128) consecutive keys:
//   - every K and V load of the block is issued before anything is computed.  K goes
//     straight from global memory into MFMA A fragments (lane l: key l%16 of a 16-key
//     tile, features 32*step + 8*(l/16) ..), two tiles per wave; V goes through LDS;
//   - scores^T[key, head] = K . Q^T per tile; accumulator register r of lane l is key
//     4*(l/16)+r, head l%16.  The rotated queries are the B fragments, held in registers;
//   - per-head max / exp / sum over the block's keys (one wave per head), exp values
//     rounded to bf16 for the second product (the reference rounds P to V's dtype);
//   - O[head, feature] = P . V: wave w owns features [w*D/4, (w+1)*D/4), P fragments are
//     16-byte LDS reads, V fragments are gathered from LDS two bytes at a time (the
//     transposition costs LDS reads, of which there are few: the kernel is bound by
//     the K/V stream);
//   - partial (m, l, o[D]) per head, merged by the last block as in the split kernel.
typedef __attribute__((ext_vector_type(8))) __bf16 ad_bf16x8;
typedef __attribute__((ext_vector_type(4))) float ad_f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t ad_u32x4;

template <int D, int CH>
__global__ void __launch_bounds__(kDecodeThreads) k_attn_decode_mfma(AttnDecodeArgs a) {
  typedef bf16_raw T;
  constexpr int KS = D / 32, KT = (CH + 63) / 64;  // 16-key tiles per wave (CH = 96: the last tile of waves 2, 3 is empty)
  constexpr int VP = D + 8, PP = CH + 8;           // LDS pitches (bf16 elements)
  constexpr int CPR = D / 8;                        // 16-byte chunks per K/V row
  constexpr int VL = CH * CPR / kDecodeThreads;     // V chunks per thread
  constexpr int DT = D / 64;                        // 16-feature tiles per wave in P.V
  extern __shared__ __attribute__((aligned(16))) float smem[];
  uint16_t *Vs = reinterpret_cast<uint16_t *>(smem);          // [CH][VP]; the first 16 rows hold Q until the scores are done
  const int R = a.Hq / a.Hkv;
  float *scores = reinterpret_cast<float *>(Vs + CH * VP);    // [R][CH]
  uint16_t *ps = reinterpret_cast<uint16_t *>(scores + R * CH);   // [16][PP]
  uint16_t *knew = ps + 16 * PP;                              // [D]
  uint16_t *vnew = knew + D;                                  // [D]
  __shared__ float sh_m[16], sh_l[16];

  const int s = blockIdx.x, hk = blockIdx.y, b = blockIdx.z;
  const int hq0 = hk * R;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lrow = lane & 15, lq = lane >> 4;
  const int NS = a.ns;
  int pos = a.pos_dev ? *a.pos_dev : a.pos_host;
  if (pos > a.Tmax - 1) pos = a.Tmax - 1;   // capacity is checked on the host; never write past the cache
  const int cnt = pos + 1;
  int chunk = (cnt + NS - 1) / NS;
  if (chunk > CH) chunk = CH;
  const int t0 = s * chunk;
  const int t1 = t0 + chunk < cnt ? t0 + chunk : cnt;
  const int n = t1 > t0 ? t1 - t0 : 0;
  const bool has_new = pos >= t0 && pos < t1;
  const int t1c = has_new ? pos : t1;       // cached keys are [t0, t1c)
  const int new_row = pos - t0;

  const int QD = a.Hq * D, KD = a.Hkv * D;
  // the new token's rows: one packed [q | k | v] row per sequence, or three separate ones
  const T *qrow = (const T *)a.qkv + (int64_t)b * (a.k_new ? a.q_row_stride : (int64_t)(QD + 2 * KD));
  const T *krow = a.k_new ? (const T *)a.k_new + (int64_t)b * a.k_row_stride : qrow + QD;
  const T *vrow = a.k_new ? (const T *)a.v_new + (int64_t)b * a.v_row_stride : qrow + QD + KD;
  T *Kc = (T *)a.kcache + ((int64_t)b * a.Hkv + hk) * a.Tmax * D;
  T *Vc = (T *)a.vcache + ((int64_t)b * a.Hkv + hk) * a.Tmax * D;
  const T *cos_t = (const T *)a.cos_t, *sin_t = (const T *)a.sin_t;

  // ---- all K and V loads of the block
  ad_bf16x8 kreg[KT][KS];
#pragma unroll
  for (int i = 0; i < KT; ++i) {
    const int t = t0 + (wave + 4 * i) * 16 + lrow;
    const bool tile_ok = (wave + 4 * i) * 16 < CH;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      ad_bf16x8 z = {};
      if (tile_ok && t < t1c) z = *reinterpret_cast<const ad_bf16x8 *>(Kc + (int64_t)t * D + ks * 32 + lq * 8);
      kreg[i][ks] = z;
    }
  }
  ad_u32x4 vreg[VL];
#pragma unroll
  for (int j = 0; j < VL; ++j) {
    const int c = tid + j * kDecodeThreads, r = c / CPR, c8 = c - r * CPR;
    ad_u32x4 z = {0u, 0u, 0u, 0u};
    if (t0 + r < t1c) z = *reinterpret_cast<const ad_u32x4 *>(Vc + (int64_t)(t0 + r) * D + c8 * 8);
    vreg[j] = z;
  }
  // ---- rotated queries (rows >= R are zero).  Eight features per item, all loads of a thread in
  //      flight together: one memory round trip instead of one per feature.
  if (a.rot % 16 == 0) {
    constexpr int QI = (16 * CPR + kDecodeThreads - 1) / kDecodeThreads;
    const int half = a.rot >> 1;
    ad_u32x4 qx[QI], qo[QI], qc[QI], qn[QI];
#pragma unroll
    for (int i = 0; i < QI; ++i) {
      const int item = tid + i * kDecodeThreads, r = item / CPR, d = (item - r * CPR) * 8;
      qx[i] = qo[i] = qc[i] = qn[i] = ad_u32x4{0u, 0u, 0u, 0u};
      if (item < 16 * CPR && r < R) {
        const T *head = qrow + (hq0 + r) * D;
        qx[i] = *reinterpret_cast<const ad_u32x4 *>(head + d);
        if (d < a.rot) {
          qo[i] = *reinterpret_cast<const ad_u32x4 *>(head + (d < half ? d + half : d - half));
          qc[i] = *reinterpret_cast<const ad_u32x4 *>(cos_t + (int64_t)pos * a.rot + d);
          qn[i] = *reinterpret_cast<const ad_u32x4 *>(sin_t + (int64_t)pos * a.rot + d);
        }
      }
    }
#pragma unroll
    for (int i = 0; i < QI; ++i) {
      const int item = tid + i * kDecodeThreads, r = item / CPR, d = (item - r * CPR) * 8;
      if (item >= 16 * CPR) continue;
      ad_u32x4 out = qx[i];
      if (r < R && d < a.rot) {
        const float sign = d < half ? -1.f : 1.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          uint32_t packed = 0;
#pragma unroll
          for (int hbit = 0; hbit < 2; ++hbit) {
            const int sh = 16 * hbit;
            const float x = bf16_bits_to_f32((uint16_t)(qx[i][w] >> sh)), o = sign * bf16_bits_to_f32((uint16_t)(qo[i][w] >> sh));
            const float c = bf16_bits_to_f32((uint16_t)(qc[i][w] >> sh)), sn = bf16_bits_to_f32((uint16_t)(qn[i][w] >> sh));
            // three roundings, as rope_feature
            const float res = round_to<T>(round_to<T>(x * c) + round_to<T>(o * sn));
            packed |= (uint32_t)f32_to_bf16_bits(res) << sh;
          }
          out[w] = packed;
        }
      }
      *reinterpret_cast<ad_u32x4 *>(Vs + r * VP + d) = out;
    }
  } else {
    for (int e = tid; e < 16 * D; e += kDecodeThreads) {
      const int r = e / D, d = e - r * D;
      const float q = r < R ? rope_feature<T>(qrow + (hq0 + r) * D, d, a.rot, cos_t, sin_t, pos) : 0.f;
      Vs[r * VP + d] = f32_to_bf16_bits(q);
    }
  }
  for (int e = tid; e < 16 * PP; e += kDecodeThreads) ps[e] = 0;
  if (has_new) {
    for (int d = tid; d < D; d += kDecodeThreads) {
      const uint16_t kr = f32_to_bf16_bits(rope_feature<T>(krow + hk * D, d, a.rot, cos_t, sin_t, pos));
      const uint16_t vr = (vrow + hk * D + d)->bits;
      knew[d] = kr;
      vnew[d] = vr;
      (Kc + (int64_t)pos * D + d)->bits = kr;
      (Vc + (int64_t)pos * D + d)->bits = vr;
    }
  }
  __syncthreads();

  // ---- scores
  {
    ad_bf16x8 qf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = *reinterpret_cast<const ad_bf16x8 *>(Vs + lrow * VP + ks * 32 + lq * 8);
#pragma unroll
    for (int i = 0; i < KT; ++i) {
      const int tile = wave + 4 * i;
      if (tile * 16 >= CH) continue;
      if (has_new && new_row == tile * 16 + lrow) {   // the lanes that hold the new token's key row
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) kreg[i][ks] = *reinterpret_cast<const ad_bf16x8 *>(knew + ks * 32 + lq * 8);
      }
      ad_f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kreg[i][ks], qf[ks], acc, 0, 0, 0);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int tl = tile * 16 + 4 * lq + r;
        float sc = a.f32_scores ? acc[r] * a.scale : round_to<T>(round_to<T>(acc[r]) * round_to<T>(a.scale));
        if (lrow < R) scores[lrow * CH + tl] = tl < n ? sc : -INFINITY;
      }
    }
  }
  __syncthreads();

  // ---- V into LDS (the new token's row from the activations), softmax statistics
#pragma unroll
  for (int j = 0; j < VL; ++j) {
    const int c = tid + j * kDecodeThreads, r = c / CPR, c8 = c - r * CPR;
    ad_u32x4 v = vreg[j];
    if (has_new && r == new_row) v = *reinterpret_cast<const ad_u32x4 *>(vnew + c8 * 8);
    *reinterpret_cast<ad_u32x4 *>(Vs + r * VP + c8 * 8) = v;
  }
  for (int r = wave; r < R; r += 4) {
    float m = -INFINITY;
    for (int t = lane; t < n; t += 64) m = fmaxf(m, scores[r * CH + t]);
    m = wave_max(m);
    float l = 0.f;
    for (int t = lane; t < n; t += 64) {
      const float e = expf(scores[r * CH + t] - m);
      ps[r * PP + t] = f32_to_bf16_bits(e);
      l += e;
    }
    l = wave_sum(l);
    if (lane == 0) { sh_m[r] = m; sh_l[r] = l; }
  }
  __syncthreads();

  // ---- O = P . V for this wave's features
  const int PW = D + 2;
  float *part = a.ws + (((int64_t)b * a.Hq + hq0) * NS + s) * PW;  // head r at part + r*NS*PW
  {
    ad_f32x4 o[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[dt] = ad_f32x4{0.f, 0.f, 0.f, 0.f};
    const int d0 = wave * (D / 4);
    for (int k0 = 0; k0 < n; k0 += 32) {
      const ad_bf16x8 pf = *reinterpret_cast<const ad_bf16x8 *>(ps + lrow * PP + k0 + lq * 8);
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        typedef __attribute__((ext_vector_type(8))) uint16_t u16x8;
        u16x8 vb;
#pragma unroll
        for (int j = 0; j < 8; ++j) vb[j] = Vs[(k0 + lq * 8 + j) * VP + d0 + dt * 16 + lrow];
        o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf, __builtin_bit_cast(ad_bf16x8, vb), o[dt], 0, 0, 0);
      }
    }
    // accumulator register r of lane l is head 4*(l/16)+r, feature l%16 of the tile
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int h = 4 * lq + r;
        if (h < R) part[(int64_t)h * NS * PW + 2 + d0 + dt * 16 + lrow] = o[dt][r];
      }
  }
  if (tid < R) {
    part[(int64_t)tid * NS * PW] = sh_m[tid];
    part[(int64_t)tid * NS * PW + 1] = sh_l[tid];
  }
}

// Merges the NS partials of one (batch, query head): block (head, batch), one
// thread per output feature.  Every wave computes the split weights
// exp(m_s - M) / L with one split per lane (NS <= 64), then each thread has all
// its partial-output loads in flight at once: two memory round trips in all.
__global__ void __launch_bounds__(256) k_attn_decode_merge_bf16(AttnDecodeArgs a) {
  const int h = blockIdx.x, b = blockIdx.y, d = threadIdx.x, lane = threadIdx.x & 63;
  const int NS = a.ns, D = a.D, PW = D + 2;
  const float *pr = a.ws + ((int64_t)b * a.Hq + h) * NS * PW;
  const float m = lane < NS ? pr[lane * PW] : -INFINITY;
  const float l = lane < NS ? pr[lane * PW + 1] : 0.f;
  const float M = wave_max(m);                    // split 0 always holds a key, so M is finite
  const float e = lane < NS ? expf(m - M) : 0.f;  // an empty split has m = -inf: weight 0
  const float L = wave_sum(e * l);
  const float w = e / L;
  float O = 0.f;
  constexpr int SB = 16;
  for (int s0 = 0; s0 < NS; s0 += SB) {
    float ov[SB];
#pragma unroll
    for (int j = 0; j < SB; ++j) ov[j] = pr[(s0 + j < NS ? s0 + j : NS - 1) * PW + 2 + d];
#pragma unroll
    for (int j = 0; j < SB; ++j)
      if (s0 + j < NS) O = fmaf(__shfl(w, s0 + j, 64), ov[j], O);
  }
  ((bf16_raw *)a.out + (int64_t)b * a.out_row_stride + (int64_t)h * D + d)->bits = f32_to_bf16_bits(O);
}

template <int D, int CH> static int launch_decode_mfma_cfg(hipStream_t st, AttnDecodeArgs a) {
  const int R = a.Hq / a.Hkv;
  a.ns = decode_splits(a, a.Hkv);
  const int need = (a.Tmax + CH - 1) / CH;
  if (a.ns < need) a.ns = need;
  a.chunk_cap = CH;
  const size_t lds = (size_t)CH * (D + 8) * 2 + (size_t)R * CH * 4 + 16 * (CH + 8) * 2 + 2 * D * 2;
  static bool attr_set = false;
  if (lds > 64 * 1024 && !attr_set) {
    RAI_HIP_TRY(hipFuncSetAttribute((const void *)k_attn_decode_mfma<D, CH>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)((size_t)CH * (D + 8) * 2 + 16 * CH * 4 + 16 * (CH + 8) * 2 + 2 * D * 2)));
    attr_set = true;
  }
  RAI_REQUIRE(a.Hkv <= 65535 && a.B <= 65535, RAI_ERR_UNSUPPORTED, "attention decode: grid too large");
  hipLaunchKernelGGL((k_attn_decode_mfma<D, CH>), dim3(a.ns, a.Hkv, a.B), dim3(kDecodeThreads), lds, st, a);
  RAI_TRY(launch_check("attention_decode_mfma"));
  hipLaunchKernelGGL(k_attn_decode_merge_bf16, dim3(a.Hq, a.B), dim3(D), 0, st, a);
  return launch_check("attention_decode_merge");
}

// Keys per block: 64, 96 or 128.  Every block issues all its loads up front and a CU holds as many blocks as their LDS
// allows, so what counts is the number of rounds the blocks need on the chip: a few blocks more than one round (1056
// blocks of 64 keys on 1024 places, Gemma-2B at batch 32 just past 2048 tokens) cost a whole block time.  Fewest
// rounds wins, then the smaller block.
constexpr int kMfmaDecodeKeysMax = 128;
template <int D> static size_t decode_mfma_lds(int CH, int R) {
  return (size_t)CH * (D + 8) * 2 + (size_t)R * CH * 4 + 16 * (CH + 8) * 2 + 2 * D * 2;
}
template <int D> static int launch_decode_mfma(hipStream_t st, const AttnDecodeArgs &a) {
  const char *knob = getenv("RAI_HIP_ATTN_KEYS");  // tuning and test aid: 64, 96 or 128 keys per block
  const int forced = knob ? atoi(knob) : 0;
  const int R = a.Hq / a.Hkv;
  int best = 0, best_rounds = 0;
  for (int ch : {64, 96, 128}) {
    const int need = (a.Tmax + ch - 1) / ch;
    if (need > kDecodeMaxSplits) continue;
    int ns = decode_splits(a, a.Hkv);
    if (ns < need) ns = need;
    const long long blocks = (long long)ns * a.Hkv * a.B;
    const long long per_cu = (long long)((160 * 1024) / (decode_mfma_lds<D>(ch, R) + 256));
    const long long places = (per_cu < 1 ? 1 : per_cu) * kNumCU;
    const int rounds = (int)((blocks + places - 1) / places);
    if (forced == ch) { best = ch; break; }
    if (!best || rounds < best_rounds) { best = ch; best_rounds = rounds; }
  }
  if (best == 64) return launch_decode_mfma_cfg<D, 64>(st, a);
  if (best == 96) return launch_decode_mfma_cfg<D, 96>(st, a);
  return launch_decode_mfma_cfg<D, 128>(st, a);
}

// The MFMA kernel serves bf16 grouped-query shapes whose longest context fits
// kDecodeMaxSplits blocks of kMfmaDecodeKeysMax keys.
static bool decode_mfma_eligible(const AttnDecodeArgs &a) {
  const bool off = getenv("RAI_HIP_NO_MFMA_DECODE") != nullptr;   // per call: a test compares both kernels in one process
  const int rep = a.Hq / a.Hkv;
  return !off && a.dtype == RAI_BF16 && rep >= 4 && rep <= 16 && (a.D == 64 || a.D == 128 || a.D == 256) &&
         (a.Tmax + kMfmaDecodeKeysMax - 1) / kMfmaDecodeKeysMax <= kDecodeMaxSplits;
}

template <typename T, int R, int CC, int UK, int UV> static int launch_decode_cfg(hipStream_t st, AttnDecodeArgs a) {
  constexpr int V = AttnVec<T>::V;
  const int ncol = a.D / V, groups = kDecodeThreads / ncol;
  const int head_groups = a.Hq / R;
  a.ns = decode_splits(a, head_groups);
  a.chunk_cap = (a.Tmax + a.ns - 1) / a.ns;
  const size_t lds = sizeof(float) * ((size_t)R * a.D + 2 * (size_t)a.D + (size_t)R * a.chunk_cap + (size_t)groups * R * a.D);
  RAI_REQUIRE(lds <= 150 * 1024, RAI_ERR_UNSUPPORTED, "attention: context %d too long for the decode kernel", a.Tmax);
  static size_t attr_bytes = 0;
  if (lds > 64 * 1024 && lds > attr_bytes) {
    RAI_HIP_TRY(hipFuncSetAttribute((const void *)k_attn_decode_split<T, R, CC, UK, UV>,
                                    hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024));
    attr_bytes = 150 * 1024;
  }
  RAI_REQUIRE(head_groups <= 65535 && a.B <= 65535, RAI_ERR_UNSUPPORTED, "attention decode: grid too large");
  hipLaunchKernelGGL((k_attn_decode_split<T, R, CC, UK, UV>), dim3(a.ns, head_groups, a.B), dim3(kDecodeThreads), lds, st, a);
  return launch_check("attention_decode");
}

template <typename T, int R> static int launch_decode_r(hipStream_t st, const AttnDecodeArgs &a) {
  constexpr int V = AttnVec<T>::V;
  const int ncol = a.D / V;
  if (ncol <= 16) return launch_decode_cfg<T, R, 1, 3, 3>(st, a);
  if (ncol <= 32) return launch_decode_cfg<T, R, 2, 2, 4>(st, a);
  return launch_decode_cfg<T, R, 4, 1, 2>(st, a);
}

template <typename T> static int launch_decode(hipStream_t st, const AttnDecodeArgs &a) {
  constexpr int V = AttnVec<T>::V;
  RAI_REQUIRE(a.D % V == 0 && a.D / V <= 64, RAI_ERR_BAD_SHAPE, "attention: head_dim %d unsupported", a.D);
  // the query heads of one KV head share a block when their count has an instantiation
  switch (a.Hq / a.Hkv) {
    case 2: return launch_decode_r<T, 2>(st, a);
    case 4: return launch_decode_r<T, 4>(st, a);
    case 6: return launch_decode_r<T, 6>(st, a);
    case 8: return launch_decode_r<T, 8>(st, a);
    default: return launch_decode_r<T, 1>(st, a);
  }
}

int launch_attention_decode(hipStream_t st, const AttnDecodeArgs &a) {
  RAI_REQUIRE(a.B > 0 && a.Hq > 0 && a.Hkv > 0 && a.D > 0 && a.Tmax > 0 && a.Hq % a.Hkv == 0, RAI_ERR_BAD_SHAPE,
              "attention decode: bad problem");
  RAI_REQUIRE(a.rot > 0 && a.rot % 2 == 0 && a.rot <= a.D, RAI_ERR_BAD_ARG, "attention decode: rot %d", a.rot);
  RAI_REQUIRE(a.ws && a.counters, RAI_ERR_BAD_ARG, "attention decode: partial-result workspace missing");
  if (decode_mfma_eligible(a)) {
    if (a.D == 64) return launch_decode_mfma<64>(st, a);
    if (a.D == 128) return launch_decode_mfma<128>(st, a);
    return launch_decode_mfma<256>(st, a);
  }
  switch (a.dtype) {
    case RAI_F32: return launch_decode<float>(st, a);
    case RAI_BF16: return launch_decode<bf16_raw>(st, a);
    default: return fail(RAI_ERR_BAD_DTYPE, "attention decode: dtype %s unsupported", dtype_name(a.dtype));
  }
}

template <typename T> static int launch_row(hipStream_t st, const AttnArgs &a) {
  constexpr int V = AttnVec<T>::V;
  RAI_REQUIRE(a.D % V == 0 && a.D / V <= 256, RAI_ERR_BAD_SHAPE, "attention: head_dim %d unsupported", a.D);
  const int ncol = a.D / V, groups = 256 / ncol;
  const size_t lds = sizeof(float) * ((size_t)a.D + (size_t)groups * a.D + (size_t)a.T);
  RAI_REQUIRE(lds <= 150 * 1024, RAI_ERR_UNSUPPORTED, "attention: context %d too long for the row kernel", a.T);
  static size_t attr_bytes = 0;
  if (lds > 64 * 1024 && lds > attr_bytes) {
    RAI_HIP_TRY(hipFuncSetAttribute((const void *)k_attn_row<T>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    150 * 1024));
    attr_bytes = 150 * 1024;
  }
  RAI_REQUIRE(a.Hq <= 65535 && a.B <= 65535, RAI_ERR_UNSUPPORTED, "attention: grid too large");
  hipLaunchKernelGGL((k_attn_row<T>), dim3(a.S, a.Hq, a.B), dim3(256), lds, st, a);
  return launch_check("attention_row");
}

// ============================================================ prefill: flash attention on MFMA (bf16)
// Block = NW waves, each owning 32 query rows; keys/values are streamed in
// tiles of 64 through LDS and shared by the waves.  Both products run on
// v_mfma_f32_32x32x16_bf16 in the transposed orientation
//     S^T = K . Q^T        (rows = keys, columns = queries)
//     O^T = V^T . P^T      (rows = head features, columns = queries)
// so every lane owns one query column: the online-softmax statistics are
// per-lane scalars, and the accumulator registers of S^T are, in order, exactly
// the B-operand fragments of the second product (no cross-lane movement).
// V is transposed while it is staged into LDS.  The score matrix never exists
// in memory (the reference materialises [B,H,S,T]).
typedef __attribute__((ext_vector_type(8))) __bf16 fa_bf16x8;
typedef __attribute__((ext_vector_type(16))) float fa_f32x16;
typedef __attribute__((ext_vector_type(4))) uint32_t fa_u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t fa_u32x2;

// KSP = 2: every 32-query group is worked on by two waves, one for the even and one for the odd key tiles, each with
// its own running maximum, sum and output; the two are merged through LDS at the end.  For short sequences and few
// heads, where the grid has about one block per CU and a wave's chain of key tiles is what the launch takes.
// (Four waves per group, KSP = 4, gained another half per cent on the Phi-2 prefill: not instantiated.)
template <int NW, int D, bool F32S, int KSP = 1>
__global__ void __launch_bounds__(NW * KSP * 64) k_flash_prefill_bf16(AttnArgs a) {
  constexpr int KS = D / 16;            // K steps of the score product
  constexpr int DT = (D + 31) / 32;     // 32-row tiles of O^T
  constexpr int KP = D + 8;             // K tile pitch (elements)
  constexpr int VP = 64 + 4;            // V^T tile pitch (elements)
  constexpr int NT = NW * KSP * 64;
  constexpr int CPR = D / 8;            // 16-byte chunks per key row
  constexpr int KTILE = 64 * KP, VTILE = DT * 32 * VP;   // elements of one K tile / one V^T tile in LDS
  __shared__ __attribute__((aligned(16))) uint16_t fa_smem[KSP * (KTILE + VTILE)];
  uint16_t *const Ks = fa_smem, *const Vt = fa_smem + KSP * KTILE;   // KSP tiles each, one behind the other
  static_assert(KSP == 1 || sizeof(float) * NW * 64 * (KSP - 1) * (2 + DT * 16) <= sizeof(uint16_t) * KSP * (KTILE + VTILE),
                "the merge of the key halves reuses the tile memory");

  const int tid = threadIdx.x, lane = tid & 63, half = lane >> 5, l32 = lane & 31;
  const int wave = (tid >> 6) / KSP, kh = (tid >> 6) % KSP;   // query group of the block, key tiles kh, kh + KSP, ...
  const int h = blockIdx.y, b = blockIdx.z;
  const int hk = h / (a.Hq / a.Hkv);
  // the last query tiles see the most keys under a causal mask: they go first so that the short ones fill the tail
  const int q0 = (int)(gridDim.x - 1 - blockIdx.x) * (NW * 32);
  const int off = a.T - a.S;  // absolute position of query row 0
  const uint16_t *Kg = (const uint16_t *)a.k + b * a.ks[0] + hk * a.ks[1];
  const uint16_t *Vg = (const uint16_t *)a.v + b * a.vs[0] + hk * a.vs[1];

  const int qrow = q0 + wave * 32 + l32;
  const int qrow_c = qrow < a.S ? qrow : a.S - 1;
  const uint16_t *qp = (const uint16_t *)a.q + b * a.qs[0] + h * a.qs[1] + (int64_t)qrow_c * a.qs[2] + half * 8;
  fa_bf16x8 qf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) qf[ks] = *reinterpret_cast<const fa_bf16x8 *>(qp + ks * 16);

  fa_f32x16 o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[dt][r] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  int kv_end = a.T;
  if (a.causal) {
    int last_q = q0 + NW * 32 < a.S ? q0 + NW * 32 : a.S;
    kv_end = off + last_q < a.T ? off + last_q : a.T;
  }
  const int wave_last_key = a.causal ? off + q0 + wave * 32 + 31 : a.T - 1;  // newest key any row of this wave may see
  const float scale_r = round_to<bf16_raw>(a.scale);

  // K/V tiles go global -> registers -> LDS; with PF the loads of tile t+1 are issued before tile t is
  // multiplied, so their latency hides behind the MFMAs (register budget allows it for D <= 128).
  // K: 16-byte chunks, row-major into Ks.  V: each work item is one pair of head features (d, d+1) for 8
  // consecutive keys: eight 4-byte loads (lanes run along d, so a wave reads whole rows), repacked in
  // registers into the two 8-key rows of V^T, which are written with 8-byte stores.
  constexpr int CH = (KSP * 64 * CPR + NT - 1) / NT;   // 16-byte chunks of K per thread (KSP tiles per round)
  constexpr int NP = D / 2;                            // feature pairs
  constexpr int VI = (KSP * 8 * NP + NT - 1) / NT;     // V work items per thread
  constexpr bool PF = D <= 128;
  fa_u32x4 kreg[CH];
  uint32_t vx[PF ? VI : 1][8];
  auto load_v = [&](int i, int k0, uint32_t (&x)[8]) {
    const int c = tid + i * NT;
    const int pr = c % NP, g = c / NP;
    if (c < KSP * 8 * NP) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        int t = k0 + g * 8 + j;
        t = t < a.T ? t : a.T - 1;   // rows past the context re-read its last row (masked below)
        x[j] = *reinterpret_cast<const uint32_t *>(Vg + (int64_t)t * a.vs[2] + 2 * pr);
      }
    }
  };
  auto store_v = [&](int i, const uint32_t (&x)[8]) {
    const int c = tid + i * NT;
    const int pr = c % NP, g = c / NP;
    if (c < KSP * 8 * NP) {
      fa_u32x2 lo0, lo1, hi0, hi1;   // feature 2*pr: keys 0-3, 4-7; feature 2*pr+1: keys 0-3, 4-7
      lo0.x = __builtin_amdgcn_perm(x[1], x[0], 0x05040100u);
      lo0.y = __builtin_amdgcn_perm(x[3], x[2], 0x05040100u);
      lo1.x = __builtin_amdgcn_perm(x[5], x[4], 0x05040100u);
      lo1.y = __builtin_amdgcn_perm(x[7], x[6], 0x05040100u);
      hi0.x = __builtin_amdgcn_perm(x[1], x[0], 0x07060302u);
      hi0.y = __builtin_amdgcn_perm(x[3], x[2], 0x07060302u);
      hi1.x = __builtin_amdgcn_perm(x[5], x[4], 0x07060302u);
      hi1.y = __builtin_amdgcn_perm(x[7], x[6], 0x07060302u);
      uint16_t *r0 = Vt + (g / 8) * VTILE + (2 * pr) * VP + (g % 8) * 8, *r1 = r0 + VP;   // key group g: tile g / 8
      *reinterpret_cast<fa_u32x2 *>(r0) = lo0;
      *reinterpret_cast<fa_u32x2 *>(r0 + 4) = lo1;
      *reinterpret_cast<fa_u32x2 *>(r1) = hi0;
      *reinterpret_cast<fa_u32x2 *>(r1 + 4) = hi1;
    }
  };
  auto load_tile = [&](int k0) {
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      const int c = tid + i * NT;
      const int key = c / CPR, dc = (c % CPR) * 8;
      int t = k0 + key;
      t = t < a.T ? t : a.T - 1;
      if (c < KSP * 64 * CPR) kreg[i] = *reinterpret_cast<const fa_u32x4 *>(Kg + (int64_t)t * a.ks[2] + dc);
    }
    if constexpr (PF) {
#pragma unroll
      for (int i = 0; i < VI; ++i) load_v(i, k0, vx[i]);
    }
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      const int c = tid + i * NT;
      const int key = c / CPR, dc = (c % CPR) * 8;
      if (c < KSP * 64 * CPR) *reinterpret_cast<fa_u32x4 *>(Ks + key * KP + dc) = kreg[i];   // tile key / 64 follows tile 0
    }
    if constexpr (PF) {
#pragma unroll
      for (int i = 0; i < VI; ++i) store_v(i, vx[i]);
    }
  };
  // without the prefetch registers the V items pass through one at a time
  auto stage_v_direct = [&](int k0) {
#pragma unroll 2
    for (int i = 0; i < VI; ++i) {
      uint32_t x[8];
      load_v(i, k0, x);
      store_v(i, x);
    }
  };
  if (PF && kv_end > 0) load_tile(0);
  for (int kb = 0; kb < kv_end; kb += 64 * KSP) {
    __syncthreads();
    // ---- stage K [64][D] and V^T [D][64], KSP tiles of each
    if (!PF) load_tile(kb);
    store_tile();
    if (!PF) stage_v_direct(kb);
    __syncthreads();
    if (PF && kb + 64 * KSP < kv_end) load_tile(kb + 64 * KSP);
    const int k0 = kb + 64 * kh;       // this wave's tile of the round
    // every key of this tile is masked for this wave, or the tile lies behind the block's keys (barriers stay uniform)
    if (k0 > wave_last_key || k0 >= kv_end) continue;
    const uint16_t *const Kt = Ks + kh * KTILE, *const Vw = Vt + kh * VTILE;

    // ---- S^T tile: 64 keys x 32 queries
    fa_f32x16 sc[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
#pragma unroll
      for (int r = 0; r < 16; ++r) sc[u][r] = 0.f;
      const uint16_t *kr = Kt + (u * 32 + l32) * KP + half * 8;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        sc[u] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<const fa_bf16x8 *>(kr + ks * 16), qf[ks], sc[u],
                                                        0, 0, 0);
    }
    // ---- scale, mask, online softmax (register r of sub-tile u is key k0 + 32u + 8*(r/4) + 4*half + r%4)
    const int q_abs = off + qrow;
    // a tile wholly inside the context and (under a causal mask) wholly at or before this wave's first query
    // needs no masking
    const bool masked = k0 + 63 >= a.T || (a.causal && k0 + 63 > off + q0 + wave * 32);
    if constexpr (F32S) {
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int r = 0; r < 16; ++r) sc[u][r] *= a.scale;
    } else {   // the product and its scaling are each rounded to bf16, two scores per conversion
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
          uint32_t pk = pack_bf16x2(sc[u][r], sc[u][r + 1]);
          pk = pack_bf16x2(__uint_as_float(pk << 16) * scale_r, __uint_as_float(pk & 0xffff0000u) * scale_r);
          sc[u][r] = __uint_as_float(pk << 16);
          sc[u][r + 1] = __uint_as_float(pk & 0xffff0000u);
        }
    }
    if (masked) {
      const int last_key = a.causal && q_abs < a.T - 1 ? q_abs : a.T - 1;   // newest key this lane's query may see
      const int rel = last_key - k0 - 4 * half;
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int r = 0; r < 16; ++r) sc[u][r] = u * 32 + 8 * (r >> 2) + (r & 3) > rel ? -INFINITY : sc[u][r];
    }
    float mx = -INFINITY;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, sc[u][r]);
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    // m_run is the exponent every p, the running sum and the output are relative to; it need not be the maximum.
    // It is moved (and sum and output rescaled) only when some query of the wave has met a score more than kLazy
    // above its own: after the first tiles that is rare, and the rescaling multiplies -- a third of this loop's
    // vector instructions at D = 128 -- are skipped.  A p may then reach e^kLazy instead of 1: nothing to bf16 or f32.
    constexpr float kLazy = 6.0f;
    const bool move = __builtin_amdgcn_ballot_w64(mx > m_run + kLazy) != 0;   // (-inf + kLazy = -inf: the first tile moves)
    const float m_new = move ? fmaxf(m_run, mx) : m_run;
    const float m_safe = m_new == -INFINITY ? 0.f : m_new;  // fully masked so far: every p is exp(-inf) = 0
    constexpr float kLog2e = 1.4426950408889634f;
    const float ml2 = m_safe * kLog2e;
    const float alpha = __builtin_amdgcn_exp2f(m_run * kLog2e - ml2);
    float psum = 0.f;
    fa_bf16x8 pf[2][2];
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        fa_u32x4 w;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float p0 = __builtin_amdgcn_exp2f(fmaf(sc[u][8 * s2 + 2 * j], kLog2e, -ml2));
          const float p1 = __builtin_amdgcn_exp2f(fmaf(sc[u][8 * s2 + 2 * j + 1], kLog2e, -ml2));
          psum += p0 + p1;
          w[j] = pack_bf16x2(p0, p1);
        }
        pf[u][s2] = __builtin_bit_cast(fa_bf16x8, w);
      }
    if (move) {
      l_run *= alpha;
      m_run = m_new;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[dt][r] *= alpha;
    }
    l_run += psum;
    // ---- O^T += V^T . P^T
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      const uint16_t *vr = Vw + (dt * 32 + l32) * VP + 4 * half;
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
          const fa_u32x2 lo = *reinterpret_cast<const fa_u32x2 *>(vr + u * 32 + 16 * s2);
          const fa_u32x2 hi = *reinterpret_cast<const fa_u32x2 *>(vr + u * 32 + 16 * s2 + 8);
          const fa_u32x4 va = {lo.x, lo.y, hi.x, hi.y};
          o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(fa_bf16x8, va), pf[u][s2], o[dt], 0, 0, 0);
        }
    }
  }

  if constexpr (KSP > 1) {
    // the waves of key tiles 1 .. KSP-1 (mod KSP) hand their maximum, sum and output over; the wave of tiles 0 merges
    // and goes on alone
    __syncthreads();   // the tiles are no longer read
    constexpr int MS = 2 + DT * 16;
    float *mb = reinterpret_cast<float *>(fa_smem) + (size_t)((wave * 64 + lane) * (KSP - 1)) * MS;
    if (kh > 0) {
      float *mine = mb + (kh - 1) * MS;
      mine[0] = m_run;
      mine[1] = l_run;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) mine[2 + dt * 16 + r] = o[dt][r];
    }
    __syncthreads();
    if (kh > 0) return;
    constexpr float kLog2e = 1.4426950408889634f;
    float m = m_run;
#pragma unroll
    for (int j = 0; j < KSP - 1; ++j) m = fmaxf(m, mb[j * MS]);
    const float ms = m == -INFINITY ? 0.f : m;   // nothing seen by any of them: every weight is exp(-inf) = 0
    const float w0 = __builtin_amdgcn_exp2f((m_run - ms) * kLog2e);
    l_run *= w0;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[dt][r] *= w0;
#pragma unroll
    for (int j = 0; j < KSP - 1; ++j) {
      const float wj = __builtin_amdgcn_exp2f((mb[j * MS] - ms) * kLog2e);
      l_run += mb[j * MS + 1] * wj;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[dt][r] += mb[j * MS + 2 + dt * 16 + r] * wj;
    }
  }
  const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
  if (qrow < a.S) {
    const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
    uint16_t *op = (uint16_t *)a.out + ((int64_t)b * a.S + qrow) * a.out_row_stride + (int64_t)h * D;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int d = dt * 32 + 8 * g + 4 * half;
        if (d < D) {
          fa_u32x2 w;
          w.x = (uint32_t)f32_to_bf16_bits(o[dt][4 * g] * inv) | ((uint32_t)f32_to_bf16_bits(o[dt][4 * g + 1] * inv) << 16);
          w.y = (uint32_t)f32_to_bf16_bits(o[dt][4 * g + 2] * inv) | ((uint32_t)f32_to_bf16_bits(o[dt][4 * g + 3] * inv) << 16);
          *reinterpret_cast<fa_u32x2 *>(op + d) = w;
        }
      }
  }
}

template <int D> static int launch_flash(hipStream_t st, const AttnArgs &a) {
  const int tiles4 = (a.S + 127) / 128;
  if ((int64_t)tiles4 * a.Hq * a.B >= kNumCU) {
    if (a.f32_scores) hipLaunchKernelGGL((k_flash_prefill_bf16<4, D, true>), dim3(tiles4, a.Hq, a.B), dim3(256), 0, st, a);
    else hipLaunchKernelGGL((k_flash_prefill_bf16<4, D, false>), dim3(tiles4, a.Hq, a.B), dim3(256), 0, st, a);
  } else {
    const dim3 grid((a.S + 63) / 64, a.Hq, a.B);
    // about one block per CU or fewer, several key tiles per block: two waves per query group, each half of the keys
    const char *no_split = getenv("RAI_HIP_FLASH_NO_KEY_SPLIT");   // read per call: tests compare both forms
    if constexpr (D <= 80) {
      if ((int64_t)grid.x * grid.y * grid.z < 2 * kNumCU && a.T > 128 && !(no_split && *no_split && *no_split != '0')) {
        if (a.f32_scores) hipLaunchKernelGGL((k_flash_prefill_bf16<2, D, true, 2>), grid, dim3(256), 0, st, a);
        else hipLaunchKernelGGL((k_flash_prefill_bf16<2, D, false, 2>), grid, dim3(256), 0, st, a);
        return launch_check("flash_prefill");
      }
    }
    if (a.f32_scores) hipLaunchKernelGGL((k_flash_prefill_bf16<2, D, true>), grid, dim3(128), 0, st, a);
    else hipLaunchKernelGGL((k_flash_prefill_bf16<2, D, false>), grid, dim3(128), 0, st, a);
  }
  return launch_check("flash_prefill");
}

static bool flash_eligible(const AttnArgs &a) {
  if (a.dtype != RAI_BF16 || a.S < 16 || a.t_dev) return false;
  if (a.D != 64 && a.D != 80 && a.D != 128 && a.D != 256) return false;
  auto al = [](const void *p, const int64_t *s) {
    return (uintptr_t)p % 16 == 0 && s[0] % 8 == 0 && s[1] % 8 == 0 && s[2] % 8 == 0;
  };
  return al(a.q, a.qs) && al(a.k, a.ks) && al(a.v, a.vs) && (uintptr_t)a.out % 8 == 0 && a.out_row_stride % 4 == 0 &&
         a.Hq <= 65535 && a.B <= 65535;
}

int launch_attention(hipStream_t st, const AttnArgs &a) {
  RAI_REQUIRE(a.B > 0 && a.Hq > 0 && a.Hkv > 0 && a.S > 0 && a.T > 0 && a.D > 0, RAI_ERR_BAD_SHAPE,
              "attention: empty problem");
  RAI_REQUIRE(a.Hq % a.Hkv == 0, RAI_ERR_BAD_SHAPE, "attention: %d query heads not divisible by %d kv heads", a.Hq,
              a.Hkv);
  if (flash_eligible(a)) {
    switch (a.D) {
      case 64: return launch_flash<64>(st, a);
      case 80: return launch_flash<80>(st, a);
      case 128: return launch_flash<128>(st, a);
      default: return launch_flash<256>(st, a);
    }
  }
  switch (a.dtype) {
    case RAI_F32: return launch_row<float>(st, a);
    case RAI_BF16: return launch_row<bf16_raw>(st, a);
    case RAI_F16: return launch_row<f16_raw>(st, a);
    default: return fail(RAI_ERR_BAD_DTYPE, "attention: dtype %s unsupported", dtype_name(a.dtype));
  }
}

}  // namespace rai

using namespace rai;

extern "C" int rai_hip_attention(int dev, const rai_hip_tensor *q, const rai_hip_tensor *k, const rai_hip_tensor *v,
                                 double scale, int32_t causal, int32_t f32_scores, const rai_hip_tensor *out) {
  RAI_TRY(validate(q, "q"));
  RAI_TRY(validate(k, "k"));
  RAI_TRY(validate(v, "v"));
  RAI_TRY(validate(out, "out"));
  RAI_REQUIRE(q->rank == 4 && k->rank == 4 && v->rank == 4 && out->rank == 3, RAI_ERR_BAD_SHAPE,
              "attention: q/k/v must be rank 4 and out rank 3");
  RAI_REQUIRE(q->dtype == k->dtype && q->dtype == v->dtype && q->dtype == out->dtype, RAI_ERR_BAD_DTYPE,
              "attention: dtype mismatch");
  const int64_t B = q->shape[0], Hq = q->shape[1], S = q->shape[2], D = q->shape[3];
  const int64_t Hkv = k->shape[1], T = k->shape[2];
  RAI_REQUIRE(k->shape[0] == B && v->shape[0] == B && k->shape[3] == D && v->shape[3] == D && v->shape[1] == Hkv &&
                  v->shape[2] == T,
              RAI_ERR_BAD_SHAPE, "attention: k/v shapes do not match q");
  RAI_REQUIRE(out->shape[0] == B && out->shape[1] == S && out->shape[2] == Hq * D && is_contiguous(out),
              RAI_ERR_BAD_SHAPE, "attention: out must be contiguous [B, S, Hq*D]");
  RAI_REQUIRE((q->stride[3] == 1 && k->stride[3] == 1 && v->stride[3] == 1) || D == 1, RAI_ERR_BAD_STRIDE,
              "attention: head_dim must have unit stride");
  RAI_REQUIRE(!causal || S <= T, RAI_ERR_BAD_SHAPE, "attention: causal needs S <= T");
  hipStream_t st = stream_of(dev);
  if (!st) return RAI_ERR_HIP;
  if (numel(out) == 0) return RAI_OK;
  const size_t es = dtype_size(q->dtype);
  const int vec = (int)(16 / es);
  auto ok = [&](const rai_hip_tensor *t) {
    if ((uintptr_t)base_ptr(t) % 16) return false;
    for (int i = 0; i < 3; ++i)
      if (t->shape[i] > 1 && t->stride[i] % vec) return false;
    return true;
  };
  RAI_REQUIRE(ok(k) && ok(v) && D % vec == 0, RAI_ERR_BAD_STRIDE, "attention: k/v rows must be 16-byte aligned");
  AttnArgs a;
  memset(&a, 0, sizeof(a));
  a.q = base_ptr(q); a.k = base_ptr(k); a.v = base_ptr(v); a.out = base_ptr(out);
  for (int i = 0; i < 3; ++i) { a.qs[i] = q->stride[i]; a.ks[i] = k->stride[i]; a.vs[i] = v->stride[i]; }
  a.out_row_stride = Hq * D;
  a.B = (int)B; a.Hq = (int)Hq; a.Hkv = (int)Hkv; a.S = (int)S; a.T = (int)T; a.D = (int)D;
  a.scale = (float)scale; a.causal = causal; a.f32_scores = f32_scores; a.dtype = q->dtype;
  return launch_attention(st, a);
}
