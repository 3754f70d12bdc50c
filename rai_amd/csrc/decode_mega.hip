// One launch per generated token: a persistent kernel that runs every decoder
// layer of a Phi-2-architecture model (rai-models/src/llm/phi2.rs:293-299,
// parallel attention + MLP block) for batch 1, bf16.
//
// One 512-thread block per CU stays resident for the whole token.  A layer is
// three weight-streaming phases separated by grid-wide barriers:
//   A  LayerNorm(x) . Wa^T + bias   -> q | k | v | gelu(fc1)      (rows split over blocks)
//   B  head h attention on block h  ||  fc2 partial products on every block
//   C  dense(attn) partial + fc2 partial + biases + residual -> x (same rows as B)
// Weights do not depend on activations, so each wave issues the first loads of
// the next phase before it arrives at the barrier: HBM keeps streaming across
// the dependency instead of draining at a kernel boundary.  Attention (latency
// bound, 0.2 MB per head) hides behind the 52 MB fc2 stream of phase B.
//
// Values that cross blocks inside the launch (x, q|k|v, act, attn) are written
// with device-scope write-through stores and read with device-scope loads: the
// per-XCD L2s are not coherent for ordinary accesses, and a device-scope fence
// would write back and invalidate a whole L2.  Weights, biases, rotary tables
// and the KV cache rows of earlier tokens are read-only here and use ordinary
// (non-temporal) loads.
//
// The grid barrier spins on a device counter; every block of the grid is
// resident (grid <= number of CUs) so the spin always ends, and it is bounded:
// on timeout the block raises DevState::fault and every later barrier falls
// through, so the kernel always terminates and the host reports the fault.
#include "decode_mega.h"

#include "gemm.h"

namespace rai {

typedef __attribute__((ext_vector_type(2))) __bf16 mg_bf16x2;
typedef __attribute__((ext_vector_type(4))) uint32_t mg_u32x4;

constexpr int kMegaThreads = 512, kMegaWaves = 8;
constexpr unsigned kMegaSpinLimit = 1u << 20;
constexpr int kMegaSlots = 4;     // phase A: weight rows in flight per wave
constexpr int kMegaRing = 8;      // phases B, C: 1 KB weight tiles in flight per wave
constexpr int kMegaRowsMax = 16;  // phases B, C: rows per block
constexpr int kMegaUK = 6, kMegaUV = 6;

__device__ __forceinline__ float mg_dot2(uint32_t a, uint32_t b, float c) {
  mg_bf16x2 p, q;
  __builtin_memcpy(&p, &a, 4);
  __builtin_memcpy(&q, &b, 4);
  return __builtin_amdgcn_fdot2_f32_bf16(p, q, c, false);
}
__device__ __forceinline__ float mg_dot8(mg_u32x4 a, mg_u32x4 b, float c) {
  c = mg_dot2(a.x, b.x, c);
  c = mg_dot2(a.y, b.y, c);
  c = mg_dot2(a.z, b.z, c);
  return mg_dot2(a.w, b.w, c);
}
__device__ __forceinline__ mg_u32x4 mg_ldw(const uint16_t *p) {
  return __builtin_nontemporal_load(reinterpret_cast<const mg_u32x4 *>(p));
}
// device-scope accesses (see the header comment)
__device__ __forceinline__ uint64_t ld_dev64(const void *p) {
  return __hip_atomic_load((const uint64_t *)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint32_t ld_dev32(const void *p) {
  return __hip_atomic_load((const uint32_t *)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ mg_u32x4 ld_dev128(const uint16_t *p) {
  const uint64_t lo = ld_dev64(p), hi = ld_dev64(p + 4);
  return mg_u32x4{(uint32_t)lo, (uint32_t)(lo >> 32), (uint32_t)hi, (uint32_t)(hi >> 32)};
}
__device__ __forceinline__ uint16_t ld_dev16(const void *p) {
  return __hip_atomic_load((const uint16_t *)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_dev16(void *p, uint16_t v) {
  __hip_atomic_store((uint16_t *)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_dev32(void *p, uint32_t v) {
  __hip_atomic_store((uint32_t *)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float mg_round(float v) { return bf16_bits_to_f32(f32_to_bf16_bits(v)); }

// Block barrier that leaves vector-memory loads in flight (only LDS traffic is drained).
__device__ __forceinline__ void wg_sync() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Grid barrier number `index` (0-based, counted from the start of the launch).
// The caller's write-through stores are complete before the arrival is counted.
__device__ __forceinline__ void grid_sync(unsigned *ctr, unsigned index, int *fault) {
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
  if (threadIdx.x == 0) {
    const unsigned target = (index + 1u) * gridDim.x;
    __hip_atomic_fetch_add(ctr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    unsigned spins = 0;
    while (__hip_atomic_load(ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
      __builtin_amdgcn_s_sleep(1);
      ++spins;
      if (spins > kMegaSpinLimit) {
        __hip_atomic_store(fault, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        break;
      }
      if ((spins & 255u) == 0 && __hip_atomic_load(fault, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) break;
    }
  }
  asm volatile("s_barrier" ::: "memory");
}

// Rotary embedding of feature d of a head whose D features sit in LDS as f32,
// with the reference's three roundings (phi2.rs:75).
__device__ __forceinline__ float mg_rope(const float *head, int d, int rot, float c, float s) {
  const float v = head[d];
  if (d >= rot) return v;
  const int half = rot >> 1;
  const float other = d < half ? -head[d + half] : head[d - half];
  return mg_round(mg_round(v * c) + mg_round(other * s));
}

// Sums over lanes with DPP (register-to-register, no LDS crossbar).
template <int CTRL> __device__ __forceinline__ float mg_dpp(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
// every lane of a 16-lane row receives the row's sum
__device__ __forceinline__ float mg_row_sum(float v) {
  v += mg_dpp<0xB1>(v);   // quad_perm [1,0,3,2]
  v += mg_dpp<0x4E>(v);   // quad_perm [2,3,0,1]
  v += mg_dpp<0x124>(v);  // row_ror:4
  v += mg_dpp<0x128>(v);  // row_ror:8
  return v;
}
// wave-uniform sum of all 64 lanes
__device__ __forceinline__ float mg_wave_sum(float v) {
  v = mg_row_sum(v);
  const int b = __builtin_bit_cast(int, v);
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0)) + __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16)) +
         (__builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32)) + __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48)));
}
// Hides a value's origin from the optimiser, so that everything derived from it
// is recomputed where it is used instead of being kept in registers across the
// whole layer loop (this kernel lives at the register limit).
__device__ __forceinline__ int mg_opaque(int v) {
  asm volatile("" : "+v"(v));
  return v;
}

#define MG_ZERO4 mg_u32x4{0u, 0u, 0u, 0u}

// KTA = H / 512 (K tiles of the phase A rows), D = head_dim.
template <int KTA, int D, bool PROF>
__global__ void __launch_bounds__(kMegaThreads) k_phi2_decode_step(MegaArgs a) {
  constexpr int NCOL = D / 8;                     // 16-byte packs per key / value row
  constexpr int NG_K = kMegaThreads / 16;         // key rows per round of the score loop
  constexpr int NG_V = kMegaThreads / NCOL;       // value rows per round of the P.V loop
  extern __shared__ __attribute__((aligned(16))) unsigned char mg_smem[];
  const int H = KTA * 512, I = a.I, QD = a.QD, KB = QD + I;
  const int KTB = I / 512, KTC = QD / 512;
  // LDS layout
  uint16_t *xs = reinterpret_cast<uint16_t *>(mg_smem);           // [I] act, then [QD] attn
  uint16_t *xa = xs + I;
  float *partB = reinterpret_cast<float *>(xa + QD);               // [rows][waves]
  float *partC = partB + kMegaRowsMax * kMegaWaves;
  float *qf = partC + kMegaRowsMax * kMegaWaves;                   // attention scratch
  float *raw = qf + D;                                             // [3*D] q | k | v before rotary
  float *knew = raw + 3 * D;
  float *vnew = knew + D;
  float *red = vnew + D;                                           // [NG_V * D]
  float *sh = red + NG_V * D;                                      // [2 * waves]
  float *red2 = sh + 2 * kMegaWaves;                               // [4 * D]
  float *scores = red2 + 4 * D;                                    // [Tmax + 1]

  const int tid0 = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid0 >> 6);      // wave-uniform: lives in scalar registers
  const int wg = blockIdx.x, G = gridDim.x;
  int *fault = &a.state->fault;
  int pos = a.state->pos;
  if (pos > a.Tmax - 1) pos = a.Tmax - 1;
  // rotary factors of this position (the same for every layer)
  float rope_c = 1.f, rope_s = 0.f;
  if (tid0 < a.rot) {
    rope_c = bf16_bits_to_f32(a.cos_t[(int64_t)pos * a.rot + tid0]);
    rope_s = bf16_bits_to_f32(a.sin_t[(int64_t)pos * a.rot + tid0]);
  }

  // ---- static work split (all wave-uniform)
  // phase A: rows [nA0, nA1) of Wa; wave w takes rows nA0 + w + 8 i
  const int nA0 = (int)((int64_t)a.NA * wg / G), nA1 = (int)((int64_t)a.NA * (wg + 1) / G);
  const int cntA = nA1 - nA0 > wave ? (nA1 - nA0 - wave + kMegaWaves - 1) / kMegaWaves : 0;
  // phases B, C: the attention blocks (wg < Hq) take rows_attn rows each, the rest is split evenly
  int n0, n1;
  const bool is_attn = wg < a.Hq;
  {
    const int n_attn_blocks = a.Hq < G ? a.Hq : G;
    const int others = G - n_attn_blocks;
    int ra = others > 0 ? a.rows_attn : (H + n_attn_blocks - 1) / n_attn_blocks;
    if (is_attn) {
      n0 = wg * ra;
      n1 = n0 + ra;
    } else {
      const int base = n_attn_blocks * ra, rem = H - base, o = wg - n_attn_blocks;
      n0 = base + (int)((int64_t)rem * o / others);
      n1 = base + (int)((int64_t)rem * (o + 1) / others);
    }
    if (n0 > H) n0 = H;
    if (n1 > H) n1 = H;
  }
  const int nrows = n1 - n0;  // <= kMegaRowsMax (checked on the host)
  // contiguous tile ranges of this wave in phases B and C
  const int ttB = nrows * KTB, ttC = nrows * KTC;
  const int tB0 = ttB * wave / kMegaWaves, tB1 = ttB * (wave + 1) / kMegaWaves;
  const int tC0 = ttC * wave / kMegaWaves, tC1 = ttC * (wave + 1) / kMegaWaves;

  mg_u32x4 slot[kMegaSlots][KTA];
  mg_u32x4 ring[kMegaRing];
  mg_u32x4 kreg[2][kMegaUK], vreg[2][kMegaUV];

  auto load_row = [&](mg_u32x4(&dst)[KTA], const uint16_t *W, int i, int lane) {
    const uint16_t *wr = W + (int64_t)(nA0 + wave + kMegaWaves * i) * H + lane * 8;
#pragma unroll
    for (int u = 0; u < KTA; ++u) dst[u] = mg_ldw(wr + u * 512);
  };
  auto prime_A = [&](const uint16_t *W, int lane) {
#pragma unroll
    for (int s = 0; s < kMegaSlots; ++s) {
      // (the else branch ends the live range of the previous contents)
      if (s < cntA) load_row(slot[s], W, s, lane);
      else
#pragma unroll
        for (int u = 0; u < KTA; ++u) slot[s][u] = MG_ZERO4;
    }
  };
  // tile t of a [rows][KT] tile grid whose K origin is column col0 of Wb
  auto tile_ptr = [&](const uint16_t *Wb, int t, int KT, int col0, int lane) -> const uint16_t * {
    const int row = t / KT, kc = t - row * KT;
    return Wb + (int64_t)(n0 + row) * KB + col0 + kc * 512 + lane * 8;
  };
  auto prime_ring = [&](const uint16_t *Wb, int t0, int t1, int KT, int col0, int lane) {
#pragma unroll
    for (int p = 0; p < kMegaRing; ++p)
      ring[p] = t0 + p < t1 ? mg_ldw(tile_ptr(Wb, t0 + p, KT, col0, lane)) : MG_ZERO4;
  };
  // Streams tiles [t0, t1) (the first kMegaRing are already in the ring), multiplies
  // them with the activation vector in LDS and leaves one partial per (row, wave).
  auto run_ring = [&](const uint16_t *Wb, int t0, int t1, int KT, int col0, const uint16_t *xv, float *part, int lane) {
    float acc = 0.f;
    int row = t0 / KT, kc = t0 - row * KT;                    // tile being consumed
    int lrow = (t0 + kMegaRing) / KT, lkc = t0 + kMegaRing - lrow * KT;  // tile being requested
    for (int tb = t0; tb < t1; tb += kMegaRing) {
#pragma unroll
      for (int p = 0; p < kMegaRing; ++p) {
        const int t = tb + p;
        if (t < t1) {
          const mg_u32x4 x4 = *reinterpret_cast<const mg_u32x4 *>(xv + kc * 512 + lane * 8);
          acc = mg_dot8(ring[p], x4, acc);
          if (t + kMegaRing < t1) {
            ring[p] = mg_ldw(Wb + (int64_t)(n0 + lrow) * KB + col0 + lkc * 512 + lane * 8);
            if (++lkc == KT) { lkc = 0; ++lrow; }
          }
          ++kc;
          if (kc == KT || t + 1 == t1) {
            const float total = mg_wave_sum(acc);
            if (lane == 0) part[row * kMegaWaves + wave] = total;
            acc = 0.f;
            if (kc == KT) { kc = 0; ++row; }
          }
        }
      }
    }
  };
  // cached keys tb + NG_K u (u < UK) of one round, 16 lanes per key row of which NCOL load
  auto k_load = [&](mg_u32x4(&kr)[kMegaUK], const uint16_t *Kc, int tb, int gl) {
#pragma unroll
    for (int u = 0; u < kMegaUK; ++u) {
      const int t = tb + NG_K * u;
      kr[u] = (t < pos && gl < NCOL) ? mg_ldw(Kc + (int64_t)t * D + gl * 8) : MG_ZERO4;
    }
  };
  auto k_scores = [&](const mg_u32x4(&kr)[kMegaUK], int tb, int gl) {
    float q8[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) q8[j] = gl < NCOL ? qf[gl * 8 + j] : 0.f;
#pragma unroll
    for (int u = 0; u < kMegaUK; ++u) {
      const int t = tb + NG_K * u;
      const uint32_t w4[4] = {kr[u].x, kr[u].y, kr[u].z, kr[u].w};
      float acc = 0.f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        acc = fmaf(q8[2 * j], __uint_as_float(w4[j] << 16), acc);
        acc = fmaf(q8[2 * j + 1], __uint_as_float(w4[j] & 0xffff0000u), acc);
      }
      acc = mg_row_sum(acc);
      if (gl == 0 && t < pos) scores[t] = acc * a.scale;
    }
  };
  auto v_load = [&](mg_u32x4(&vr)[kMegaUV], const uint16_t *Vc, int tb, int col, bool active) {
#pragma unroll
    for (int u = 0; u < kMegaUV; ++u) {
      const int t = tb + NG_V * u;
      vr[u] = (active && t < pos) ? mg_ldw(Vc + (int64_t)t * D + col * 8) : MG_ZERO4;
    }
  };
  auto v_accum = [&](const mg_u32x4(&vr)[kMegaUV], int tb, float(&acc)[8]) {
#pragma unroll
    for (int u = 0; u < kMegaUV; ++u) {
      const int t = tb + NG_V * u;
      const float p = t < pos ? scores[t] : 0.f;  // rows past the context hold zeros
      const uint32_t w4[4] = {vr[u].x, vr[u].y, vr[u].z, vr[u].w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        acc[2 * j] = fmaf(p, __uint_as_float(w4[j] << 16), acc[2 * j]);
        acc[2 * j + 1] = fmaf(p, __uint_as_float(w4[j] & 0xffff0000u), acc[2 * j + 1]);
      }
    }
  };

  unsigned bar = 0;
  prime_A(a.layers[0].Wa, tid0 & 63);
  // optional time stamps (100 MHz clock) of thread 0 of every block: [block][layer][8]
  auto stamp = [&](int l, int k) {
    if constexpr (PROF) {
      if (threadIdx.x == 0) a.prof[((int64_t)wg * a.L + l) * 8 + k] = wall_clock64();
    }
  };

  for (int l = 0; l < a.L; ++l) {
    const MegaLayer ly = a.layers[l];
    uint16_t *Kc = a.kcache + ((int64_t)l * a.kv_layer_stride) + (int64_t)wg * a.Tmax * D;  // attention blocks: head wg
    uint16_t *Vc = a.vcache + ((int64_t)l * a.kv_layer_stride) + (int64_t)wg * a.Tmax * D;
    // =================================================== phase A
    stamp(l, 0);
    {
      const int tid = mg_opaque(tid0), lane = tid & 63;
      // lane i keeps the bias of this wave's row i
      const float bias_lane = lane < cntA ? bf16_bits_to_f32(ly.ba[nA0 + wave + kMegaWaves * lane]) : 0.f;
      // activation vector of this lane: K positions lane*8 + 512 u
      mg_u32x4 xv[KTA];
#pragma unroll
      for (int u = 0; u < KTA; ++u) xv[u] = ld_dev128(a.x + u * 512 + lane * 8);
      // LayerNorm statistics from packed pairs (exact products, f32 accumulation)
      const uint32_t ones = 0x3f803f80u;
      float s1 = 0.f, s2 = 0.f;
#pragma unroll
      for (int u = 0; u < KTA; ++u) {
        const uint32_t w4[4] = {xv[u].x, xv[u].y, xv[u].z, xv[u].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          s1 = mg_dot2(w4[j], ones, s1);
          s2 = mg_dot2(w4[j], w4[j], s2);
        }
      }
      s1 = mg_wave_sum(s1);
      s2 = mg_wave_sum(s2);
      const float mean = s1 / (float)H;
      float var = s2 / (float)H - mean * mean;
      var = var > 0.f ? var : 0.f;
      const float scale = 1.0f / sqrtf(var + a.ln_eps), shift = -mean * scale;
#pragma unroll
      for (int u = 0; u < KTA; ++u) {
        const mg_u32x4 lw = *reinterpret_cast<const mg_u32x4 *>(ly.ln_w + u * 512 + lane * 8);
        const mg_u32x4 lb = *reinterpret_cast<const mg_u32x4 *>(ly.ln_b + u * 512 + lane * 8);
        const uint32_t xx[4] = {xv[u].x, xv[u].y, xv[u].z, xv[u].w};
        const uint32_t ww[4] = {lw.x, lw.y, lw.z, lw.w};
        const uint32_t bb[4] = {lb.x, lb.y, lb.z, lb.w};
        uint32_t o[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float y0 = fmaf(fmaf(__uint_as_float(xx[j] << 16), scale, shift), __uint_as_float(ww[j] << 16),
                                __uint_as_float(bb[j] << 16));
          const float y1 = fmaf(fmaf(__uint_as_float(xx[j] & 0xffff0000u), scale, shift),
                                __uint_as_float(ww[j] & 0xffff0000u), __uint_as_float(bb[j] & 0xffff0000u));
          o[j] = pack_bf16x2(y0, y1);  // the reference materialises the normalised activations in bf16
        }
        xv[u] = mg_u32x4{o[0], o[1], o[2], o[3]};
      }
      // rows of this wave, kMegaSlots at a time: products, next loads, then the four
      // reductions together; lane s finishes row i0 + s.  Results are staged in LDS
      // (the act buffer is free until phase B).
      float *stage = reinterpret_cast<float *>(xs);  // [nA1 - nA0] f32
      for (int i0 = 0; i0 < cntA; i0 += kMegaSlots) {
        float acc[kMegaSlots];
#pragma unroll
        for (int s = 0; s < kMegaSlots; ++s) {
          acc[s] = 0.f;
#pragma unroll
          for (int u = 0; u < KTA; ++u) acc[s] = mg_dot8(slot[s][u], xv[u], acc[s]);
        }
#pragma unroll
        for (int s = 0; s < kMegaSlots; ++s)
          if (i0 + s + kMegaSlots < cntA) load_row(slot[s], ly.Wa, i0 + s + kMegaSlots, lane);
        float mine = 0.f;
#pragma unroll
        for (int s = 0; s < kMegaSlots; ++s) {
          const float total = mg_wave_sum(acc[s]);
          if (lane == s) mine = total;
        }
        const float bias = __shfl(bias_lane, i0 + lane, 64);
        if (lane < kMegaSlots && i0 + lane < cntA) {
          const int n = nA0 + wave + kMegaWaves * (i0 + lane);
          float v = mine + bias;
          if (n >= a.n_qkv) v = act_eval(a.act, v);
          stage[n - nA0] = v;
        }
      }
      // first loads of phase B: this wave's fc2 tiles; the attention blocks also fetch
      // the first two rounds of cached keys and values of their head
      prime_ring(ly.Wb, tB0, tB1, KTB, QD, lane);
      if (is_attn) {
        const int g = tid >> 4, gl = tid & 15, col = tid % NCOL, grp = tid / NCOL;
        k_load(kreg[0], Kc, g, gl);
        k_load(kreg[1], Kc, g + NG_K * kMegaUK, gl);
        v_load(vreg[0], Vc, grp, col, grp < NG_V);
        v_load(vreg[1], Vc, grp + NG_V * kMegaUV, col, grp < NG_V);
      } else {
#pragma unroll
        for (int u = 0; u < kMegaUK; ++u) kreg[0][u] = kreg[1][u] = MG_ZERO4;
#pragma unroll
        for (int u = 0; u < kMegaUV; ++u) vreg[0][u] = vreg[1][u] = MG_ZERO4;
      }
      wg_sync();
      // write q|k|v and act with write-through stores
      for (int e = tid; e < nA1 - nA0; e += kMegaThreads) {
        const int n = nA0 + e;
        st_dev16(n < a.n_qkv ? a.qkv + n : a.act_buf + (n - a.n_qkv), f32_to_bf16_bits(stage[e]));
      }
      stamp(l, 1);
      grid_sync(a.barrier, bar++, fault);
      stamp(l, 2);
    }

    // =================================================== phase B
    {
      const int tid = mg_opaque(tid0), lane = tid & 63;
      if (tid < 2 * kMegaRowsMax * kMegaWaves) partB[tid] = 0.f;  // partB and partC are adjacent
      // act -> LDS
      for (int k = tid * 4; k < I; k += kMegaThreads * 4) {
        const uint64_t v = ld_dev64(a.act_buf + k);
        *reinterpret_cast<uint64_t *>(xs + k) = v;
      }
      if (is_attn) {
        const int h = wg;
        // q, k, v of the new token
        if (tid < 3 * D / 2) {
          const int which = tid / (D / 2), e = (tid - which * (D / 2)) * 2;
          const uint32_t w = ld_dev32(a.qkv + which * QD + h * D + e);
          raw[which * D + e] = __uint_as_float(w << 16);
          raw[which * D + e + 1] = __uint_as_float(w & 0xffff0000u);
        }
        wg_sync();
        if (tid < D) {
          qf[tid] = mg_rope(raw, tid, a.rot, rope_c, rope_s);
          const float kr = mg_rope(raw + D, tid, a.rot, rope_c, rope_s);
          const float vr = raw[2 * D + tid];
          knew[tid] = kr;
          vnew[tid] = vr;
          Kc[(int64_t)pos * D + tid] = f32_to_bf16_bits(kr);
          Vc[(int64_t)pos * D + tid] = f32_to_bf16_bits(vr);
        }
        wg_sync();
        // scores against the cached keys, two rounds of NG_K * UK keys in flight
        {
          const int g = tid >> 4, gl = tid & 15;
          constexpr int RK = NG_K * kMegaUK;
          for (int tb = 0; tb < pos; tb += 2 * RK) {
            k_scores(kreg[0], tb + g, gl);
            if (tb + 2 * RK < pos) k_load(kreg[0], Kc, tb + 2 * RK + g, gl);
            if (tb + RK < pos) {
              k_scores(kreg[1], tb + RK + g, gl);
              if (tb + 3 * RK < pos) k_load(kreg[1], Kc, tb + 3 * RK + g, gl);
            }
          }
        }
        if (wave == kMegaWaves - 1) {  // the new token's own key
          float acc = 0.f;
          for (int d = lane; d < D; d += 64) acc = fmaf(qf[d], knew[d], acc);
          acc = mg_wave_sum(acc);
          if (lane == 0) scores[pos] = acc * a.scale;
        }
        wg_sync();
        const int cnt = pos + 1;
        float m = -INFINITY;
        for (int t = tid; t < cnt; t += kMegaThreads) m = fmaxf(m, scores[t]);
        m = wave_max(m);
        if (lane == 0) sh[wave] = m;
        wg_sync();
        m = sh[0];
#pragma unroll
        for (int w = 1; w < kMegaWaves; ++w) m = fmaxf(m, sh[w]);
        float sum = 0.f;
        for (int t = tid; t < cnt; t += kMegaThreads) {
          const float e = expf(scores[t] - m);
          scores[t] = e;
          sum += e;
        }
        sum = mg_wave_sum(sum);
        if (lane == 0) sh[kMegaWaves + wave] = sum;
        wg_sync();
        sum = 0.f;
#pragma unroll
        for (int w = 0; w < kMegaWaves; ++w) sum += sh[kMegaWaves + w];
        // unnormalised P.V over the cached values, two rounds of NG_V * UV rows in flight
        {
          const int col = tid % NCOL, grp = tid / NCOL;
          const bool active = grp < NG_V;
          constexpr int RV = NG_V * kMegaUV;
          float acc[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) acc[j] = 0.f;
          for (int tb = 0; tb < pos; tb += 2 * RV) {
            v_accum(vreg[0], tb + grp, acc);
            if (tb + 2 * RV < pos) v_load(vreg[0], Vc, tb + 2 * RV + grp, col, active);
            if (tb + RV < pos) {
              v_accum(vreg[1], tb + RV + grp, acc);
              if (tb + 3 * RV < pos) v_load(vreg[1], Vc, tb + 3 * RV + grp, col, active);
            }
          }
          if (active) {
#pragma unroll
            for (int j = 0; j < 8; ++j) red[grp * D + col * 8 + j] = acc[j];
          }
        }
        wg_sync();
        // two-level sum over the NG_V groups, then the head's D outputs as D/2 packed pairs
        if (tid < 4 * D) {
          const int d = tid % D, q4 = tid / D;
          float r = 0.f;
          for (int gg = q4; gg < NG_V; gg += 4) r += red[gg * D + d];
          red2[tid] = r;
        }
        wg_sync();
        if (tid < D / 2) {
          const float inv = 1.0f / sum, p_new = scores[pos];
          float o[2];
#pragma unroll
          for (int k = 0; k < 2; ++k) {
            const int d = 2 * tid + k;
            o[k] = (p_new * vnew[d] + red2[d] + red2[D + d] + red2[2 * D + d] + red2[3 * D + d]) * inv;
          }
          st_dev32(a.attn + h * D + 2 * tid, pack_bf16x2(o[0], o[1]));
        }
      }
      wg_sync();
      stamp(l, 3);
      run_ring(ly.Wb, tB0, tB1, KTB, QD, xs, partB, lane);
      // first loads of phase C: the dense columns of the same rows
      prime_ring(ly.Wb, tC0, tC1, KTC, 0, lane);
      stamp(l, 4);
      grid_sync(a.barrier, bar++, fault);
      stamp(l, 5);
    }

    // =================================================== phase C
    {
      const int tid = mg_opaque(tid0), lane = tid & 63;
      // epilogue operands of this thread's row, requested before the stream
      float bsum = 0.f, res = 0.f;
      if (tid < nrows) {
        res = bf16_bits_to_f32(ld_dev16(a.x + n0 + tid));
        bsum = bf16_bits_to_f32(ly.bd[n0 + tid]) + bf16_bits_to_f32(ly.bf[n0 + tid]);
      }
      for (int k = tid * 4; k < QD; k += kMegaThreads * 4) {
        const uint64_t v = ld_dev64(a.attn + k);
        *reinterpret_cast<uint64_t *>(xa + k) = v;
      }
      wg_sync();
      run_ring(ly.Wb, tC0, tC1, KTC, 0, xa, partC, lane);
      if (l + 1 < a.L) prime_A(a.layers[l + 1].Wa, lane);
      wg_sync();
      // x[n] += dense + fc2 + biases for the rows of this block.
      // Fixed summation order: fc2 partials of the waves, then the dense partials.
      if (tid < nrows) {
        float sacc = 0.f;
#pragma unroll
        for (int w = 0; w < kMegaWaves; ++w) sacc += partB[tid * kMegaWaves + w];
#pragma unroll
        for (int w = 0; w < kMegaWaves; ++w) sacc += partC[tid * kMegaWaves + w];
        st_dev16(a.x + n0 + tid, f32_to_bf16_bits(sacc + bsum + res));
      }
      stamp(l, 6);
      if (l + 1 < a.L) grid_sync(a.barrier, bar++, fault);
      stamp(l, 7);
    }
  }
}

size_t mega_lds_bytes(const MegaArgs &a, int D) {
  const int NG_V = kMegaThreads / (D / 8);
  size_t n = (size_t)(a.I + a.QD) * 2;
  n += sizeof(float) * (2 * kMegaRowsMax * kMegaWaves + 6 * (size_t)D + (size_t)NG_V * D + 2 * kMegaWaves +
                        4 * (size_t)D + (size_t)a.Tmax + 1);
  return (n + 15) & ~(size_t)15;
}

bool mega_eligible(const MegaArgs &a, int D, int num_cu, const char **why) {
  auto no = [&](const char *w) { if (why) *why = w; return false; };
  if (a.H != 2560) return no("hidden size is not 2560");
  if (D != 80) return no("head_dim is not 80");
  if (a.Hq * D != a.QD || a.QD % 512 || a.I % 512) return no("projection widths are not multiples of 512");
  if (a.Hq > num_cu) return no("more heads than CUs");
  if (a.n_qkv != 3 * a.QD || a.NA != a.n_qkv + a.I) return no("q|k|v layout");
  if (a.rot > D || (a.rot & 1)) return no("rotary_dim");
  // rows per block in phases B and C
  const int others = num_cu - a.Hq;
  const int ra = others > 0 ? a.rows_attn : (a.H + a.Hq - 1) / a.Hq;
  if (ra < 0 || ra > kMegaRowsMax) return no("rows_attn");
  if (others > 0) {
    const int rem = a.H - a.Hq * ra;
    if (rem < 0 || (rem + others - 1) / others + 1 > kMegaRowsMax) return no("too many rows per block");
  }
  if ((size_t)(a.NA / num_cu + 2) * sizeof(float) > (size_t)a.I * 2) return no("phase A staging does not fit");
  if (mega_lds_bytes(a, D) > 150 * 1024) return no("context too long for the LDS score buffer");
  return true;
}

int launch_phi2_decode_step(hipStream_t st, const MegaArgs &a, int D, int num_cu) {
  const char *why = nullptr;
  RAI_REQUIRE(mega_eligible(a, D, num_cu, &why), RAI_ERR_UNSUPPORTED, "persistent decode step: %s", why ? why : "?");
  const size_t lds = mega_lds_bytes(a, D);
  static size_t attr_bytes = 0;
  if (lds > 64 * 1024 && lds > attr_bytes) {
    RAI_HIP_TRY(hipFuncSetAttribute((const void *)k_phi2_decode_step<5, 80, false>,
                                    hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024));
    RAI_HIP_TRY(hipFuncSetAttribute((const void *)k_phi2_decode_step<5, 80, true>,
                                    hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024));
    attr_bytes = 150 * 1024;
  }
  if (a.prof) hipLaunchKernelGGL((k_phi2_decode_step<5, 80, true>), dim3(num_cu), dim3(kMegaThreads), lds, st, a);
  else hipLaunchKernelGGL((k_phi2_decode_step<5, 80, false>), dim3(num_cu), dim3(kMegaThreads), lds, st, a);
  return launch_check("phi2_decode_step");
}

}  // namespace rai
