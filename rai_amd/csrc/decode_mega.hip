// One launch per generated token: a persistent kernel that runs every decoder
// layer of a Phi-2-architecture model (rai-models/src/llm/phi2.rs:293-299,
// parallel attention + MLP block) for batch 1, bf16.
//
// One 512-thread block per CU stays resident for the whole token.  A layer is
// three weight-streaming segments:
//   A1  LayerNorm(x) . Wa[q|k|v rows]^T + bias -> q | k | v   (rows split over all blocks, streamed first)
//   A2  LayerNorm(x) . Wa[fc1 rows]^T + bias   -> gelu(fc1)   (rows split over the blocks without an attention head)
//       head h attention on block h, started as soon as the A1 packets arrive, i.e. while A2 streams
//   BC  [attn | act] . Wb^T + biases + residual -> x          (whole rows of Wb = dense | fc2 columns)
// Weights do not depend on activations: every wave keeps a ring of weight tiles
// in flight that runs ahead across the segment boundaries, so HBM keeps streaming
// while a block waits for its inputs; when the ring is full a wave has the next
// kMegaStage tiles copied straight into LDS (global -> LDS loads need no registers) and
// takes them from there when it streams again.  A1 runs into A2 without a pause: each stream wave
// bumps a counter in LDS when it leaves A1, and the service wave publishes the q|k|v
// packets when all have.
//
// There is no grid barrier.  The vectors that cross blocks (x, q|k|v, act, attn) are
// written as 8-byte packets, tag = launch epoch * 1024 + exchange index + 1, with
// device-scope write-through stores, and every consumer polls exactly the packets it
// needs with device-scope loads until their tags match (an 8-byte store is single-copy
// atomic, so a matching tag proves the payload).  x and q|k|v use {two bf16 values,
// 32-bit tag} at the vector's own index; act and attn, which every Wb block needs whole,
// use {three bf16 values, low 16 bits of the tag} in producer-owned slots (16 per fc1
// block, ceil(D / 3) per head), so that nine packets per thread, one poll, fetch both.
// Data and notification are therefore one memory trip, not a store, its
// acknowledgement, a flag and a second read; a buffer is safe to overwrite two
// exchanges later because receiving a block's packets proves that block has left the
// phase in which it read the older ones.  The per-XCD L2s are not coherent for
// ordinary accesses and a device-scope fence would write back and invalidate a whole
// L2, hence packets and no fences.  Weights, biases, rotary tables and the KV cache
// rows of earlier tokens are read-only here and use ordinary loads.
//
// Every block of the grid is resident (grid <= number of CUs), so a poll always ends,
// and it is bounded: on timeout the wave raises DevState::fault, later polls fall
// through, the kernel terminates and the host reports the fault.
#include "decode_mega.h"

#include "gemm.h"

namespace rai {

typedef __attribute__((ext_vector_type(2))) __bf16 mg_bf16x2;
typedef __attribute__((ext_vector_type(4))) uint32_t mg_u32x4;

constexpr int kMegaThreads = 512, kMegaWaves = 8;

constexpr int kMegaStream = kMegaWaves - 1, kMegaService = kMegaWaves - 1;
constexpr unsigned kMegaSpinLimit = 1u << 20;
constexpr uint32_t kMegaTagsPerLaunch = 1024;   // more than the 3 exchanges per layer of any eligible model
constexpr int kMegaRing = 16;
constexpr int kMegaStage = 8;              // tiles (1 KB each) per stream wave held in LDS beyond the ring
constexpr size_t kMegaLdsMax = 160 * 1024;
constexpr int kMegaRowsAMax = 96;
constexpr int kMegaRowsMax = 16;
constexpr int kMegaUK = 13, kMegaUV = 12;

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
__device__ __forceinline__ void st_dev64(void *p, uint64_t v) {
  __hip_atomic_store((uint64_t *)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_dev32(void *p, uint32_t v) {
  __hip_atomic_store((uint32_t *)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float mg_round(float v) { return bf16_bits_to_f32(f32_to_bf16_bits(v)); }

__device__ __forceinline__ void wg_sync() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Rotary embedding of feature d of a head whose D features sit in LDS as f32,
// with the reference's three roundings (phi2.rs:75).
__device__ __forceinline__ float mg_rope(const float *head, int d, int rot, float c, float s) {
  const float v = head[d];
  if (d >= rot) return v;
  const int half = rot >> 1;
  const float other = d < half ? -head[d + half] : head[d - half];
  return mg_round(mg_round(v * c) + mg_round(other * s));
}

template <int CTRL> __device__ __forceinline__ float mg_dpp(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}

__device__ __forceinline__ float mg_row_sum(float v) {
  v += mg_dpp<0xB1>(v);
  v += mg_dpp<0x4E>(v);
  v += mg_dpp<0x124>(v);
  v += mg_dpp<0x128>(v);
  return v;
}

__device__ __forceinline__ float mg_wave_sum(float v) {
  v = mg_row_sum(v);
  const int b = __builtin_bit_cast(int, v);
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0)) + __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16)) +
         (__builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32)) + __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48)));
}

__device__ __forceinline__ int mg_opaque(int v) {
  asm volatile("" : "+v"(v));
  return v;
}

#define MG_ZERO4 mg_u32x4{0u, 0u, 0u, 0u}

// Rotates the ring so that entry R becomes entry 0 (all of its loads have landed).
template <int R> __device__ __forceinline__ void mg_rotate(mg_u32x4 (&ring)[kMegaRing]) {
  mg_u32x4 tmp[kMegaRing];
#pragma unroll
  for (int p = 0; p < kMegaRing; ++p) tmp[p] = ring[(p + R) % kMegaRing];
#pragma unroll
  for (int p = 0; p < kMegaRing; ++p) ring[p] = tmp[p];
}

// A wave's weight stream: per layer up to three segments, in streaming order A1 (q|k|v rows of Wa), A2 (fc1 rows
// of Wa), BC (whole rows of Wb: dense columns, then fc2 columns).  Everything about a segment that does not change
// from layer to layer is worked out once, so that moving the cursor to the next segment is a few selects: no loop
// and no division inside the streaming loops (with those in every step the compiler kept the ring in a second set
// of registers and copied it back, after waiting for every load, once per pass).
struct MgSplit {
  const uint16_t *Wa0, *Wb0;
  int64_t wa_stride, wb_stride;
  int L, H, KB, KTA, KTBC;
  int64_t off0, off1, off2;   // element offset of the segment's first tile from its matrix in the same layer
  int kc0, kc1, kc2;          // column tile of its first tile
  int cnt0, cnt1, cnt2;       // tiles
  int nx0, nx1, nx2;          // the next segment that is not empty (cyclic; the segment itself when it is the only one)
};

// ptr is the tile that is requested next; the tiles of a row follow each other (`step` = 512 elements), the next
// row starts `jump` elements behind the row's last tile.  Behind the last layer step and jump are 0: the last tile
// is requested again and again (never used; the streaming loops need no end-of-stream case that way).
struct MgCursor {
  int layer, seg, kc, KT, left;   // left: tiles of the segment not yet requested, the one under the cursor included
  int64_t jump, step;
  const uint16_t *ptr;
};

__device__ __forceinline__ void mg_seg_enter(MgCursor &c, const MgSplit &sp, int layer, int seg) {
  // (the fields are copied into values first: selecting between struct members by `seg` directly makes the
  // compiler keep the struct in scratch memory and select addresses)
  const int64_t off0 = sp.off0, off1 = sp.off1, off2 = sp.off2;
  const int kc0 = sp.kc0, kc1 = sp.kc1, kc2 = sp.kc2, cnt0 = sp.cnt0, cnt1 = sp.cnt1, cnt2 = sp.cnt2;
  const bool wa = seg <= 1;
  const uint16_t *base = wa ? sp.Wa0 + layer * sp.wa_stride : sp.Wb0 + layer * sp.wb_stride;
  c.layer = layer;
  c.seg = seg;
  c.KT = wa ? sp.KTA : sp.KTBC;
  c.jump = (int64_t)(wa ? sp.H : sp.KB) - (int64_t)(c.KT - 1) * 512;
  c.step = 512;
  c.kc = seg == 0 ? kc0 : seg == 1 ? kc1 : kc2;
  c.left = seg == 0 ? cnt0 : seg == 1 ? cnt1 : cnt2;
  c.ptr = base + (seg == 0 ? off0 : seg == 1 ? off1 : off2) + c.kc * 512;
}
__device__ __forceinline__ void mg_advance(MgCursor &c, const MgSplit &sp) {
  if (--c.left == 0) {
    const int nx0 = sp.nx0, nx1 = sp.nx1, nx2 = sp.nx2;
    const int ns = c.seg == 0 ? nx0 : c.seg == 1 ? nx1 : nx2;
    const int nl = c.layer + (ns <= c.seg ? 1 : 0);
    if (nl >= sp.L) {   // behind the last layer: the cursor stays on the last tile (requests that hit the caches)
      c.kc = 0; c.KT = 0x7fffffff; c.left = 0x7fffffff; c.jump = 0; c.step = 0;
    } else {
      mg_seg_enter(c, sp, nl, ns);
    }
  } else {
    const bool wrap = c.kc + 1 == c.KT;
    c.kc = wrap ? 0 : c.kc + 1;
    c.ptr += wrap ? c.jump : c.step;
  }
}
// requests the tile under the cursor and advances the cursor
__device__ __forceinline__ mg_u32x4 mg_next_load(MgCursor &c, const MgSplit &sp, int lane) {
  const mg_u32x4 v = mg_ldw(c.ptr + lane * 8);
  mg_advance(c, sp);
  return v;
}
// the same request with LDS as its destination: lane i's 16 bytes land at slot + 16 i
__device__ __forceinline__ void mg_next_stage(MgCursor &c, const MgSplit &sp, int lane, unsigned char *slot) {
  typedef __attribute__((address_space(3))) void *lds_ptr;
  __builtin_amdgcn_global_load_lds((const void *)(c.ptr + lane * 8), (lds_ptr)slot, 16, 0, 2 /* nt */);
  mg_advance(c, sp);
}
// Two ranges of tiles of [rows][KT] tile grids that one phase of a wave consumes one after the other (the second may
// be empty, and so may the first); the same in every layer.
struct MgPhase {
  int n1, kc1, row1;   // tiles, column tile and row of the first tile
  int n2, kc2, row2;
};
__device__ __forceinline__ MgPhase mg_phase(int t0, int t1, int u0, int u1, int KT) {
  MgPhase ph;
  ph.n1 = t1 > t0 ? t1 - t0 : 0; ph.row1 = t0 / KT; ph.kc1 = t0 - ph.row1 * KT;
  ph.n2 = u1 > u0 ? u1 - u0 : 0; ph.row2 = u0 / KT; ph.kc2 = u0 - ph.row2 * KT;
  return ph;
}
// Consumes the tiles of a phase from the ring (entry 0 first), the second range behind the first without a pause;
// multiplies them with the activation vector in LDS (the same for both ranges) and leaves one partial sum per
// (row, wave) in `part` / `part2`.  When the first range is done (also when it is empty) lane 0 adds one to *done1,
// after its partial sums are in LDS.  Returns how many entries the ring must be rotated afterwards.
// `staged`: the kMegaStage tiles that follow the ring's sixteen are in LDS at `stage` (1 KB each, in order); the
// first pass over the ring then refills its first kMegaStage entries from there (a wave that stages has at least
// kMegaRing tiles in every phase that is not empty).
// A wave issues one instruction every four clocks at best, and the stream is bound by that, not by the loads: a
// step is kept to the multiply, the refill and a handful of scalar instructions.  The activation tile of the next
// step is read from LDS a step ahead; the only counter in a step is the distance to the end of the row.
__device__ __forceinline__ int mg_run_phase(mg_u32x4 (&ring)[kMegaRing], MgCursor &c, const MgSplit &sp, const MgPhase &ph,
                                            int KT, const uint16_t *xv, float *part, float *part2, uint32_t *done1,
                                            int lane, int wave, const unsigned char *stage, bool &staged) {
  float acc = 0.f;
  const int total = ph.n1 + ph.n2;
  int left = total;
  bool second = ph.n1 == 0;
  if (second && done1 && lane == 0) __hip_atomic_fetch_add(done1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  int rr = second ? ph.n2 : ph.n1;             // tiles left in the range, the current row included
  int row = second ? ph.row2 : ph.row1;
  float *prow = (second ? part2 : part) + row * kMegaWaves + wave;   // where this row's partial sum goes
  const int kc_first = second ? ph.kc2 : ph.kc1;
  int rem = KT - kc_first < rr ? KT - kc_first : rr;                 // steps to the end of the row (or of the range)
  int row_len = rem;
  const int xo2 = ph.kc2 * 1024;
  int xo_row = (!second && ph.n2 > 0 && rr == row_len) ? xo2 : 0;    // LDS offset of the tile that follows this row's last
  int xo = kc_first * 1024;
  const unsigned char *xl = reinterpret_cast<const unsigned char *>(xv) + lane * 16;
  // Everything requested before this point has landed: the ring a whole exchange ago, the staged tiles before the
  // poll that ended the wait (loads return in order).  Saying so keeps the compiler from guarding the LDS reads of
  // the loops below against the global -> LDS loads, and, more important, lets it count: the layer's biases are read
  // through pointers that were themselves loaded from memory, i.e. with flat loads, and while one of those is
  // outstanding (the service wave uses them after the stream) every wait for a ring entry becomes a wait for all
  // loads, which empties the ring once per pass.
  __builtin_amdgcn_s_waitcnt(0x0070);   // vmcnt(0) lgkmcnt(0)
  mg_u32x4 x4n = *reinterpret_cast<const mg_u32x4 *>(xl + xo);
#define MG_STEP(r) MG_STEP_FROM(r, mg_next_load(c, sp, lane))
#define MG_STEP_FROM(r, REFILL)                                                                     \
  {                                                                                                 \
    const mg_u32x4 x4 = x4n;                                                                        \
    const bool last = rem == 1;                                                                     \
    xo = last ? xo_row : xo + 1024;                                                                 \
    x4n = *reinterpret_cast<const mg_u32x4 *>(xl + xo);                                             \
    acc = mg_dot8(r, x4, acc);                                                                      \
    asm volatile("" : "+v"(acc)); /* the products stay ahead of the refill: were they sunk below */ \
    r = REFILL;                   /* it, old and new tile would need two registers              */ \
    --rem;                                                                                          \
    if (last) {                                                                                     \
      const float total_ = mg_wave_sum(acc);                                                        \
      if (lane == 0) *prow = total_;                                                                \
      acc = 0.f;                                                                                    \
      rr -= row_len;                                                                                \
      prow += kMegaWaves;                                                                           \
      if (rr == 0 && !second) {                                                                     \
        if (done1 && lane == 0) __hip_atomic_fetch_add(done1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP); \
        second = true;                                                                              \
        rr = ph.n2;                                                                                 \
        prow = part2 + ph.row2 * kMegaWaves + wave;                                                 \
        row_len = KT - ph.kc2 < rr ? KT - ph.kc2 : rr;                                              \
      } else {                                                                                      \
        row_len = KT < rr ? KT : rr;                                                                \
      }                                                                                             \
      rem = row_len;                                                                                \
      xo_row = (!second && ph.n2 > 0 && rr == row_len) ? xo2 : 0;                                   \
    }                                                                                               \
  }
  if (staged && total > 0) {
#pragma unroll
    for (int p = 0; p < kMegaRing; ++p) {
      if (p < kMegaStage) MG_STEP_FROM(ring[p], *reinterpret_cast<const mg_u32x4 *>(stage + p * 1024 + lane * 16))
      else MG_STEP(ring[p])
    }
    left -= kMegaRing;
    staged = false;
  }
  while (left >= kMegaRing) {
#pragma unroll
    for (int p = 0; p < kMegaRing; ++p) MG_STEP(ring[p])
    left -= kMegaRing;
  }
  // the rest: step p runs only if every step before it ran, and the control flow says so (an early exit, not sixteen
  // independent conditions), so that the compiler can count the loads between a tile's request and its use; with
  // independent conditions it has to wait for every outstanding load before each of these steps
#define MG_REST(p)                  \
  if (left <= p) goto rest_done;    \
  MG_STEP(ring[p])
  static_assert(kMegaRing == 16, "the steps below are written out");
  MG_REST(0) MG_REST(1) MG_REST(2) MG_REST(3) MG_REST(4) MG_REST(5) MG_REST(6) MG_REST(7)
  MG_REST(8) MG_REST(9) MG_REST(10) MG_REST(11) MG_REST(12) MG_REST(13) MG_REST(14)
rest_done:
#undef MG_REST
#undef MG_STEP
#undef MG_STEP_FROM
  return total % kMegaRing;
}
__device__ __forceinline__ void mg_rotate_by(mg_u32x4 (&ring)[kMegaRing], int r) {
  static_assert((kMegaRing & (kMegaRing - 1)) == 0 && kMegaRing <= 16, "rotation is composed from powers of two");
  if (r & 1) mg_rotate<1>(ring);
  if (r & 2) mg_rotate<2 % kMegaRing>(ring);
  if (r & 4) mg_rotate<4 % kMegaRing>(ring);
  if (r & 8) mg_rotate<8 % kMegaRing>(ring);
}

// Reads N packets per lane (packet i at src[idx[i]] when on[i]) until each carries `tag`; returns the
// payloads.  The wave leaves the loop together; the spin is bounded (by kMegaSpinLimit; the instrumented
// build of the kernel, DBG, takes the bound from the launch arguments so that a test can make it tiny).
template <int N, bool DBG>
__device__ __forceinline__ void mg_poll(const uint64_t *src, const int (&idx)[N], const bool (&on)[N], uint32_t tag,
                                        uint32_t (&out)[N], int *fault, unsigned spin_limit) {
  bool need[N];
#pragma unroll
  for (int i = 0; i < N; ++i) { need[i] = on[i]; out[i] = 0u; }
  unsigned spins = 0;
  for (;;) {
    uint64_t pk[N];
#pragma unroll
    for (int i = 0; i < N; ++i) pk[i] = need[i] ? ld_dev64(src + idx[i]) : 0ull;
    bool pending = false;
#pragma unroll
    for (int i = 0; i < N; ++i) {
      if (need[i]) {
        if ((uint32_t)(pk[i] >> 32) == tag) { out[i] = (uint32_t)pk[i]; need[i] = false; }
        else pending = true;
      }
    }
    if (!__any(pending)) break;
    __builtin_amdgcn_s_sleep(1);   // a short pause between rounds: bounds the polling traffic
    if (++spins > (DBG ? spin_limit : kMegaSpinLimit)) {
      __hip_atomic_store(fault, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      break;
    }
    if ((spins & 255u) == 0 && __hip_atomic_load(fault, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) break;
  }
}
// mg_poll over one list drawn from two packet arrays: entries below n0 come from src0 (tag0), the others from
// src1 at index - n0 (tag1).
template <int N, bool DBG>
__device__ __forceinline__ void mg_poll2(const uint64_t *src0, uint32_t tag0, int n0, const uint64_t *src1, uint32_t tag1,
                                         const int (&idx)[N], const bool (&on)[N], uint32_t (&out)[N], int *fault,
                                         unsigned spin_limit) {
  bool need[N];
#pragma unroll
  for (int i = 0; i < N; ++i) { need[i] = on[i]; out[i] = 0u; }
  unsigned spins = 0;
  for (;;) {
    uint64_t pk[N];
#pragma unroll
    for (int i = 0; i < N; ++i)
      pk[i] = need[i] ? ld_dev64(idx[i] < n0 ? src0 + idx[i] : src1 + (idx[i] - n0)) : 0ull;
    bool pending = false;
#pragma unroll
    for (int i = 0; i < N; ++i) {
      if (need[i]) {
        if ((uint32_t)(pk[i] >> 32) == (idx[i] < n0 ? tag0 : tag1)) { out[i] = (uint32_t)pk[i]; need[i] = false; }
        else pending = true;
      }
    }
    if (!__any(pending)) break;
    __builtin_amdgcn_s_sleep(1);
    if (++spins > (DBG ? spin_limit : kMegaSpinLimit)) {
      __hip_atomic_store(fault, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      break;
    }
    if ((spins & 255u) == 0 && __hip_atomic_load(fault, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) break;
  }
}
template <int KTA, int D, bool PROF>
__global__ void __launch_bounds__(kMegaThreads) k_phi2_decode_step(MegaArgs a) {
  constexpr int NCOL = D / 8;
  constexpr int NG_V = kMegaThreads / NCOL;
  extern __shared__ __attribute__((aligned(16))) unsigned char mg_smem[];
  const int H = KTA * 512, I = a.I, QD = a.QD, KB = QD + I;
  const int KTBC = KB / 512;

  // xa (attention output, QD values) and xs (activations, I values) are adjacent: together they are the input
  // vector of a whole row of Wb (dense columns | fc2 columns).  xa also stages the residual stream for LayerNorm.
  uint16_t *xa = reinterpret_cast<uint16_t *>(mg_smem);
  uint16_t *xs = xa + QD;
  uint16_t *xn = xs + I;
  float *partA = reinterpret_cast<float *>(xn + H);
  float *partB = partA + kMegaRowsAMax * kMegaWaves;
  uint32_t *a1_done = reinterpret_cast<uint32_t *>(partB + kMegaRowsMax * kMegaWaves);   // stream waves past segment A1
  float *qf = partB + 2 * kMegaRowsMax * kMegaWaves;
  float *raw = qf + D;
  float *knew = raw + 3 * D;
  float *vnew = knew + D;
  float *red = vnew + D;
  float *sh = red + NG_V * D;
  float *red2 = sh + 2 * kMegaWaves;
  uint32_t *qh = reinterpret_cast<uint32_t *>(red2);   // q of the current head as packed bf16 (red2 is used after the scores)
  float *scores = red2 + 4 * D;
  float *pd = scores + a.Tmax + 1;
  uint32_t *pkmeta = reinterpret_cast<uint32_t *>(pd + (size_t)a.Tmax * NCOL);   // [9][512]

  const int tid0 = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid0 >> 6);
  const int wg = blockIdx.x, G = gridDim.x;
  int *fault = &a.state->fault;
  int pos = a.state->pos;
  if (pos > a.Tmax - 1) pos = a.Tmax - 1;

  float rope_c = 1.f, rope_s = 0.f;
  if (tid0 < a.rot) {
    rope_c = bf16_bits_to_f32(a.cos_t[(int64_t)pos * a.rot + tid0]);
    rope_s = bf16_bits_to_f32(a.sin_t[(int64_t)pos * a.rot + tid0]);
  }

  // Phase A rows.  Every block takes a share of the q|k|v rows and streams them first (segment A1), so that the
  // attention blocks can start while the fc1 rows (segment A2) are still being streamed; the fc1 rows go to the
  // blocks that run no attention head (to all blocks when every block runs one).  (A head's polls come back behind
  // the weight requests of its own block, loads returning in order.  Two ways around that were measured and are not
  // kept: no q|k|v rows for the blocks with a head, 992 against 986 us per launch; fewer rows for them, consumed from
  // the ring while the refills go to a cached dummy tile and the real requests follow when the head is done: no
  // change.)
  const bool is_attn = wg < a.Hq;
  const int kv_group = a.Hq / a.Hkv;                 // query heads per key/value head (repeat_kv, phi2.rs:190-200)
  const int wg_kv = is_attn ? wg / kv_group : 0;     // the key/value head of this block's query head
  const int KD = a.Hkv * D;
  const int nA0 = 4 * (int)((int64_t)(a.n_qkv / 4) * wg / G), nA1 = 4 * (int)((int64_t)(a.n_qkv / 4) * (wg + 1) / G);
  const int rowsA = nA1 - nA0;
  int fA0 = 0, fA1 = 0;
  {
    const int n_attn_blocks = a.Hq < G ? a.Hq : G;
    const int others = G - n_attn_blocks;
    if (others == 0) {
      fA0 = 4 * (int)((int64_t)(I / 4) * wg / G);
      fA1 = 4 * (int)((int64_t)(I / 4) * (wg + 1) / G);
    } else if (!is_attn) {
      const int o = wg - n_attn_blocks;
      fA0 = 4 * (int)((int64_t)(I / 4) * o / others);
      fA1 = 4 * (int)((int64_t)(I / 4) * (o + 1) / others);
    }
  }
  const int rowsA2 = fA1 - fA0;
  const int nA2 = a.n_qkv + fA0;
  // The activations and the attention output travel three values to a packet ({3 bf16, 16-bit tag}), in slots
  // that belong to their producer: block o of the fc1 producers owns 16 slots (it has at most 48 rows), head h owns
  // kPkHead = ceil(D / 3).  A consumer wants both vectors whole, and 9 packets per thread cover them in one poll.
  constexpr int kPkFc1 = 16, kPkHead = (D + 2) / 3, kPkPoll = 9;
  const int fc1_first = (a.Hq < G ? a.Hq : G) < G ? (a.Hq < G ? a.Hq : G) : 0;   // index of the first fc1 producer
  const int fc1_blocks = G - fc1_first;
  const int fc1_me = wg - fc1_first;
  const int n_attn_pk = a.Hq * kPkHead;
  for (int i = 0; i < kPkPoll; ++i) {   // this thread's packets of the combined poll (the same in every layer)
    const int idx = i * kMegaThreads + tid0;
    int first = 0, count = 0;
    if (idx < n_attn_pk) {
      const int h = idx / kPkHead, p3 = (idx - h * kPkHead) * 3;
      first = h * D + p3;
      count = D - p3;
    } else if (idx < n_attn_pk + fc1_blocks * kPkFc1) {
      const int s2 = idx - n_attn_pk, o = s2 / kPkFc1, p3 = (s2 - o * kPkFc1) * 3;
      const int r0 = 4 * (int)((int64_t)(I / 4) * o / fc1_blocks), r1 = 4 * (int)((int64_t)(I / 4) * (o + 1) / fc1_blocks);
      first = QD + r0 + p3;
      count = r1 - r0 - p3;
    }
    count = count < 0 ? 0 : count > 3 ? 3 : count;
    pkmeta[idx] = (uint32_t)first | ((uint32_t)count << 16);
  }

  int n0, n1;
  {
    const int n_attn_blocks = a.Hq < G ? a.Hq : G;
    const int others = G - n_attn_blocks;
    int ra = others > 0 ? a.rows_attn : (H + n_attn_blocks - 1) / n_attn_blocks;
    if (is_attn) {
      n0 = wg * ra;
      n1 = n0 + ra;
    } else {
      const int base = n_attn_blocks * ra, rem = H - base, o = wg - n_attn_blocks;
      n0 = base + 4 * (int)((int64_t)(rem / 4) * o / others);
      n1 = base + 4 * (int)((int64_t)(rem / 4) * (o + 1) / others);
    }
    if (n0 > H) n0 = H;
    if (n1 > H) n1 = H;
  }
  const int nrows = n1 - n0;

  const int ttA = rowsA * KTA, ttA2 = rowsA2 * KTA, ttB = nrows * KTBC;
  const bool streams = wave < kMegaStream;
  const int tA0 = streams ? ttA * wave / kMegaStream : 0, tA1 = streams ? ttA * (wave + 1) / kMegaStream : 0;
  const int tA2_0 = streams ? ttA2 * wave / kMegaStream : 0, tA2_1 = streams ? ttA2 * (wave + 1) / kMegaStream : 0;
  const int tB0 = streams ? ttB * wave / kMegaStream : 0, tB1 = streams ? ttB * (wave + 1) / kMegaStream : 0;
  const int ttA_w = (tA1 - tA0) + (tA2_1 - tA2_0), ttB_w = tB1 - tB0;   // this wave's tiles per layer: Wa, Wb

  mg_u32x4 ring[kMegaRing];
  mg_u32x4 kreg[kMegaUK], vreg[kMegaUV];
  // A stream wave whose phases all hold at least one pass over the ring (or nothing) also keeps kMegaStage tiles
  // in LDS: requested when the wave starts to wait with a full ring, consumed first when it streams again.
  unsigned char *const stage = mg_smem + a.stage_off + wave * (kMegaStage * 1024);
  const bool stages = a.stage_off != 0 && streams && ttA_w + ttB_w > 0 && (ttA_w == 0 || ttA_w >= kMegaRing) &&
                      (ttB_w == 0 || ttB_w >= kMegaRing);
  bool staged = false;

  MgSplit sp;
  sp.Wa0 = a.Wa0; sp.Wb0 = a.Wb0; sp.wa_stride = a.wa_stride; sp.wb_stride = a.wb_stride; sp.L = a.L; sp.H = H; sp.KB = KB; sp.KTA = KTA; sp.KTBC = KTBC;
  sp.cnt0 = tA1 - tA0; sp.cnt1 = tA2_1 - tA2_0; sp.cnt2 = tB1 - tB0;
  sp.kc0 = tA0 % KTA; sp.kc1 = tA2_0 % KTA; sp.kc2 = tB0 % KTBC;
  sp.off0 = (int64_t)(nA0 + tA0 / KTA) * H; sp.off1 = (int64_t)(nA2 + tA2_0 / KTA) * H; sp.off2 = (int64_t)(n0 + tB0 / KTBC) * KB;
  {
    const bool e0 = sp.cnt0 > 0, e1 = sp.cnt1 > 0, e2 = sp.cnt2 > 0;
    sp.nx0 = e1 ? 1 : e2 ? 2 : 0;
    sp.nx1 = e2 ? 2 : e0 ? 0 : 1;
    sp.nx2 = e0 ? 0 : e1 ? 1 : 2;
  }
  MgCursor cur;
  cur.layer = 0; cur.seg = 0; cur.kc = 0; cur.KT = 1; cur.left = 0; cur.jump = 0; cur.step = 0;
  cur.ptr = a.Wa0;
  const bool streams_any = streams && ttA_w + ttB_w > 0;   // (a wave without tiles never requests one)
  if (streams_any) mg_seg_enter(cur, sp, 0, sp.cnt0 > 0 ? 0 : sp.cnt1 > 0 ? 1 : 2);
  const MgPhase phA = mg_phase(tA0, tA1, tA2_0, tA2_1, KTA), phB = mg_phase(tB0, tB1, 0, 0, KTBC);
  unsigned bar = 0;
  int pending_rot = 0;
  const uint32_t tagbase = a.state->epoch * kMegaTagsPerLaunch;   // exchange tags of this launch: tagbase + index + 1
  uint32_t tag_x = 0;                                // tag of the residual-stream packets of the previous layer
  const float att_scale = a.scale;
  unsigned long long *const prof = a.prof;
  const int n_layers = a.L;

  auto k_load = [&](const uint16_t *Kc, int q0) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < kMegaUK; ++u) {
      const int q = q0 + kMegaThreads * u;
      kreg[u] = q < pos * NCOL ? mg_ldw(Kc + (int64_t)q * 8) : MG_ZERO4;
    }
  };

  auto k_partials = [&](int q0) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < kMegaUK; ++u) {
      const int q = q0 + kMegaThreads * u;
      if (q < pos * NCOL) {
        const int c = q % NCOL;
        // q after the rotary embedding is exactly representable in bf16 (the reference rounds it to the model
        // dtype before the upcast, phi2.rs:244-247), so the products equal the f32 ones
        const mg_u32x4 q4 = *reinterpret_cast<const mg_u32x4 *>(qh + c * 4);
        const float acc = mg_dot8(kreg[u], q4, 0.f);
        pd[q] = acc;
      }
    }
  };

  auto v_load = [&](const uint16_t *Vc, int tb, int col, bool active) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < kMegaUV; ++u) {
      const int t = tb + NG_V * u;
      vreg[u] = (active && t < pos) ? mg_ldw(Vc + (int64_t)t * D + col * 8) : MG_ZERO4;
    }
  };
  auto v_accum = [&](int tb, float(&acc)[8]) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < kMegaUV; ++u) {
      const int t = tb + NG_V * u;
      const float p = t < pos ? scores[t] : 0.f;
      const uint32_t w4[4] = {vreg[u].x, vreg[u].y, vreg[u].z, vreg[u].w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        acc[2 * j] = fmaf(p, __uint_as_float(w4[j] << 16), acc[2 * j]);
        acc[2 * j + 1] = fmaf(p, __uint_as_float(w4[j] & 0xffff0000u), acc[2 * j + 1]);
      }
    }
  };

  auto stamp = [&](int l, int k) __attribute__((always_inline)) {
    if constexpr (PROF) {
      if (threadIdx.x == kMegaService * 64) prof[((int64_t)wg * n_layers + l) * 16 + k] = wall_clock64();
    }
  };

  auto stage_ahead = [&](int lane) __attribute__((always_inline)) {
    if (stages && !staged) {
#pragma unroll
      for (int j = 0; j < kMegaStage; ++j) mg_next_stage(cur, sp, lane, stage + j * 1024);
      staged = true;
    }
  };

  for (int e = tid0; e < kMegaRowsAMax * kMegaWaves; e += kMegaThreads) partA[e] = 0.f;
  if (tid0 == 0) *a1_done = 0u;

  {
    const int lane = tid0 & 63;
#pragma unroll
    for (int p = 0; p < kMegaRing; ++p) {
      ring[p] = streams_any ? mg_next_load(cur, sp, lane) : MG_ZERO4;
    }
  }
#pragma unroll
  for (int u = 0; u < kMegaUK; ++u) kreg[u] = MG_ZERO4;
#pragma unroll
  for (int u = 0; u < kMegaUV; ++u) vreg[u] = MG_ZERO4;

  for (int l = 0; l < a.L; ++l) {
    const MegaLayer ly = a.layers[l];
    // (a block without a head never touches the cache; wg_kv is only meaningful where is_attn)
    uint16_t *Kc = a.kcache + ((int64_t)l * a.kv_layer_stride) + (int64_t)wg_kv * a.Tmax * D;
    uint16_t *Vc = a.vcache + ((int64_t)l * a.kv_layer_stride) + (int64_t)wg_kv * a.Tmax * D;

    stamp(l, 0);
    {
      const int tid = mg_opaque(tid0), lane = tid & 63;
      const bool service = wave == kMegaService;
      stage_ahead(lane);   // the ring is full: the wait for the residual stream fetches the tiles behind it into LDS
      // An attention block requests the cached keys and values of its head first: they do not depend on this
      // layer's inputs, one CU can only keep so many cache lines in flight (the ~200 KB take several memory
      // round trips), and the block would otherwise just wait for the residual stream.
      if (is_attn) {
        const int col = tid % NCOL, grp = tid / NCOL;
        k_load(Kc, tid);
        v_load(Vc, grp, col, grp < NG_V);
      }

      uint64_t bias_a = 0, bias_a2 = 0;
      if (service && lane * 4 < rowsA) bias_a = *reinterpret_cast<const uint64_t *>(ly.ba + nA0 + lane * 4);
      if (service) {   // rows 3 lane .. 3 lane + 2 of this block's fc1 share
#pragma unroll
        for (int j = 0; j < 3; ++j)
          if (lane * 3 + j < rowsA2) bias_a2 |= (uint64_t)ly.ba[nA2 + lane * 3 + j] << (16 * j);
      }
      if (tid < kMegaRowsMax * kMegaWaves) partB[tid] = 0.f;
      if (tid == 0) *a1_done = 0u;
      // the residual stream into LDS (xa is free until phase C): the plain vector for layer 0 (written
      // before this launch), else the packets of the previous layer's last phase, polled by all threads
      if (l == 0) {
        for (int i = tid; i < H / 2; i += kMegaThreads) reinterpret_cast<uint32_t *>(xa)[i] = ld_dev32(a.x + 2 * i);
      } else {
        for (int base = 0; base < H / 2; base += kMegaThreads * 4) {
          int idx[4];
          bool on[4];
          uint32_t val[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) { idx[i] = base + i * kMegaThreads + tid; on[i] = idx[i] < H / 2; }
          mg_poll<4, PROF>(a.xp, idx, on, tag_x, val, fault, a.spin_limit);
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (on[i]) reinterpret_cast<uint32_t *>(xa)[idx[i]] = val[i];
        }
      }
      stamp(l, 8);   // the residual stream has arrived
      wg_sync();
      if (wave < KTA) {

        mg_u32x4 xv[KTA];
#pragma unroll
        for (int u = 0; u < KTA; ++u) xv[u] = *reinterpret_cast<const mg_u32x4 *>(xa + u * 512 + lane * 8);
        const mg_u32x4 lw = *reinterpret_cast<const mg_u32x4 *>(ly.ln_w + wave * 512 + lane * 8);
        const mg_u32x4 lb = *reinterpret_cast<const mg_u32x4 *>(ly.ln_b + wave * 512 + lane * 8);

        const uint32_t ones = 0x3f803f80u;
        float s1 = 0.f, s2 = 0.f;
        mg_u32x4 mine = MG_ZERO4;
#pragma unroll
        for (int u = 0; u < KTA; ++u) {
          const uint32_t w4[4] = {xv[u].x, xv[u].y, xv[u].z, xv[u].w};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            s1 = mg_dot2(w4[j], ones, s1);
            s2 = mg_dot2(w4[j], w4[j], s2);
          }
          if (wave == u) mine = xv[u];
        }
        s1 = mg_wave_sum(s1);
        s2 = mg_wave_sum(s2);
        const float mean = s1 / (float)H;
        float var = s2 / (float)H - mean * mean;
        var = var > 0.f ? var : 0.f;
        const float scale = 1.0f / sqrtf(var + a.ln_eps), shift = -mean * scale;
        const uint32_t xx[4] = {mine.x, mine.y, mine.z, mine.w};
        const uint32_t ww[4] = {lw.x, lw.y, lw.z, lw.w};
        const uint32_t bb[4] = {lb.x, lb.y, lb.z, lb.w};
        uint32_t o[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float y0 = fmaf(fmaf(__uint_as_float(xx[j] << 16), scale, shift), __uint_as_float(ww[j] << 16),
                                __uint_as_float(bb[j] << 16));
          const float y1 = fmaf(fmaf(__uint_as_float(xx[j] & 0xffff0000u), scale, shift),
                                __uint_as_float(ww[j] & 0xffff0000u), __uint_as_float(bb[j] & 0xffff0000u));
          o[j] = pack_bf16x2(y0, y1);
        }
        *reinterpret_cast<mg_u32x4 *>(xn + wave * 512 + lane * 8) = mg_u32x4{o[0], o[1], o[2], o[3]};
      }
      wg_sync();
      // The service wave turns the partial sums of a finished segment into packets (bias; activation for the
      // fc1 rows).  It does so for the q|k|v rows as soon as every stream wave has left segment A1, while those
      // waves stream the fc1 rows: the attention blocks get their inputs a whole segment early.
      auto publish_a = [&](int n_first, int rows, const float *part, uint64_t bias, bool is_fc1) __attribute__((always_inline)) {
        if (service && lane * 4 < rows) {
          const int n = n_first + lane * 4;
          uint32_t packed[2];
#pragma unroll
          for (int h2 = 0; h2 < 2; ++h2) {
            float v[2];
#pragma unroll
            for (int k = 0; k < 2; ++k) {
              const int e = lane * 4 + h2 * 2 + k;
              float s4 = __uint_as_float((uint32_t)((bias >> (16 * (h2 * 2 + k))) & 0xffffu) << 16);
#pragma unroll
              for (int w = 0; w < kMegaStream; ++w) s4 += part[e * kMegaWaves + w];
              if (is_fc1) s4 = act_eval(a.act, s4);
              v[k] = s4;
            }
            packed[h2] = pack_bf16x2(v[0], v[1]);
          }
          uint64_t *dst = is_fc1 ? a.actp + ((n - a.n_qkv) >> 1) : a.qkvp + (n >> 1);
          const uint64_t tg = (uint64_t)(tagbase + bar + 1u) << 32;
          if (!PROF || wg != a.mute_block) {
            st_dev64(dst, tg | packed[0]);
            st_dev64(dst + 1, tg | packed[1]);
          }
        }
      };
      // the ring is rotated only now, just before it is consumed again: a rotation moves registers that loads
      // are still writing, i.e. it waits for the newest of them, and by now those have had a whole exchange to land
      mg_rotate_by(ring, pending_rot);
      pending_rot = mg_run_phase(ring, cur, sp, phA, KTA, xn, partA, partA + rowsA * kMegaWaves, a1_done, lane, wave,
                                 stage, staged);
      if (service) {   // its own ranges are empty: it arrives here at once and waits for the seven others
        unsigned spins = 0;
        while (__hip_atomic_load(a1_done, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) < (uint32_t)kMegaWaves) {
          __builtin_amdgcn_s_sleep(1);
          if (++spins > kMegaSpinLimit) {
            __hip_atomic_store(fault, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            break;
          }
        }
        publish_a(nA0, rowsA, partA, bias_a, false);
        stamp(l, 9);   // q|k|v rows of this block published
      }
      wg_sync();
      if (service && lane * 3 < rowsA2) {   // gelu(fc1) of this block's rows, three to a packet
        const float *part = partA + rowsA * kMegaWaves;
        uint32_t hv[3] = {0u, 0u, 0u};
#pragma unroll
        for (int j = 0; j < 3; ++j) {
          const int e = lane * 3 + j;
          if (e < rowsA2) {
            float s4 = __uint_as_float((uint32_t)((bias_a2 >> (16 * j)) & 0xffffu) << 16);
#pragma unroll
            for (int w = 0; w < kMegaStream; ++w) s4 += part[e * kMegaWaves + w];
            hv[j] = f32_to_bf16_bits(act_eval(a.act, s4));
          }
        }
        const uint64_t tg = (uint64_t)((tagbase + bar + 1u) & 0xffffu) << 48;
        if (!PROF || wg != a.mute_block)
          st_dev64(a.actp + fc1_me * kPkFc1 + lane, tg | ((uint64_t)hv[2] << 32) | ((uint64_t)hv[1] << 16) | hv[0]);
      }
      stamp(l, 1);
      ++bar;   // no barrier: phase B polls the packets it needs
      wg_sync();
      stamp(l, 2);
    }

    {
      const int tid = mg_opaque(tid0), lane = tid & 63;
      for (int e = tid; e < kMegaRowsAMax * kMegaWaves; e += kMegaThreads) partA[e] = 0.f;

      const uint32_t tag_a = tagbase + bar;   // bar was advanced past the A -> B exchange: its tag is index + 1
      // (a block with rows of Wb polls the activations together with the attention output, further down)
      if (is_attn) {
        const int h = wg;
        {
          const int which = tid / (D / 2), pe = tid - which * (D / 2);
          // q of head h at h D; k and v of its key/value head behind the QD query rows and the KD key rows
          int idx[1] = {(which == 0 ? h * D : which == 1 ? QD + wg_kv * D : QD + KD + wg_kv * D) / 2 + pe};
          bool on[1] = {tid < 3 * D / 2};
          if (!on[0]) idx[0] = 0;
          uint32_t val[1];
          mg_poll<1, PROF>(a.qkvp, idx, on, tag_a, val, fault, a.spin_limit);
          if (on[0]) {
            raw[which * D + 2 * pe] = __uint_as_float(val[0] << 16);
            raw[which * D + 2 * pe + 1] = __uint_as_float(val[0] & 0xffff0000u);
          }
        }
        stamp(l, 10);
        wg_sync();
        if (tid < D) {
          const float qr = mg_rope(raw, tid, a.rot, rope_c, rope_s);
          const float kr = mg_rope(raw + D, tid, a.rot, rope_c, rope_s);
          const float vr = raw[2 * D + tid];
          qf[tid] = qr;
          reinterpret_cast<uint16_t *>(qh)[tid] = f32_to_bf16_bits(qr);   // exact: qr carries bf16 precision
          knew[tid] = kr;
          vnew[tid] = vr;
          if (wg % kv_group == 0) {   // one of the heads that share the key/value head appends the new row
            Kc[(int64_t)pos * D + tid] = f32_to_bf16_bits(kr);
            Vc[(int64_t)pos * D + tid] = f32_to_bf16_bits(vr);
          }
        }
        wg_sync();

        {
          constexpr int RKP = kMegaThreads * kMegaUK;
          for (int qb = 0; qb < pos * NCOL; qb += RKP) {
            if (qb > 0) k_load(Kc, qb + tid);
            k_partials(qb + tid);
          }
        }
        stamp(l, 11);
        wg_sync();
        for (int t = tid; t < pos; t += kMegaThreads) {
          float sc = 0.f;
#pragma unroll
          for (int c = 0; c < NCOL; ++c) sc += pd[t * NCOL + c];
          scores[t] = sc * att_scale;
        }
        if (wave == kMegaWaves - 1) {
          float acc = 0.f;
          for (int d = lane; d < D; d += 64) acc = fmaf(qf[d], knew[d], acc);
          acc = mg_wave_sum(acc);
          if (lane == 0) scores[pos] = acc * att_scale;
        }
        wg_sync();
        const int cnt = pos + 1;
        float m = -(__builtin_inff ());
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
        stamp(l, 12);

        {
          const int col = tid % NCOL, grp = tid / NCOL;
          const bool active = grp < NG_V;
          constexpr int RV = NG_V * kMegaUV;
          float acc[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) acc[j] = 0.f;
          for (int tb = 0; tb < pos; tb += RV) {
            if (tb > 0) v_load(Vc, tb + grp, col, active);
            v_accum(tb + grp, acc);
          }
          if (active) {
#pragma unroll
            for (int j = 0; j < 8; ++j) red[grp * D + col * 8 + j] = acc[j];
          }
        }
        wg_sync();

        if (tid < 4 * D) {
          const int d = tid % D, q4 = tid / D;
          float r = 0.f;
          for (int gg = q4; gg < NG_V; gg += 4) r += red[gg * D + d];
          red2[tid] = r;
        }
        wg_sync();
        if (wave == kMegaService && lane < kPkHead) {
          const float inv = 1.0f / sum, p_new = scores[pos];
          uint32_t hv[3] = {0u, 0u, 0u};
#pragma unroll
          for (int k = 0; k < 3; ++k) {
            const int d = 3 * lane + k;
            if (d < D)
              hv[k] = f32_to_bf16_bits((p_new * vnew[d] + red2[d] + red2[D + d] + red2[2 * D + d] + red2[3 * D + d]) * inv);
          }
          const uint64_t tg = (uint64_t)((tagbase + bar + 1u) & 0xffffu) << 48;
          st_dev64(a.attnp + h * kPkHead + lane, tg | ((uint64_t)hv[2] << 32) | ((uint64_t)hv[1] << 16) | hv[0]);
        }
        stamp(l, 13);
      }
      // ---- rows of Wb: [attention output | activations] . [dense columns | fc2 columns], one stream
      const bool service = wave == kMegaService;
      stage_ahead(lane);   // (an attention block is past its head here: nothing of its own waits behind these loads)
      uint64_t res4 = 0, bd4 = 0, bf4 = 0;
      if (service && lane * 4 < nrows) {
        res4 = ld_dev64(a.x + n0 + lane * 4);
        bd4 = *reinterpret_cast<const uint64_t *>(ly.bd + n0 + lane * 4);
        bf4 = *reinterpret_cast<const uint64_t *>(ly.bf + n0 + lane * 4);
      }
      const uint32_t tag_b = tagbase + bar + 1u;
      ++bar;
      // one list of packets: Hq * kPkHead of the attention output, then fc1_blocks * kPkFc1 of the activations;
      // nine per thread cover it in one poll, i.e. one memory round trip when everything has arrived.  Where a
      // packet's values go in [xa | xs] and how many of its three are real sits in pkmeta (filled at kernel start).
      if (nrows > 0) {
        uint64_t pk[kPkPoll];
        uint32_t need = 0u;
#pragma unroll
        for (int i = 0; i < kPkPoll; ++i) {
          pk[i] = 0ull;
          if ((pkmeta[i * kMegaThreads + tid] >> 16) != 0u) need |= 1u << i;
        }
        const uint32_t t16a = tag_b & 0xffffu, t16f = tag_a & 0xffffu;
        unsigned spins = 0;
        for (;;) {
#pragma unroll
          for (int i = 0; i < kPkPoll; ++i) {
            const int idx = i * kMegaThreads + tid;
            if (need & (1u << i)) pk[i] = ld_dev64(idx < n_attn_pk ? a.attnp + idx : a.actp + (idx - n_attn_pk));
          }
#pragma unroll
          for (int i = 0; i < kPkPoll; ++i) {
            const int idx = i * kMegaThreads + tid;
            if ((need & (1u << i)) && (uint32_t)(pk[i] >> 48) == (idx < n_attn_pk ? t16a : t16f)) need &= ~(1u << i);
          }
          if (!__any(need != 0u)) break;
          __builtin_amdgcn_s_sleep(1);
          if (++spins > (PROF ? a.spin_limit : kMegaSpinLimit)) {
            __hip_atomic_store(fault, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            break;
          }
          if ((spins & 255u) == 0 && __hip_atomic_load(fault, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) break;
        }
#pragma unroll
        for (int i = 0; i < kPkPoll; ++i) {
          const uint32_t meta = pkmeta[i * kMegaThreads + tid];
          const uint32_t first = meta & 0xffffu, count = meta >> 16;
          if (count > 0) xa[first] = (uint16_t)(pk[i] & 0xffffu);
          if (count > 1) xa[first + 1] = (uint16_t)((pk[i] >> 16) & 0xffffu);
          if (count > 2) xa[first + 2] = (uint16_t)((pk[i] >> 32) & 0xffffu);
        }
      }
      wg_sync();
      stamp(l, 3);
      mg_rotate_by(ring, pending_rot);
      pending_rot = mg_run_phase(ring, cur, sp, phB, KTBC, xa, partB, partB, nullptr, lane, wave, stage, staged);
      stamp(l, 4);
      wg_sync();
      stamp(l, 5);

      if (service && lane * 4 < nrows) {
        auto elem = [](uint64_t v, int k) { return __uint_as_float((uint32_t)((v >> (16 * k)) & 0xffffu) << 16); };
        float v[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const int e = lane * 4 + k;
          float sacc = 0.f;
#pragma unroll
          for (int w = 0; w < kMegaStream; ++w) sacc += partB[e * kMegaWaves + w];
          v[k] = sacc + (elem(bd4, k) + elem(bf4, k)) + elem(res4, k);
        }
        const uint32_t lo = pack_bf16x2(v[0], v[1]), hi = pack_bf16x2(v[2], v[3]);
        st_dev64(a.x + n0 + lane * 4, (uint64_t)lo | ((uint64_t)hi << 32));   // plain copy: this block's residual, and the head's input
        const uint64_t tg = (uint64_t)(tagbase + bar + 1u) << 32;
        st_dev64(a.xp + ((n0 + lane * 4) >> 1), tg | lo);
        st_dev64(a.xp + ((n0 + lane * 4) >> 1) + 1, tg | hi);
      }
      tag_x = tagbase + bar + 1u;
      ++bar;
      stamp(l, 6);
      if (l + 1 < a.L) wg_sync();   // no grid barrier: the next layer's LayerNorm polls the packets
      stamp(l, 7);
    }
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);   // nothing still on its way into LDS when the block ends
}

// ---- the head behind the step -------------------------------------------------------------------------------------
// logits = LayerNorm(x) . W^T + bias for one row, and the greedy choice on them, in one launch of one block per CU.
// Every block normalises x once (as the step kernel does at the start of a layer), streams its share of the rows of W
// through the same register ring (seven stream waves as there: with all eight streaming the launch took 48 us
// instead of 43; the first sixteen tiles are requested before x is even read),
// rounds its logits to bf16, stores them and keeps the best of them: the first maximum, NaNs passed over, except
// that a NaN in row 0 takes the choice (what a scan from element 0 that replaces on a strict comparison gives).  The
// blocks' bests travel as 8-byte (value, row) words written past the L2; a block counts itself in when its word has
// reached memory, and the block that counts last, whichever it is, picks among the words, writes the token, copies
// its embedding row to the next step's input and advances the device-side counters.  Nobody waits for anybody.
constexpr int kHeadRowsMax = 256;

// whether candidate (v, i) replaces (bv, bi): a NaN value only ever comes with row 0 and is final; row 0xffffffff
// means nothing seen yet
__device__ __forceinline__ bool head_replaces(float v, uint32_t i, float bv, uint32_t bi) {
  if (bv != bv) return false;
  if (v != v) return true;
  if (i == 0xffffffffu) return false;
  return bi == 0xffffffffu || v > bv || (v == bv && i < bi);
}

template <int KTA>
__global__ void __launch_bounds__(kMegaThreads) k_phi2_head_choice(HeadArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char hd_smem[];
  constexpr int H = KTA * 512;
  uint16_t *xr = reinterpret_cast<uint16_t *>(hd_smem);   // x as it is
  uint16_t *xn = xr + H;                                   // LayerNorm(x), bf16
  float *part = reinterpret_cast<float *>(xn + H);         // [rows][kMegaWaves]
  __shared__ float s_v[kMegaWaves];
  __shared__ uint32_t s_i[kMegaWaves];
  __shared__ int s_ticket;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wg = blockIdx.x, G = gridDim.x;
  const int r0 = (int)((int64_t)a.V * wg / G), r1 = (int)((int64_t)a.V * (wg + 1) / G);
  const int nrows = r1 - r0;

  const bool streams = wave < kMegaStream;
  const int tt = nrows * KTA;
  const int t0 = streams ? tt * wave / kMegaStream : 0, t1 = streams ? tt * (wave + 1) / kMegaStream : 0;
  MgSplit sp;
  sp.Wa0 = a.W; sp.Wb0 = a.W; sp.wa_stride = 0; sp.wb_stride = 0; sp.L = 1; sp.H = H; sp.KB = H; sp.KTA = KTA; sp.KTBC = 1;
  sp.cnt0 = t1 - t0; sp.cnt1 = 0; sp.cnt2 = 0;
  sp.kc0 = t0 % KTA; sp.kc1 = 0; sp.kc2 = 0;
  sp.off0 = (int64_t)(r0 + t0 / KTA) * H; sp.off1 = 0; sp.off2 = 0;
  sp.nx0 = 0; sp.nx1 = 0; sp.nx2 = 0;
  MgCursor cur;
  cur.layer = 0; cur.seg = 0; cur.kc = 0; cur.KT = 1; cur.left = 0; cur.jump = 0; cur.step = 0;
  cur.ptr = a.W;
  const bool streams_any = sp.cnt0 > 0;
  if (streams_any) mg_seg_enter(cur, sp, 0, 0);
  const MgPhase ph = mg_phase(t0, t1, 0, 0, KTA);
  mg_u32x4 ring[kMegaRing];
#pragma unroll
  for (int p = 0; p < kMegaRing; ++p) ring[p] = streams_any ? mg_next_load(cur, sp, lane) : MG_ZERO4;

  // x into LDS, the partial sums to zero (a wave leaves one per row it touches)
  for (int i = tid; i < H / 2; i += kMegaThreads) reinterpret_cast<uint32_t *>(xr)[i] = reinterpret_cast<const uint32_t *>(a.x)[i];
  for (int e = tid; e < nrows * kMegaWaves; e += kMegaThreads) part[e] = 0.f;
  wg_sync();
  if (wave < KTA) {   // wave u normalises features [512 u, 512 u + 512); every one of them computes the statistics
    mg_u32x4 xv[KTA];
#pragma unroll
    for (int u = 0; u < KTA; ++u) xv[u] = *reinterpret_cast<const mg_u32x4 *>(xr + u * 512 + lane * 8);
    const mg_u32x4 lw = *reinterpret_cast<const mg_u32x4 *>(a.ln_w + wave * 512 + lane * 8);
    const mg_u32x4 lb = *reinterpret_cast<const mg_u32x4 *>(a.ln_b + wave * 512 + lane * 8);
    const uint32_t ones = 0x3f803f80u;
    float s1 = 0.f, s2 = 0.f;
    mg_u32x4 mine = MG_ZERO4;
#pragma unroll
    for (int u = 0; u < KTA; ++u) {
      const uint32_t w4[4] = {xv[u].x, xv[u].y, xv[u].z, xv[u].w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        s1 = mg_dot2(w4[j], ones, s1);
        s2 = mg_dot2(w4[j], w4[j], s2);
      }
      if (wave == u) mine = xv[u];
    }
    s1 = mg_wave_sum(s1);
    s2 = mg_wave_sum(s2);
    const float mean = s1 / (float)H;
    float var = s2 / (float)H - mean * mean;
    var = var > 0.f ? var : 0.f;
    const float scale = 1.0f / sqrtf(var + a.ln_eps), shift = -mean * scale;
    const uint32_t xx[4] = {mine.x, mine.y, mine.z, mine.w};
    const uint32_t ww[4] = {lw.x, lw.y, lw.z, lw.w};
    const uint32_t bb[4] = {lb.x, lb.y, lb.z, lb.w};
    uint32_t o[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float y0 = fmaf(fmaf(__uint_as_float(xx[j] << 16), scale, shift), __uint_as_float(ww[j] << 16), __uint_as_float(bb[j] << 16));
      const float y1 = fmaf(fmaf(__uint_as_float(xx[j] & 0xffff0000u), scale, shift), __uint_as_float(ww[j] & 0xffff0000u),
                            __uint_as_float(bb[j] & 0xffff0000u));
      o[j] = pack_bf16x2(y0, y1);
    }
    *reinterpret_cast<mg_u32x4 *>(xn + wave * 512 + lane * 8) = mg_u32x4{o[0], o[1], o[2], o[3]};
  }
  wg_sync();

  bool staged = false;
  (void)mg_run_phase(ring, cur, sp, ph, KTA, xn, part, part, nullptr, lane, wave, nullptr, staged);
  wg_sync();

  // this block's logits and the best of them
  float bv = -INFINITY;
  uint32_t bi = 0xffffffffu;
  for (int e = tid; e < nrows; e += kMegaThreads) {
    float sacc = 0.f;
#pragma unroll
    for (int w = 0; w < kMegaStream; ++w) sacc += part[e * kMegaWaves + w];
    if (a.bias) sacc += bf16_bits_to_f32(a.bias[r0 + e]);
    const uint16_t vb = f32_to_bf16_bits(sacc);
    a.logits[r0 + e] = vb;
    const float r = bf16_bits_to_f32(vb);
    const uint32_t n = (uint32_t)(r0 + e);
    if (r != r) {
      if (n == 0u) { bv = r; bi = 0u; }
    } else if (head_replaces(r, n, bv, bi)) {
      bv = r;
      bi = n;
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(bv, o, 64);
    const uint32_t oi = (uint32_t)__shfl_xor((int)bi, o, 64);
    if (head_replaces(ov, oi, bv, bi)) { bv = ov; bi = oi; }
  }
  if (lane == 0) { s_v[wave] = bv; s_i[wave] = bi; }
  wg_sync();
  if (tid == 0) {
#pragma unroll
    for (int w = 1; w < kMegaWaves; ++w)
      if (head_replaces(s_v[w], s_i[w], bv, bi)) { bv = s_v[w]; bi = s_i[w]; }
    st_dev64(a.best + wg, ((uint64_t)__float_as_uint(bv) << 32) | bi);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the word has reached memory before this block counts itself in
    s_ticket = __hip_atomic_fetch_add(&a.state->done, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  wg_sync();
  if (s_ticket != G - 1) return;

  // the last block: every word is in memory
  if (tid == 0) __hip_atomic_store(&a.state->done, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // for the next launch
  bv = -INFINITY;
  bi = 0xffffffffu;
  for (int p = tid; p < G; p += kMegaThreads) {
    const uint64_t pk = ld_dev64(a.best + p);
    const float v = __uint_as_float((uint32_t)(pk >> 32));
    const uint32_t i = (uint32_t)pk;
    if (head_replaces(v, i, bv, bi)) { bv = v; bi = i; }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(bv, o, 64);
    const uint32_t oi = (uint32_t)__shfl_xor((int)bi, o, 64);
    if (head_replaces(ov, oi, bv, bi)) { bv = ov; bi = oi; }
  }
  if (lane == 0) { s_v[wave] = bv; s_i[wave] = bi; }
  wg_sync();
  bv = s_v[0];
  bi = s_i[0];
#pragma unroll
  for (int w = 1; w < kMegaWaves; ++w)
    if (head_replaces(s_v[w], s_i[w], bv, bi)) { bv = s_v[w]; bi = s_i[w]; }
  const uint32_t chosen = bi == 0xffffffffu ? 0u : bi;   // (every logit NaN)
  if (a.x_next) {
    const uint16_t *row = a.embed + (int64_t)chosen * H;
    for (int k = tid; k < H; k += kMegaThreads)
      a.x_next[k] = a.embed_scale != 1.0f ? f32_to_bf16_bits(bf16_bits_to_f32(row[k]) * a.embed_scale) : row[k];
  }
  if (tid == 0) {
    *a.token = chosen;
    if (a.history) a.history[a.state->step] = chosen;
    a.state->epoch += 1u;   // the next launch of the step kernel tags its packets differently
    a.state->pos += a.dpos;
    a.state->step += a.dstep;
  }
}

static size_t head_lds_bytes(const HeadArgs &a, int num_cu) {
  const int rows = (a.V + num_cu - 1) / num_cu + 1;
  return (size_t)a.H * 4 + (size_t)rows * kMegaWaves * sizeof(float);
}

bool head_choice_eligible(const HeadArgs &a, int num_cu) {
  if (!(a.H == 2560 || a.H == 2048) || num_cu < 1 || num_cu > 256) return false;
  if (a.V < num_cu * 16 || (a.V + num_cu - 1) / num_cu + 1 > kHeadRowsMax) return false;   // at least a pass over the ring per wave
  auto al16 = [](const void *p) { return ((uintptr_t)p & 15) == 0; };
  return a.W && a.x && a.ln_w && a.ln_b && a.logits && a.best && a.token && a.state && al16(a.W) && al16(a.x) && al16(a.ln_w) &&
         al16(a.ln_b) && (!a.x_next || a.embed);
}

int launch_phi2_head_choice(hipStream_t st, const HeadArgs &a, int num_cu) {
  RAI_REQUIRE(head_choice_eligible(a, num_cu), RAI_ERR_UNSUPPORTED, "head with choice: H=%d V=%d on %d CUs not served", a.H, a.V, num_cu);
  const size_t lds = head_lds_bytes(a, num_cu);
  if (a.H == 2560) hipLaunchKernelGGL((k_phi2_head_choice<5>), dim3(num_cu), dim3(kMegaThreads), lds, st, a);
  else hipLaunchKernelGGL((k_phi2_head_choice<4>), dim3(num_cu), dim3(kMegaThreads), lds, st, a);
  return launch_check("phi2_head_choice");
}

size_t mega_lds_bytes(const MegaArgs &a, int D) {
  const int NG_V = kMegaThreads / (D / 8);
  size_t n = (size_t)(a.I + a.QD + a.H) * 2;
  n += sizeof(float) * ((kMegaRowsAMax + 2 * kMegaRowsMax) * kMegaWaves + 6 * (size_t)D + (size_t)NG_V * D +
                        2 * kMegaWaves + 4 * (size_t)D + (size_t)a.Tmax + 1 + (size_t)a.Tmax * (D / 8) + 9 * kMegaThreads);
  return (n + 15) & ~(size_t)15;
}

unsigned mega_default_spin_limit() { return kMegaSpinLimit; }

bool mega_eligible(const MegaArgs &a, int D, int num_cu, const char **why) {
  auto no = [&](const char *w) { if (why) *why = w; return false; };
  // the widths the kernel is built for: Phi-2 (2560 = 32 heads x 80) and Phi-1 / Phi-1.5 (2048 = 32 heads x 64)
  if (!((a.H == 2560 && D == 80) || (a.H == 2048 && D == 64))) return no("hidden size / head_dim is neither 2560 / 80 nor 2048 / 64");
  if (a.Hq * D != a.QD || a.QD % 512 || a.I % 512) return no("projection widths are not multiples of 512");
  if (a.Hq > num_cu || num_cu > 256) return no("more heads than CUs, or more than 256 CUs");
  if (a.Hkv < 1 || a.Hq % a.Hkv) return no("query heads are not a multiple of the key/value heads");
  if (a.n_qkv != a.QD + 2 * a.Hkv * D || a.NA != a.n_qkv + a.I || a.n_qkv % 4 || a.NA % 4) return no("q|k|v layout");
  if (a.rot > D || (a.rot & 1)) return no("rotary_dim");
  if (3 * a.L >= (int)kMegaTagsPerLaunch) return no("too many layers for the exchange tags of one launch");

  const int others = num_cu - a.Hq;
  const int ra = others > 0 ? a.rows_attn : (a.H + a.Hq - 1) / a.Hq;
  if (ra < 0 || ra > kMegaRowsMax || ra % 4) return no("rows_attn");
  if (others > 0) {
    const int rem = a.H - a.Hq * ra;
    if (rem < 0 || rem / others + 4 > kMegaRowsMax) return no("too many rows per block");
  }
  {
    const int fc1_blocks = others > 0 ? others : num_cu;
    if (a.n_qkv / num_cu + 4 + a.I / fc1_blocks + 4 > kMegaRowsAMax) return no("too many phase A rows per block");
    // three-value packets: 16 slots per fc1 producer, ceil(D / 3) per head, inside the packet arrays of I / 2 and QD / 2
    if (4 * ((a.I / 4 + fc1_blocks - 1) / fc1_blocks) > 48 || fc1_blocks * 16 > kMegaActPackets)
      return no("activation packets do not fit their slots");
  }
  if (mega_lds_bytes(a, D) > 150 * 1024) return no("context too long for the LDS score buffer");
  return true;
}

int launch_phi2_decode_step(hipStream_t st, const MegaArgs &a, int D, int num_cu) {
  const char *why = nullptr;
  RAI_REQUIRE(mega_eligible(a, D, num_cu, &why), RAI_ERR_UNSUPPORTED, "persistent decode step: %s", why ? why : "?");
  size_t lds = mega_lds_bytes(a, D);
  MegaArgs m = a;
  // the weight staging area (kMegaStage KB per stream wave) goes behind everything else where the CU's LDS holds both
  const size_t stage_bytes = (size_t)kMegaStream * kMegaStage * 1024;
  const char *no_stage = getenv("RAI_HIP_MEGA_NO_STAGE");   // read per call: tests run both forms in one process
  m.stage_off = 0;
  if (lds + stage_bytes <= kMegaLdsMax && !(no_stage && *no_stage && *no_stage != '0')) {
    m.stage_off = (int)lds;
    lds += stage_bytes;
  }
  static bool attr_set = false;
  if (!attr_set) {
    RAI_HIP_TRY(hipFuncSetAttribute((const void *)k_phi2_decode_step<5, 80, false>,
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMegaLdsMax));
    RAI_HIP_TRY(hipFuncSetAttribute((const void *)k_phi2_decode_step<5, 80, true>,
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMegaLdsMax));
    RAI_HIP_TRY(hipFuncSetAttribute((const void *)k_phi2_decode_step<4, 64, false>,
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMegaLdsMax));
    RAI_HIP_TRY(hipFuncSetAttribute((const void *)k_phi2_decode_step<4, 64, true>,
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMegaLdsMax));
    attr_set = true;
  }
  if (D == 80) {
    if (m.prof) hipLaunchKernelGGL((k_phi2_decode_step<5, 80, true>), dim3(num_cu), dim3(kMegaThreads), lds, st, m);
    else hipLaunchKernelGGL((k_phi2_decode_step<5, 80, false>), dim3(num_cu), dim3(kMegaThreads), lds, st, m);
  } else {
    if (m.prof) hipLaunchKernelGGL((k_phi2_decode_step<4, 64, true>), dim3(num_cu), dim3(kMegaThreads), lds, st, m);
    else hipLaunchKernelGGL((k_phi2_decode_step<4, 64, false>), dim3(num_cu), dim3(kMegaThreads), lds, st, m);
  }
  return launch_check("phi2_decode_step");
}

}  // namespace rai
