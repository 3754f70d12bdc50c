// A chain of small-M Linears in one persistent launch (one block of eight waves per CU).
//
// Between two attention calls a batched decode step of a sequential-block decoder (qwen2.rs:253-266, gemma.rs:286-299)
// is four Linears on 9..32 rows: o_proj (+ residual), gate|up with the gated-MLP epilogue behind an RMSNorm, down
// (+ residual), and the next layer's q|k|v behind its RMSNorm.  Each is a pure weight stream, and as a launch of its own
// each starts cold: 2048 waves load their activations, normalise them and only then ask for their first weight tiles,
// while the memory pipe sits idle (a third of such a launch).  Here the four run as phases of one launch:
//   - the weight stream of a phase is the one of k_linear_bf16_mfma_stream (gemm_mfma.hip): weights in fragment order
//     as the MFMA A operand straight from global memory, activations as B fragments in registers, K split over the
//     eight waves of a block, partial accumulators summed through LDS, the Linear epilogue on four columns per thread;
//   - a block asks for the first weight tiles of the NEXT phase before it waits at the barrier that ends the current
//     one (weights do not depend on anything computed here), so that memory keeps streaming through the barrier, the
//     activation loads and the norm;
//   - what one phase writes and the next one reads crosses blocks, i.e. XCDs whose L2s are not coherent with each other:
//     those buffers are written with device-scope stores (write-through) and read with device-scope loads, no fences;
//   - the barrier has no read-modify-write traffic (256 blocks bumping one counter serialise at its memory channel:
//     14 us per barrier): every block stores the barrier's number to a flag of its own and polls all flags, one per
//     thread; numbers only grow, so nothing is reset.  A wait is bounded: one that expires flags the device's fault
//     word and every later wait falls through, so all waves exit and the host reports the step as failed instead of
//     hanging.
// The K split of the down projection (K = intermediate size: 8 spans of 2048) leaves f32 partial products that a
// fifth, tiny phase sums in split order together with the residual.
#include "decode_chain.h"
#include "gemm.h"

namespace rai {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int kChainThreads = 512, kChainWaves = 8, kChainMT = 2, kChainRing = 3;

// 16 / 8 / 4 / 2 bytes read or written past the L2 of this XCD when `fresh`, as ordinary accesses otherwise
__device__ __forceinline__ bf16x8 chain_load16(const uint16_t *p, bool fresh) {
  if (!fresh) return *reinterpret_cast<const bf16x8 *>(p);
  unsigned long long u[2];
  u[0] = __hip_atomic_load(reinterpret_cast<const unsigned long long *>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  u[1] = __hip_atomic_load(reinterpret_cast<const unsigned long long *>(p) + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  bf16x8 v;
  __builtin_memcpy(&v, u, 16);
  return v;
}
__device__ __forceinline__ unsigned long long chain_load8(const uint16_t *p, bool fresh) {   // four bf16, 8-byte aligned
  const unsigned long long *q = reinterpret_cast<const unsigned long long *>(p);
  return fresh ? __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : *q;
}
__device__ __forceinline__ void chain_store8(void *p, uint32_t lo, uint32_t hi) {
  __hip_atomic_store(reinterpret_cast<unsigned long long *>(p), (unsigned long long)lo | ((unsigned long long)hi << 32),
                     __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void chain_store4(void *p, uint32_t v) {
  __hip_atomic_store(reinterpret_cast<uint32_t *>(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void chain_store_f32x4(float *p, const f32x4 &v) {
  chain_store8(p, __float_as_uint(v.x), __float_as_uint(v.y));
  chain_store8(p + 2, __float_as_uint(v.z), __float_as_uint(v.w));
}
__device__ __forceinline__ f32x4 chain_load_f32x4(const float *p) {
  const unsigned long long a = __hip_atomic_load(reinterpret_cast<const unsigned long long *>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const unsigned long long b = __hip_atomic_load(reinterpret_cast<const unsigned long long *>(p) + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return f32x4{__uint_as_float((uint32_t)a), __uint_as_float((uint32_t)(a >> 32)), __uint_as_float((uint32_t)b),
               __uint_as_float((uint32_t)(b >> 32))};
}

// How a phase is laid over the grid: `bx` of `nbx` blocks walk the 16-row weight tiles in groups of G, `split` picks
// the K span; blocks beyond nbx * splits sit the phase out.
struct ChainPlace {
  int tiles, nbx, bx, split;
  bool active;
};
__device__ __forceinline__ ChainPlace chain_place(const ChainPhase &p) {
  ChainPlace c;
  c.tiles = (p.N + 15) / 16;
  const int groups = (c.tiles + p.G - 1) / p.G;
  int nbx = (int)gridDim.x / p.splits;
  if (nbx < 1) nbx = 1;
  if (nbx > groups) nbx = groups;
  c.nbx = nbx;
  c.bx = (int)blockIdx.x % nbx;
  c.split = (int)blockIdx.x / nbx;
  c.active = c.split < p.splits;
  return c;
}

// Tile at position pos counted from the start of the group that begins at tile g0 (positions past the group's end
// run into the block's next group)
template <int G> __device__ __forceinline__ int chain_tile_at(int g0, int pos, int stride) { return g0 + (pos / G) * stride + pos % G; }

template <int KS>
__device__ __forceinline__ void chain_load_tile(bf16x8 (&wt)[8], const ChainPhase &p, const ChainPlace &c, int tile, int k0, int lane) {
  tile = tile < c.tiles ? tile : c.tiles - 1;
  const int ksteps = p.K / 32;
  const bf16x8 *f = reinterpret_cast<const bf16x8 *>(p.Wfrag) + lane + (int64_t)tile * ksteps * 64;
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const int k = k0 + ks * 32 < p.K ? k0 + ks * 32 : 0;   // steps beyond K read step 0 (their activations are zero)
    wt[ks] = __builtin_nontemporal_load(f + (k >> 5) * 64);
  }
  // keep the tile's loads together and ahead of what follows: left alone the scheduler sinks each load to its use
  __builtin_amdgcn_sched_barrier(0);
}

// The first tiles of a phase, requested before the barrier in front of it.
template <int KS, int G>
__device__ __forceinline__ void chain_prefetch(bf16x8 (&w)[kChainRing][8], const ChainPhase &p, int wave, int lane) {
  const ChainPlace c = chain_place(p);
  if (!c.active) return;
  const int k0 = (c.split * kChainWaves + wave) * KS * 32;
  const int g0 = c.bx * G, stride = c.nbx * G;
#pragma unroll
  for (int pos = 0; pos + 1 < kChainRing; ++pos) chain_load_tile<KS>(w[pos], p, c, chain_tile_at<G>(g0, pos, stride), k0, lane);
}

template <int KS, int G>
__device__ __forceinline__ void chain_linear(bf16x8 (&w)[kChainRing][8], const ChainPhase &p, f32x4 *red, int tid, int wave, int lane) {
  constexpr int MT = kChainMT, NW = kChainWaves, RING = kChainRing;
  constexpr int PCH = 4 * G + 1;   // row pitch of the parked accumulators, in f32x4
  const ChainPlace c = chain_place(p);
  if (!c.active) return;
  const int lrow = lane & 15, lq = lane >> 4;
  const int k0 = (c.split * NW + wave) * KS * 32;
  const bool afresh = p.a_fresh != 0, rfresh = p.res_fresh != 0;

  // activation fragments of this wave's K slice (zero beyond M and K)
  bf16x8 xf[MT][KS];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int m = mt * 16 + lrow, k = k0 + ks * 32;
      bf16x8 z = {};
      if (m < p.M && k < p.K) z = chain_load16((const uint16_t *)p.A + (int64_t)m * p.lda + k + lq * 8, afresh);
      xf[mt][ks] = z;
    }
  if (p.ln_kind > 0) {   // RMSNorm of the rows (K whole in this block): x * w / rms or x * (1 + w) / rms, rounded to bf16
    float *rs = reinterpret_cast<float *>(red);   // [8 waves][MT * 16 rows]; the accumulator area is not in use yet
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      float ss = 0.f;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int j = 0; j < 8; ++j) { const float v = (float)xf[mt][ks][j]; ss = fmaf(v, v, ss); }
      ss += __shfl_xor(ss, 16, 64);
      ss += __shfl_xor(ss, 32, 64);
      if (lq == 0) rs[wave * (MT * 16) + mt * 16 + lrow] = ss;
    }
    __syncthreads();
    const uint16_t *lw = (const uint16_t *)p.ln_w;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      float tot = 0.f;
#pragma unroll
      for (int wv = 0; wv < NW; ++wv) tot += rs[wv * (MT * 16) + mt * 16 + lrow];
      const float scale = 1.0f / sqrtf(tot / (float)p.K + p.ln_eps);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const int k = k0 + ks * 32;
        if (k < p.K) {
          const bf16x8 wv = *reinterpret_cast<const bf16x8 *>(lw + k + lq * 8);
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const float wf = (float)wv[j];
            xf[mt][ks][j] = (__bf16)((float)xf[mt][ks][j] * scale * (p.ln_kind == 2 ? 1.0f + wf : wf));
          }
        }
      }
    }
    __syncthreads();   // the statistics have been read before the area is reused
  }

  const int stride = c.nbx * G;
  const uint16_t *bias = (const uint16_t *)p.bias;
  const uint16_t *res = (const uint16_t *)p.residual;
  auto group = [&](auto rot, const int g0) {
    constexpr int R = decltype(rot)::value;
    f32x4 acc[G][MT];
#pragma unroll
    for (int j = 0; j < G; ++j)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[j][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < G; ++j) {
      chain_load_tile<KS>(w[(R + j + RING - 1) % RING], p, c, chain_tile_at<G>(g0, j + RING - 1, stride), k0, lane);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[j][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[(R + j) % RING][ks], xf[mt][ks], acc[j][mt], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    // sum the eight K slices through LDS ([row m][G tiles x 4 column quads], odd pitch), four columns per thread
    __syncthreads();   // the previous group's sums have been read
#pragma unroll
    for (int j = 0; j < G; ++j)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) red[(wave * MT * 16 + mt * 16 + lrow) * PCH + j * 4 + lq] = acc[j][mt];
    __syncthreads();
    for (int v = tid; v < MT * G * 64; v += kChainThreads) {
      const int m = v / (G * 4), cc = v - m * (G * 4);
      const int tile = g0 + (cc >> 2);
      const int n = tile * 16 + 4 * (cc & 3);
      if (tile >= c.tiles || n >= p.N || m >= p.M) continue;
      f32x4 s4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int wv = 0; wv < NW; ++wv) {
        const f32x4 t = red[(wv * MT * 16 + m) * PCH + cc];
        s4.x += t.x; s4.y += t.y; s4.z += t.z; s4.w += t.w;
      }
      const float x[4] = {s4.x, s4.y, s4.z, s4.w};
      if (p.partial) {   // N is a multiple of 4 (checked on the host)
        chain_store_f32x4(p.partial + ((int64_t)c.split * p.M + m) * p.N + n, s4);
        continue;
      }
      if (p.glu) {   // columns (n, n+1) and (n+2, n+3) are (gate, up) pairs; N is a multiple of 8
        uint16_t o[2];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          const float gt = x[2 * e] + (bias ? bf16_bits_to_f32(bias[n + 2 * e]) : 0.f);
          const float up = x[2 * e + 1] + (bias ? bf16_bits_to_f32(bias[n + 2 * e + 1]) : 0.f);
          o[e] = f32_to_bf16_bits(glu_bf16(p.act, gt, up));
        }
        chain_store4((uint16_t *)p.out + (int64_t)m * p.ldo + (n >> 1), (uint32_t)o[0] | ((uint32_t)o[1] << 16));
        continue;
      }
      uint16_t o[4];   // N is a multiple of 4 (checked on the host): the four columns exist
      const unsigned long long r4 = res ? chain_load8(res + (int64_t)m * p.ldr + n, rfresh) : 0ull;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float y = x[e] + (bias ? bf16_bits_to_f32(bias[n + e]) : 0.f);
        if (p.act >= 0) y = act_eval(p.act, y);
        if (res) y += bf16_bits_to_f32((uint16_t)(r4 >> (16 * e)));
        o[e] = f32_to_bf16_bits(y);
      }
      chain_store8((uint16_t *)p.out + (int64_t)m * p.ldo + n, (uint32_t)o[0] | ((uint32_t)o[1] << 16),
                   (uint32_t)o[2] | ((uint32_t)o[3] << 16));
    }
  };
  int g0 = c.bx * G;
  for (;;) {
    group(std::integral_constant<int, 0>{}, g0);
    if ((g0 += stride) >= c.tiles) break;
    group(std::integral_constant<int, G % RING>{}, g0);
    if ((g0 += stride) >= c.tiles) break;
    group(std::integral_constant<int, (2 * G) % RING>{}, g0);
    if ((g0 += stride) >= c.tiles) break;
  }
  __syncthreads();   // the last group's sums have been read: the next phase may use the LDS area
}

// out = residual + sum of the `splits` partial products, in split order; four columns per thread over the whole grid
__device__ __forceinline__ void chain_sum(const ChainPhase &p, int tid) {
  const int64_t quads = (int64_t)p.M * p.N / 4, total = (int64_t)p.M * p.N;
  const uint16_t *res = (const uint16_t *)p.residual;
  const uint16_t *bias = (const uint16_t *)p.bias;
  for (int64_t q = (int64_t)blockIdx.x * kChainThreads + tid; q < quads; q += (int64_t)gridDim.x * kChainThreads) {
    const int64_t e0 = q * 4;
    const int m = (int)(e0 / p.N), n = (int)(e0 - (int64_t)m * p.N);
    f32x4 s = chain_load_f32x4(p.partial + e0);
    for (int sp = 1; sp < p.splits; ++sp) {
      const f32x4 t = chain_load_f32x4(p.partial + (int64_t)sp * total + e0);
      s.x += t.x; s.y += t.y; s.z += t.z; s.w += t.w;
    }
    const float x[4] = {s.x, s.y, s.z, s.w};
    uint16_t o[4];
    const unsigned long long r4 = res ? chain_load8(res + (int64_t)m * p.ldr + n, p.res_fresh != 0) : 0ull;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float y = x[e] + (bias ? bf16_bits_to_f32(bias[n + e]) : 0.f);
      if (p.act >= 0) y = act_eval(p.act, y);
      if (res) y += bf16_bits_to_f32((uint16_t)(r4 >> (16 * e)));
      o[e] = f32_to_bf16_bits(y);
    }
    chain_store8((uint16_t *)p.out + (int64_t)m * p.ldo + n, (uint32_t)o[0] | ((uint32_t)o[1] << 16),
                 (uint32_t)o[2] | ((uint32_t)o[3] << 16));
  }
}

#define RAI_CHAIN_DISPATCH(p, CALL)                          \
  do {                                                       \
    if ((p).KS == 8) {                                       \
      if ((p).G == 4) { CALL(8, 4); } else { CALL(8, 1); }   \
    } else {                                                 \
      if ((p).G == 4) { CALL(6, 4); } else { CALL(6, 1); }   \
    }                                                        \
  } while (0)

__global__ void __launch_bounds__(kChainThreads) k_decode_chain(ChainArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char chain_lds[];
  __shared__ int s_fault;
  f32x4 *red = reinterpret_cast<f32x4 *>(chain_lds);
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  if (tid == 0) s_fault = 0;
  const unsigned long long epoch_base = ((unsigned long long)*a.epoch << 12) + (unsigned long long)a.launch * 8ull;
  bf16x8 w[kChainRing][8];
#pragma unroll
  for (int r = 0; r < kChainRing; ++r)
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) w[r][ks] = bf16x8{};
  if (a.ph[0].kind == RAI_CHAIN_LINEAR) {
#define RAI_CHAIN_PREFETCH(KS, G) chain_prefetch<KS, G>(w, a.ph[0], wave, lane)
    RAI_CHAIN_DISPATCH(a.ph[0], RAI_CHAIN_PREFETCH);
  }
  __syncthreads();
  for (int i = 0; i < a.n; ++i) {
    const ChainPhase &p = a.ph[i];
    if (p.kind == RAI_CHAIN_LINEAR) {
#define RAI_CHAIN_RUN(KS, G) chain_linear<KS, G>(w, p, red, tid, wave, lane)
      RAI_CHAIN_DISPATCH(p, RAI_CHAIN_RUN);
    } else {
      chain_sum(p, tid);
    }
    if (i + 1 == a.n) break;
    // ---- the phase's stores have left this wave; the next phase's first weight tiles are asked for; then the barrier
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (a.ph[i + 1].kind == RAI_CHAIN_LINEAR) {
#define RAI_CHAIN_PREFETCH_NEXT(KS, G) chain_prefetch<KS, G>(w, a.ph[i + 1], wave, lane)
      RAI_CHAIN_DISPATCH(a.ph[i + 1], RAI_CHAIN_PREFETCH_NEXT);
    }
    __syncthreads();
    if (!s_fault) {
      const unsigned long long number = epoch_base + (unsigned long long)(i + 1);
      if (tid == 0) __hip_atomic_store(a.flags + blockIdx.x, number, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      bool through = false;
      for (int spin = 0; spin < a.spin_limit && !through; ++spin) {
        const bool mine = tid >= (int)gridDim.x ||
                          __hip_atomic_load(a.flags + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= number;
        through = __syncthreads_and(mine) != 0;
      }
      if (!through && tid == 0) {
        s_fault = 1;
        __hip_atomic_store(a.fault, (int)RAI_FAULT_CHAIN, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      }
      __syncthreads();
    }
  }
}
#undef RAI_CHAIN_PREFETCH
#undef RAI_CHAIN_RUN
#undef RAI_CHAIN_PREFETCH_NEXT
#undef RAI_CHAIN_DISPATCH

bool decode_chain_serves(int M, int N, int K, bool k_split) {
  if (M < 1 || M > 16 * kChainMT || N % 8 != 0 || K % 32 != 0) return false;
  if (k_split) return K > 2048;                       // spans of 8 waves x 8 steps x 32 columns
  return K == 2048 || K == 1536;                      // one span: KS = 8 or 6 steps per wave
}

int launch_decode_chain(hipStream_t st, const ChainArgs &a, int dev) {
  RAI_REQUIRE(a.n >= 1 && a.n <= kChainMaxPhases && a.flags && a.epoch && a.fault && a.spin_limit > 0 && a.launch >= 0 && a.launch < 512,
              RAI_ERR_BAD_ARG, "decode chain: bad arguments");
  const int grid = device_cu_count(dev);
  RAI_REQUIRE(grid >= 64 && grid <= kChainThreads, RAI_ERR_UNSUPPORTED, "decode chain: device %d reports %d CUs", dev, grid);
  int max_g = 1;
  for (int i = 0; i < a.n; ++i) {
    const ChainPhase &p = a.ph[i];
    RAI_REQUIRE(p.M >= 1 && p.M <= 16 * kChainMT && p.N % 4 == 0 && p.out && p.ldo % 4 == 0 && ((uintptr_t)p.out & 7) == 0,
                RAI_ERR_BAD_SHAPE, "decode chain: phase %d output not served", i);
    if (p.kind == RAI_CHAIN_SUM) {
      RAI_REQUIRE(p.partial && p.splits >= 1 && ((uintptr_t)p.partial & 15) == 0, RAI_ERR_BAD_ARG, "decode chain: phase %d has no partial sums", i);
      continue;
    }
    RAI_REQUIRE(p.kind == RAI_CHAIN_LINEAR && p.A && p.Wfrag && (p.KS == 6 || p.KS == 8) && (p.G == 1 || p.G == 4) && p.splits >= 1 &&
                    p.splits <= grid && p.K % 32 == 0 && p.lda % 8 == 0 && ((uintptr_t)p.A & 15) == 0 && ((uintptr_t)p.Wfrag & 15) == 0,
                RAI_ERR_BAD_ARG, "decode chain: phase %d operands not served", i);
    RAI_REQUIRE((int64_t)p.splits * kChainWaves * p.KS * 32 >= p.K, RAI_ERR_BAD_SHAPE, "decode chain: phase %d: %d spans of %d do not cover K = %d",
                i, p.splits, kChainWaves * p.KS * 32, p.K);
    RAI_REQUIRE((p.splits == 1) == (p.partial == nullptr), RAI_ERR_BAD_ARG, "decode chain: phase %d: a K split needs partial sums and only it", i);
    RAI_REQUIRE(p.ln_kind <= 0 || (p.splits == 1 && p.ln_w), RAI_ERR_BAD_ARG, "decode chain: phase %d: the norm needs K whole", i);
    RAI_REQUIRE(!p.glu || (p.N % 8 == 0 && !p.residual && p.act >= 0 && p.ldo % 2 == 0), RAI_ERR_BAD_ARG, "decode chain: phase %d: bad gated-MLP arguments", i);
    if (p.G > max_g) max_g = p.G;
  }
  const size_t lds = (size_t)kChainWaves * kChainMT * 16 * (4 * max_g + 1) * sizeof(f32x4);
  static bool attr_set[64];
  RAI_REQUIRE(dev >= 0 && dev < 64, RAI_ERR_BAD_ARG, "device %d out of range", dev);
  if (!attr_set[dev]) {
    RAI_HIP_TRY(hipFuncSetAttribute((const void *)k_decode_chain, hipFuncAttributeMaxDynamicSharedMemorySize, 80 * 1024));
    attr_set[dev] = true;
  }
  hipLaunchKernelGGL(k_decode_chain, dim3(grid), dim3(kChainThreads), lds, st, a);
  return launch_check("decode_chain");
}

}  // namespace rai
