// bf16 x bf16 -> f32 MFMA GEMM for the Linear layout (out = A[M,K] . W[N,K]^T),
// gfx950 v_mfma_f32_32x32x16_bf16.
//
//   - block tile BM x BN, 4 waves in a 2x2 grid, each wave (BM/2) x (BN/2) made of
//     32x32 MFMA tiles; K step BK.
//   - global -> registers -> LDS with a two-deep LDS buffer: the loads of tile
//     k+1 are in flight while tile k is multiplied; one barrier per K step.
//     Rows are clamped instead of predicated, so the main loop has no branches.
//   - LDS rows are padded by 16 bytes: the 16-byte fragment reads of 16 lanes hit
//     64 distinct banks.
//   - blockIdx -> tile mapping is XCD-aware: hardware hands consecutive blocks to
//     the 8 XCDs round-robin, so each XCD is given a contiguous run of tiles and
//     the tiles that share a weight panel share one L2.
//   - epilogue through LDS: every wave stages 32 x (BN/2) accumulators at a time
//     and writes 16-byte rows with bias / activation / residual applied (or raw
//     f32 partial sums when K is split over several blocks).
#include "gemm.h"

namespace rai {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int kXcds = 8;

__device__ __forceinline__ int xcd_remap(int bid, int total) {
  // blocks bid, bid+8, bid+16, ... run on the same XCD; give them consecutive tiles
  const int per = (total + kXcds - 1) / kXcds;
  return (bid % kXcds) * per + bid / kXcds;
}

template <int BM, int BN, int BK>
__global__ void __launch_bounds__(256) k_gemm_bf16_mfma(LinearArgs a, int splits, int k_per_split, float *partial) {
  constexpr int PITCH = BK + 8;
  constexpr int WM = BM / 2, WN = BN / 2;
  constexpr int MT = WM / 32, NT = WN / 32;
  constexpr int CPR = BK / 8;               // 16-byte chunks per tile row
  constexpr int A_CH = BM * CPR / 256;      // chunks per thread
  constexpr int B_CH = BN * CPR / 256;
  constexpr int EP = WN + 4;                // epilogue staging pitch (floats)
  static_assert(A_CH >= 1 && B_CH >= 1, "tile too small for 256 threads");
  extern __shared__ __attribute__((aligned(16))) uint16_t lds[];
  uint16_t *As = lds;                       // [2][BM][PITCH]
  uint16_t *Bs = lds + 2 * BM * PITCH;      // [2][BN][PITCH]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int tiles_m = (a.M + BM - 1) / BM, tiles_n = (a.N + BN - 1) / BN;
  const int total = tiles_m * tiles_n;
  const int tile = xcd_remap(blockIdx.x, total);
  if (tile >= total) return;
  const int tile_n = tile / tiles_m, tile_m = tile % tiles_m;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int split = blockIdx.y;
  const int k_begin = split * k_per_split;
  const int k_end = k_begin + k_per_split < a.K ? k_begin + k_per_split : a.K;
  const int KT = (k_end - k_begin) / BK;

  // per-thread source pointers (rows clamped into range; results of clamped rows are never stored)
  const uint16_t *ga[A_CH], *gb[B_CH];
  int sa[A_CH], sb[B_CH];
#pragma unroll
  for (int i = 0; i < A_CH; ++i) {
    const int c = tid + i * 256, row = c / CPR, kc = (c % CPR) * 8;
    int m = m0 + row;
    m = m < a.M ? m : a.M - 1;
    ga[i] = (const uint16_t *)a.A + (int64_t)m * a.lda + k_begin + kc;
    sa[i] = row * PITCH + kc;
  }
#pragma unroll
  for (int i = 0; i < B_CH; ++i) {
    const int c = tid + i * 256, row = c / CPR, kc = (c % CPR) * 8;
    int n = n0 + row;
    n = n < a.N ? n : a.N - 1;
    gb[i] = (const uint16_t *)a.W + (int64_t)n * a.ldw + k_begin + kc;
    sb[i] = row * PITCH + kc;
  }

  f32x16 acc[MT][NT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  u32x4 ra[A_CH], rb[B_CH];
#pragma unroll
  for (int i = 0; i < A_CH; ++i) ra[i] = *reinterpret_cast<const u32x4 *>(ga[i]);
#pragma unroll
  for (int i = 0; i < B_CH; ++i) rb[i] = *reinterpret_cast<const u32x4 *>(gb[i]);
#pragma unroll
  for (int i = 0; i < A_CH; ++i) *reinterpret_cast<u32x4 *>(As + sa[i]) = ra[i];
#pragma unroll
  for (int i = 0; i < B_CH; ++i) *reinterpret_cast<u32x4 *>(Bs + sb[i]) = rb[i];
  __syncthreads();

  const int frag = (lane & 31) * PITCH + (lane >> 5) * 8;
  for (int kt = 0; kt < KT; ++kt) {
    const int buf = kt & 1;
    const bool more = kt + 1 < KT;
    if (more) {
#pragma unroll
      for (int i = 0; i < A_CH; ++i) ra[i] = *reinterpret_cast<const u32x4 *>(ga[i] + (kt + 1) * BK);
#pragma unroll
      for (int i = 0; i < B_CH; ++i) rb[i] = *reinterpret_cast<const u32x4 *>(gb[i] + (kt + 1) * BK);
    }
    const uint16_t *as = As + buf * BM * PITCH + wm * WM * PITCH + frag;
    const uint16_t *bs = Bs + buf * BN * PITCH + wn * WN * PITCH + frag;
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      bf16x8 fa[MT], fb[NT];
#pragma unroll
      for (int i = 0; i < MT; ++i) fa[i] = *reinterpret_cast<const bf16x8 *>(as + i * 32 * PITCH + ks * 16);
#pragma unroll
      for (int j = 0; j < NT; ++j) fb[j] = *reinterpret_cast<const bf16x8 *>(bs + j * 32 * PITCH + ks * 16);
#pragma unroll
      for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
    if (more) {
      uint16_t *ad = As + (buf ^ 1) * BM * PITCH, *bd = Bs + (buf ^ 1) * BN * PITCH;
#pragma unroll
      for (int i = 0; i < A_CH; ++i) *reinterpret_cast<u32x4 *>(ad + sa[i]) = ra[i];
#pragma unroll
      for (int i = 0; i < B_CH; ++i) *reinterpret_cast<u32x4 *>(bd + sb[i]) = rb[i];
    }
    __syncthreads();
  }

  // ---- epilogue: stage 32 x WN accumulators per wave in LDS, write 8 columns per lane
  float *stage = reinterpret_cast<float *>(lds) + wave * 32 * EP;
  static_assert(4 * 32 * EP * 4 <= 2 * (BM + BN) * PITCH * 2, "epilogue staging does not fit the tile buffers");
  constexpr int CG = WN / 8;                 // 8-column groups per staged row
  constexpr int ITEMS = 32 * CG / 64;        // per lane
  const uint16_t *bias = (const uint16_t *)a.bias;
  const uint16_t *bias2 = (const uint16_t *)a.bias2;
  const uint16_t *res = (const uint16_t *)a.residual;
  const bool vec_out = (a.ld1 % 8 == 0) && (a.n_split % 8 == 0) && (a.n_split == a.N || a.ld2 % 8 == 0) &&
                       ((uintptr_t)a.out1 % 16 == 0) && (a.n_split == a.N || (uintptr_t)a.out2 % 16 == 0) &&
                       (!res || (a.ldr % 8 == 0 && (uintptr_t)res % 16 == 0)) && a.N % 8 == 0;
#pragma unroll
  for (int i = 0; i < MT; ++i) {
    // accumulator register r of lane l is C[8*(r/4) + 4*(l/32) + r%4][l%32]
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        stage[(8 * (r >> 2) + 4 * (lane >> 5) + (r & 3)) * EP + j * 32 + (lane & 31)] = acc[i][j][r];
    // LDS operations of one wave complete in order; no block barrier is needed for a wave-private region
#pragma unroll 1
    for (int it = 0; it < ITEMS; ++it) {
      const int item = lane + it * 64;
      const int row = item / CG, cg = item % CG;
      const int m = m0 + wm * WM + i * 32 + row;
      const int n = n0 + wn * WN + cg * 8;
      if (m >= a.M || n >= a.N) continue;
      const f32x4 v0 = *reinterpret_cast<const f32x4 *>(stage + row * EP + cg * 8);
      const f32x4 v1 = *reinterpret_cast<const f32x4 *>(stage + row * EP + cg * 8 + 4);
      float v[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
      if (partial) {
        float *p = partial + ((int64_t)split * a.M + m) * a.N + n;
        if (a.N % 4 == 0) {
          *reinterpret_cast<f32x4 *>(p) = v0;
          if (n + 4 < a.N) *reinterpret_cast<f32x4 *>(p + 4) = v1;
        } else {
          for (int e = 0; e < 8 && n + e < a.N; ++e) p[e] = v[e];
        }
        continue;
      }
      if (a.glu) {  // columns n..n+7 are four (gate, up) pairs -> four outputs at column n/2
        uint16_t *dst = (uint16_t *)a.out1 + (int64_t)m * a.ld1 + (n >> 1);
        float gl[4];
        for (int e = 0; e < 8; e += 2) {
          const float g = v[e] + (bias ? bf16_bits_to_f32(bias[n + e]) : 0.f);
          const float u = v[e + 1] + (bias ? bf16_bits_to_f32(bias[n + e + 1]) : 0.f);
          gl[e >> 1] = glu_bf16(a.act, g, u);
        }
        if (n + 8 <= a.N && a.ld1 % 4 == 0 && (uintptr_t)a.out1 % 8 == 0) {
          typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
          u32x2 o = {pack_bf16x2(gl[0], gl[1]), pack_bf16x2(gl[2], gl[3])};
          *reinterpret_cast<u32x2 *>(dst) = o;
        } else {
          for (int e = 0; e < 4 && n + 2 * e + 1 < a.N; ++e) dst[e] = f32_to_bf16_bits(gl[e]);
        }
        continue;
      }
      const int lim = a.N - n < 8 ? a.N - n : 8;
      for (int e = 0; e < lim; ++e) {
        const int nn = n + e;
        float x = v[e] + (bias ? bf16_bits_to_f32(bias[nn]) : 0.f) + (bias2 ? bf16_bits_to_f32(bias2[nn]) : 0.f);
        if (a.act >= 0 && nn >= a.act_from) x = act_eval(a.act, x);
        if (res) x += bf16_bits_to_f32(res[(int64_t)m * a.ldr + nn]);
        v[e] = x;
      }
      if (vec_out) {
        u32x4 o;
        o.x = (uint32_t)f32_to_bf16_bits(v[0]) | ((uint32_t)f32_to_bf16_bits(v[1]) << 16);
        o.y = (uint32_t)f32_to_bf16_bits(v[2]) | ((uint32_t)f32_to_bf16_bits(v[3]) << 16);
        o.z = (uint32_t)f32_to_bf16_bits(v[4]) | ((uint32_t)f32_to_bf16_bits(v[5]) << 16);
        o.w = (uint32_t)f32_to_bf16_bits(v[6]) | ((uint32_t)f32_to_bf16_bits(v[7]) << 16);
        uint16_t *dst = n < a.n_split ? (uint16_t *)a.out1 + (int64_t)m * a.ld1 + n
                                      : (uint16_t *)a.out2 + (int64_t)m * a.ld2 + (n - a.n_split);
        *reinterpret_cast<u32x4 *>(dst) = o;
      } else {
        for (int e = 0; e < lim; ++e) {
          const int nn = n + e;
          if (nn < a.n_split) ((uint16_t *)a.out1)[(int64_t)m * a.ld1 + nn] = f32_to_bf16_bits(v[e]);
          else ((uint16_t *)a.out2)[(int64_t)m * a.ld2 + (nn - a.n_split)] = f32_to_bf16_bits(v[e]);
        }
      }
    }
  }
}

// Sums the per-split partial products and applies the Linear epilogue.
__global__ void __launch_bounds__(256) k_splitk_epilogue(LinearArgs a, int splits, const float *partial) {
  const int64_t total = (int64_t)a.M * a.N;
  const uint16_t *bias = (const uint16_t *)a.bias;
  const uint16_t *bias2 = (const uint16_t *)a.bias2;
  const uint16_t *res = (const uint16_t *)a.residual;
  for (int64_t e = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; e < total; e += (int64_t)gridDim.x * blockDim.x) {
    const int m = (int)(e / a.N), n = (int)(e % a.N);
    if (a.glu) {
      if (n & 1) continue;
      float g = 0.f, u = 0.f;
      for (int s = 0; s < splits; ++s) { g += partial[(int64_t)s * total + e]; u += partial[(int64_t)s * total + e + 1]; }
      g += bias ? bf16_bits_to_f32(bias[n]) : 0.f;
      u += bias ? bf16_bits_to_f32(bias[n + 1]) : 0.f;
      ((uint16_t *)a.out1)[(int64_t)m * a.ld1 + (n >> 1)] = f32_to_bf16_bits(glu_bf16(a.act, g, u));
      continue;
    }
    float x = 0.f;
    for (int s = 0; s < splits; ++s) x += partial[(int64_t)s * total + e];
    x += (bias ? bf16_bits_to_f32(bias[n]) : 0.f) + (bias2 ? bf16_bits_to_f32(bias2[n]) : 0.f);
    if (a.act >= 0 && n >= a.act_from) x = act_eval(a.act, x);
    if (res) x += bf16_bits_to_f32(res[(int64_t)m * a.ldr + n]);
    if (n < a.n_split) ((uint16_t *)a.out1)[(int64_t)m * a.ld1 + n] = f32_to_bf16_bits(x);
    else ((uint16_t *)a.out2)[(int64_t)m * a.ld2 + (n - a.n_split)] = f32_to_bf16_bits(x);
  }
}

template <int BM, int BN, int BK> static int launch_cfg(hipStream_t st, const LinearArgs &a, int splits) {
  constexpr size_t lds = (size_t)2 * (BM + BN) * (BK + 8) * sizeof(uint16_t);
  static bool attr_set = false;
  if (lds > 64 * 1024 && !attr_set) {
    RAI_HIP_TRY(hipFuncSetAttribute((const void *)k_gemm_bf16_mfma<BM, BN, BK>,
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attr_set = true;
  }
  const int tiles = ((a.M + BM - 1) / BM) * ((a.N + BN - 1) / BN);
  const int grid_x = ((tiles + kXcds - 1) / kXcds) * kXcds;  // whole rounds over the XCDs
  int k_per_split = a.K;
  float *partial = nullptr;
  if (splits > 1) {
    const int k_tiles = a.K / BK, per = (k_tiles + splits - 1) / splits;
    splits = (k_tiles + per - 1) / per;  // every split gets at least one K tile
    k_per_split = per * BK;
    partial = (float *)a.splitk_ws;
  }
  hipLaunchKernelGGL((k_gemm_bf16_mfma<BM, BN, BK>), dim3(grid_x, splits), dim3(256), lds, st, a, splits, k_per_split,
                     partial);
  RAI_TRY(launch_check("gemm_bf16_mfma"));
  if (splits > 1) {
    int64_t total = (int64_t)a.M * a.N;
    int blocks = (int)((total + 255) / 256 < 4096 ? (total + 255) / 256 : 4096);
    hipLaunchKernelGGL(k_splitk_epilogue, dim3(blocks), dim3(256), 0, st, a, splits, (const float *)partial);
    RAI_TRY(launch_check("splitk_epilogue"));
  }
  return RAI_OK;
}

// ---- small M (9..64 rows): weight streaming through 16x16x32 MFMA -----------------------
// The activations are tiny and the weights are read exactly once, so the kernel is a
// stream over W: every wave owns 16 weight rows and reads them straight from global
// memory in MFMA fragment order (lane l: row l%16, 8 consecutive k at 8*(l/16)), U
// fragments ahead of the multiply.  The activation rows sit in LDS (16-byte padded
// pitch: the fragment reads of 16 lanes hit distinct banks) and are the B operand, so
// accumulator register r of lane l is out[m = l%16][n = 4*(l/16) + r]: four consecutive
// columns per lane.  K may be split over blockIdx.y (f32 partial sums, summed by
// k_splitk_epilogue) so that narrow outputs still fill the chip.
template <int MT, int U>
__global__ void __launch_bounds__(256) k_linear_bf16_mfma_skinny(LinearArgs a, int k_per_split, int k_chunk,
                                                                 float *partial) {
  extern __shared__ __attribute__((aligned(16))) uint16_t lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int split = blockIdx.y;
  const int kb = split * k_per_split;
  const int ke = kb + k_per_split < a.K ? kb + k_per_split : a.K;
  const int pitch = k_chunk + 8;
  const int n0 = (blockIdx.x * 4 + wave) * 16;
  int nrow = n0 + (lane & 15);
  nrow = nrow < a.N ? nrow : a.N - 1;  // clamped rows are computed and never stored
  const uint16_t *wrow = (const uint16_t *)a.W + (int64_t)nrow * a.ldw + (lane >> 4) * 8;
  const uint16_t *xfrag = lds + (lane & 15) * pitch + (lane >> 4) * 8;

  f32x4 acc[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};

  for (int kc0 = kb; kc0 < ke; kc0 += k_chunk) {
    const int clen = ke - kc0 < k_chunk ? ke - kc0 : k_chunk;  // multiple of 32
    const int cpr = clen >> 3;
    if (kc0 != kb) __syncthreads();
    for (int c = tid; c < MT * 16 * cpr; c += 256) {
      const int row = c / cpr, kc = (c - row * cpr) * 8;
      u32x4 v = {0u, 0u, 0u, 0u};
      if (row < a.M) v = *reinterpret_cast<const u32x4 *>((const uint16_t *)a.A + (int64_t)row * a.lda + kc0 + kc);
      *reinterpret_cast<u32x4 *>(lds + row * pitch + kc) = v;
    }
    const uint16_t *wp = wrow + kc0;
    bf16x8 w[U];
    const int full = clen / (32 * U);
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (full > 0) w[u] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8 *>(wp + u * 32));
    __syncthreads();
    int k = 0;
    for (int it = 0; it < full; ++it, k += 32 * U) {
      bf16x8 cur[U];
#pragma unroll
      for (int u = 0; u < U; ++u) cur[u] = w[u];
      if (it + 1 < full) {
#pragma unroll
        for (int u = 0; u < U; ++u)
          w[u] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8 *>(wp + k + 32 * U + u * 32));
      }
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int i = 0; i < MT; ++i) {
          const bf16x8 x = *reinterpret_cast<const bf16x8 *>(xfrag + i * 16 * pitch + k + u * 32);
          acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur[u], x, acc[i], 0, 0, 0);
        }
    }
    for (; k < clen; k += 32) {
      const bf16x8 wv = __builtin_nontemporal_load(reinterpret_cast<const bf16x8 *>(wp + k));
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        const bf16x8 x = *reinterpret_cast<const bf16x8 *>(xfrag + i * 16 * pitch + k);
        acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv, x, acc[i], 0, 0, 0);
      }
    }
  }

  const int n = n0 + 4 * (lane >> 4);
  if (n >= a.N) return;
  const uint16_t *bias = (const uint16_t *)a.bias;
  const uint16_t *bias2 = (const uint16_t *)a.bias2;
  const uint16_t *res = (const uint16_t *)a.residual;
#pragma unroll
  for (int i = 0; i < MT; ++i) {
    const int m = i * 16 + (lane & 15);
    if (m >= a.M) continue;
    const float v[4] = {acc[i][0], acc[i][1], acc[i][2], acc[i][3]};
    if (partial) {
      float *p = partial + ((int64_t)split * a.M + m) * a.N + n;
      if (a.N % 4 == 0) *reinterpret_cast<f32x4 *>(p) = acc[i];
      else for (int e = 0; e < 4 && n + e < a.N; ++e) p[e] = v[e];
      continue;
    }
    if (a.glu) {  // columns n..n+3 are two (gate, up) pairs
      uint16_t *dst = (uint16_t *)a.out1 + (int64_t)m * a.ld1 + (n >> 1);
      for (int e = 0; e < 4 && n + e + 1 < a.N; e += 2) {
        const float g = v[e] + (bias ? bf16_bits_to_f32(bias[n + e]) : 0.f);
        const float u = v[e + 1] + (bias ? bf16_bits_to_f32(bias[n + e + 1]) : 0.f);
        dst[e >> 1] = f32_to_bf16_bits(glu_bf16(a.act, g, u));
      }
      continue;
    }
    for (int e = 0; e < 4 && n + e < a.N; ++e) {
      const int nn = n + e;
      float x = v[e] + (bias ? bf16_bits_to_f32(bias[nn]) : 0.f) + (bias2 ? bf16_bits_to_f32(bias2[nn]) : 0.f);
      if (a.act >= 0 && nn >= a.act_from) x = act_eval(a.act, x);
      if (res) x += bf16_bits_to_f32(res[(int64_t)m * a.ldr + nn]);
      if (nn < a.n_split) ((uint16_t *)a.out1)[(int64_t)m * a.ld1 + nn] = f32_to_bf16_bits(x);
      else ((uint16_t *)a.out2)[(int64_t)m * a.ld2 + (nn - a.n_split)] = f32_to_bf16_bits(x);
    }
  }
}

template <int MT> static int launch_mfma_skinny(hipStream_t st, const LinearArgs &a) {
  constexpr int U = 8;
  constexpr int kcap = MT == 1 ? 2048 : MT == 2 ? 1024 : 512;  // LDS: MT*16 rows of (chunk + 8) bf16, about 64 KB
  const int blocks_x = ((a.N + 15) / 16 + 3) / 4;
  // Split K until there are about four blocks per CU, keeping at least 256 columns per split.
  int splits = 1;
  if (a.splitk_ws) {
    while (blocks_x * splits < 4 * kNumCU && a.K / (splits * 2) >= 256 &&
           (size_t)(splits * 2) * a.M * a.N * sizeof(float) <= a.splitk_ws_bytes)
      splits *= 2;
  }
  int kps = (a.K + splits - 1) / splits;
  kps = (kps + 127) / 128 * 128;
  splits = (a.K + kps - 1) / kps;
  const int chunk = kps < kcap ? kps : kcap;
  const size_t lds = (size_t)MT * 16 * (chunk + 8) * sizeof(uint16_t);
  static bool attr_set = false;
  if (!attr_set) {
    RAI_HIP_TRY(hipFuncSetAttribute((const void *)k_linear_bf16_mfma_skinny<MT, U>,
                                    hipFuncAttributeMaxDynamicSharedMemorySize, 80 * 1024));
    attr_set = true;
  }
  float *partial = splits > 1 ? (float *)a.splitk_ws : nullptr;
  hipLaunchKernelGGL((k_linear_bf16_mfma_skinny<MT, U>), dim3(blocks_x, splits), dim3(256), lds, st, a, kps, chunk,
                     partial);
  RAI_TRY(launch_check("linear_bf16_mfma_skinny"));
  if (splits > 1) {
    const int64_t total = (int64_t)a.M * a.N;
    const int blocks = (int)((total + 255) / 256 < 4096 ? (total + 255) / 256 : 4096);
    hipLaunchKernelGGL(k_splitk_epilogue, dim3(blocks), dim3(256), 0, st, a, splits, (const float *)partial);
    RAI_TRY(launch_check("splitk_epilogue"));
  }
  return RAI_OK;
}

// ---- small M, second form: activations in registers, K split over the waves of a block ----
// Block = 8 waves; wave w owns K columns [k0 + w*32*KS, k0 + (w+1)*32*KS) of the block's
// K span and keeps the activation fragments of that slice in registers for the whole
// launch (MT*KS fragments).  The block walks over 16-row weight tiles: every wave reads
// its slice of the tile's rows straight into MFMA A fragments (one tile ahead of the
// multiply), so the block as a whole reads one contiguous 16-row panel after another and
// nothing is staged through LDS.  After G tiles the eight partial accumulators of each
// output are summed through LDS and the Linear epilogue is applied.  A K span of
// 256*KS covers K = 2048 (M <= 32) without splitting K over blocks, so the qkv / dense
// shapes of a batched decode step need neither a partial-sum buffer nor a second kernel.
template <int MT, int KS, int G>
__global__ void __launch_bounds__(512) k_linear_bf16_mfma_stream(LinearArgs a, int tiles, float *partial) {
  constexpr int NW = 8;
  extern __shared__ __attribute__((aligned(16))) uint16_t lds[];
  f32x4 *red = reinterpret_cast<f32x4 *>(lds);        // [NW][G*MT][64]
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lrow = lane & 15, lq = lane >> 4;
  const int split = blockIdx.y;
  const int k0 = (split * NW + wave) * KS * 32;

  // activation fragments of this wave's K slice (zero beyond M and K)
  bf16x8 xf[MT][KS];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int m = mt * 16 + lrow, k = k0 + ks * 32;
      bf16x8 z = {};
      if (m < a.M && k < a.K)
        z = *reinterpret_cast<const bf16x8 *>((const uint16_t *)a.A + (int64_t)m * a.lda + k + lq * 8);
      xf[mt][ks] = z;
    }
  int koff[KS];   // K steps beyond K read column 0 (their activation fragments are zero)
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) koff[ks] = k0 + ks * 32 < a.K ? k0 + ks * 32 : 0;
  const uint16_t *wbase = (const uint16_t *)a.W + lq * 8;

  bf16x8 wa[KS], wb[KS];
  auto load_tile = [&](bf16x8 (&w)[KS], int tile) {
    tile = tile < tiles ? tile : tiles - 1;
    int n = tile * 16 + lrow;
    n = n < a.N ? n : a.N - 1;
    const uint16_t *p = wbase + (int64_t)n * a.ldw;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) w[ks] = *reinterpret_cast<const bf16x8 *>(p + koff[ks]);
    // keep the whole tile's loads together and ahead of the multiplies that follow: left alone,
    // the scheduler sinks each load to just before its use and the prefetch distance collapses
    __builtin_amdgcn_sched_barrier(0);
  };
  const int stride = gridDim.x * G;
  int g0 = blockIdx.x * G;
  load_tile(wa, g0);
  for (; g0 < tiles; g0 += stride) {
    f32x4 acc[G][MT];
#pragma unroll
    for (int j = 0; j < G; ++j)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[j][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < G; j += 2) {
      if (G > 1) load_tile(wb, g0 + j + 1);
      else load_tile(wb, g0 + stride);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[j][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[ks], xf[mt][ks], acc[j][mt], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      if (G > 1) {
        load_tile(wa, j + 2 < G ? g0 + j + 2 : g0 + stride);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            acc[j + 1 < G ? j + 1 : j][mt] =
                __builtin_amdgcn_mfma_f32_16x16x32_bf16(wb[ks], xf[mt][ks], acc[j + 1 < G ? j + 1 : j][mt], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      } else {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) wa[ks] = wb[ks];
      }
    }
    // ---- sum the eight K slices and write G tiles of 16 columns x 16*MT rows
    __syncthreads();   // the previous group's sums have been read
#pragma unroll
    for (int j = 0; j < G; ++j)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) red[(wave * G * MT + j * MT + mt) * 64 + lane] = acc[j][mt];
    __syncthreads();
    const float *redf = reinterpret_cast<const float *>(red);
    const uint16_t *bias = (const uint16_t *)a.bias;
    const uint16_t *bias2 = (const uint16_t *)a.bias2;
    const uint16_t *res = (const uint16_t *)a.residual;
    for (int v = tid; v < G * MT * 256; v += 512) {
      const int slot = v >> 8, rem = v & 255, ln = rem >> 2, r = rem & 3;
      const int j = slot / MT, mt = slot - j * MT;
      const int tile = g0 + j;
      const int n = tile * 16 + 4 * (ln >> 4) + r, m = mt * 16 + (ln & 15);
      if (tile >= tiles || n >= a.N || m >= a.M) continue;
      float x = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) x += redf[(w * G * MT + slot) * 256 + rem];
      if (partial) {
        partial[((int64_t)split * a.M + m) * a.N + n] = x;
        continue;
      }
      if (a.glu) {   // columns (n, n+1) are a (gate, up) pair
        if (r & 1) continue;
        float u = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) u += redf[(w * G * MT + slot) * 256 + rem + 1];
        x += bias ? bf16_bits_to_f32(bias[n]) : 0.f;
        u += bias ? bf16_bits_to_f32(bias[n + 1]) : 0.f;
        ((uint16_t *)a.out1)[(int64_t)m * a.ld1 + (n >> 1)] = f32_to_bf16_bits(glu_bf16(a.act, x, u));
        continue;
      }
      x += (bias ? bf16_bits_to_f32(bias[n]) : 0.f) + (bias2 ? bf16_bits_to_f32(bias2[n]) : 0.f);
      if (a.act >= 0 && n >= a.act_from) x = act_eval(a.act, x);
      if (res) x += bf16_bits_to_f32(res[(int64_t)m * a.ldr + n]);
      if (n < a.n_split) ((uint16_t *)a.out1)[(int64_t)m * a.ld1 + n] = f32_to_bf16_bits(x);
      else ((uint16_t *)a.out2)[(int64_t)m * a.ld2 + (n - a.n_split)] = f32_to_bf16_bits(x);
    }
  }
}

template <int MT, int KS, int G> static int launch_mfma_stream_cfg(hipStream_t st, const LinearArgs &a, int splits) {
  const int tiles = (a.N + 15) / 16;
  const int groups = (tiles + G - 1) / G;
  int blocks_x = kNumCU / splits;
  if (blocks_x < 1) blocks_x = 1;
  if (blocks_x > groups) blocks_x = groups;
  const size_t lds = (size_t)8 * G * MT * 64 * sizeof(f32x4);
  static bool attr_set = false;
  if (lds > 64 * 1024 && !attr_set) {
    RAI_HIP_TRY(hipFuncSetAttribute((const void *)k_linear_bf16_mfma_stream<MT, KS, G>,
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attr_set = true;
  }
  float *partial = splits > 1 ? (float *)a.splitk_ws : nullptr;
  hipLaunchKernelGGL((k_linear_bf16_mfma_stream<MT, KS, G>), dim3(blocks_x, splits), dim3(512), lds, st, a, tiles,
                     partial);
  RAI_TRY(launch_check("linear_bf16_mfma_stream"));
  if (splits > 1) {
    const int64_t total = (int64_t)a.M * a.N;
    const int blocks = (int)((total + 255) / 256 < 4096 ? (total + 255) / 256 : 4096);
    hipLaunchKernelGGL(k_splitk_epilogue, dim3(blocks), dim3(256), 0, st, a, splits, (const float *)partial);
    RAI_TRY(launch_check("splitk_epilogue"));
  }
  return RAI_OK;
}

// False when the shape needs a K split and no (or too small a) workspace was lent.
template <int MT, int KS> static bool mfma_stream_fits(const LinearArgs &a, int *splits) {
  const int span = 8 * KS * 32;
  *splits = (a.K + span - 1) / span;
  return *splits == 1 || (a.splitk_ws && (size_t)*splits * a.M * a.N * sizeof(float) <= a.splitk_ws_bytes);
}

template <int MT, int KS> static int launch_mfma_stream(hipStream_t st, const LinearArgs &a, int splits) {
  const int tiles = (a.N + 15) / 16;
  const int per_block = tiles * splits / kNumCU;   // tiles per block when every CU holds one block
  if (per_block >= 4) return launch_mfma_stream_cfg<MT, KS, 4>(st, a, splits);
  if (per_block >= 2) return launch_mfma_stream_cfg<MT, KS, 2>(st, a, splits);
  return launch_mfma_stream_cfg<MT, KS, 1>(st, a, splits);
}

int launch_linear_bf16_mfma(hipStream_t st, const LinearArgs &a) {
  RAI_REQUIRE(a.M > 0 && a.N > 0 && a.K > 0, RAI_ERR_BAD_SHAPE, "linear: empty problem %dx%dx%d", a.M, a.N, a.K);
  RAI_REQUIRE(a.A && a.W && a.out1, RAI_ERR_BAD_ARG, "linear: null operand");
  RAI_REQUIRE(a.n_split >= 0 && a.n_split <= a.N && (a.n_split == a.N || a.out2), RAI_ERR_BAD_ARG,
              "linear: bad output split");
  RAI_REQUIRE(a.ln_kind < 0, RAI_ERR_UNSUPPORTED, "linear: fused norm only on the skinny path");
  if (a.glu) RAI_REQUIRE(a.N % 8 == 0 && !a.residual && a.n_split == a.N && a.act >= 0, RAI_ERR_BAD_ARG,
                         "linear mfma: bad gated-MLP arguments");
  RAI_REQUIRE(a.K % 32 == 0, RAI_ERR_UNSUPPORTED, "linear mfma: K=%d must be a multiple of 32", a.K);
  RAI_REQUIRE(a.lda % 8 == 0 && a.ldw % 8 == 0 && (uintptr_t)a.A % 16 == 0 && (uintptr_t)a.W % 16 == 0,
              RAI_ERR_BAD_STRIDE, "linear mfma: operands must be 16-byte aligned with row strides multiple of 8");
  static const bool no_skinny = getenv("RAI_HIP_NO_MFMA_SKINNY") != nullptr;
  static const bool no_stream = getenv("RAI_HIP_NO_MFMA_STREAM") != nullptr;
  if (a.M <= 64 && !no_skinny && !no_stream) {
    int splits = 1;
    if (a.M <= 16 && mfma_stream_fits<1, 8>(a, &splits)) return launch_mfma_stream<1, 8>(st, a, splits);
    if (a.M > 16 && a.M <= 32 && mfma_stream_fits<2, 8>(a, &splits)) return launch_mfma_stream<2, 8>(st, a, splits);
    if (a.M > 32 && a.M <= 48 && mfma_stream_fits<3, 4>(a, &splits)) return launch_mfma_stream<3, 4>(st, a, splits);
    if (a.M > 48 && mfma_stream_fits<4, 4>(a, &splits)) return launch_mfma_stream<4, 4>(st, a, splits);
  }
  if (a.M <= 64 && !no_skinny) {
    const int mt = (a.M + 15) / 16;
    if (mt == 1) return launch_mfma_skinny<1>(st, a);
    if (mt == 2) return launch_mfma_skinny<2>(st, a);
    if (mt == 3) return launch_mfma_skinny<3>(st, a);
    return launch_mfma_skinny<4>(st, a);
  }
  // Split K when the tile count alone cannot fill the GPU and a workspace was provided.
  const int tiles = ((a.M + 127) / 128) * ((a.N + 127) / 128);
  int splits = 1;
  if (a.splitk_ws && tiles < kNumCU) {
    while (splits < 8 && tiles * splits * 2 <= 2 * kNumCU && a.K / (splits * 2) >= 512) splits *= 2;
    while (splits > 1 && (size_t)splits * a.M * a.N * sizeof(float) > a.splitk_ws_bytes) splits /= 2;
  }
  return launch_cfg<128, 128, 32>(st, a, splits);
}

}  // namespace rai
