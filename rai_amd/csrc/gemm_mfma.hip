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
#include <cstring>
#include <type_traits>

#include "gemm.h"

namespace rai {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int kXcds = 8;

// Tile order inside an XCD's run: bands of kGroupM tile rows swept across all tile columns, so the
// ~100 tiles that are resident on an XCD at any moment form a block of about kGroupM x 12 tiles and
// share their A and B panels through that XCD's L2 (a column-by-column order re-reads all of A from
// memory for every tile column).
constexpr int kGroupM = 8;
__device__ __forceinline__ void tile_coords(int tile, int tiles_m, int tiles_n, int *tile_m, int *tile_n) {
  const int band = tile / (kGroupM * tiles_n);
  const int first_m = band * kGroupM;
  const int height = tiles_m - first_m < kGroupM ? tiles_m - first_m : kGroupM;
  const int in_band = tile - band * kGroupM * tiles_n;
  *tile_m = first_m + in_band % height;
  *tile_n = in_band / height;
}

__device__ __forceinline__ int xcd_remap(int bid, int total) {
  // blocks bid, bid+8, bid+16, ... run on the same XCD; give them consecutive tiles
  const int per = (total + kXcds - 1) / kXcds;
  return (bid % kXcds) * per + bid / kXcds;
}

// LDS a tile kernel needs: two stages of A and B tiles, or the epilogue staging area if that is larger.
template <int BM, int BN, int PITCH, int WGN = 2, int WGM = 2> constexpr int gemm_lds_bytes() {
  constexpr int tiles = 2 * (BM + BN) * PITCH * 2, staging = WGM * WGN * 32 * (BN / WGN + 4) * 4;
  return tiles > staging ? tiles : staging;
}

// LDS of the LDS-DMA tile kernels: NS stages of 32 of K, or (NS == 2) two stages of 64.
template <int BM, int BN, int NS, int WGN, int WGM = 2> constexpr int dma_lds_bytes() {
  return gemm_lds_bytes<BM, BN, NS == 2 ? 64 : 32 * NS / 2, WGN, WGM>();
}

// Applies activation `act` to the elements of x[8] whose column n + e is >= from.  The switch on the
// (block-uniform) activation sits outside the element loop, so only one activation's code runs.
// The results are rounded to bf16 (relative step 2^-8), so tanh-GELU and SiLU are evaluated through the hardware
// exponential and reciprocal (relative error ~1e-6) instead of the library tanhf / expf and a division:
// 0.5 x (1 + tanh u) = x / (1 + exp(-2u)).  The f32 Linear keeps the library functions (act_eval).
__device__ __forceinline__ float act_eval_bf16_out(int act, float x) {
  if (act == RAI_UN_NEW_GELU) {
    const float u = 0.7978845608028654f * (x + 0.044715f * x * x * x);
    return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-2.0f * 1.4426950408889634f * u));
  }
  if (act == RAI_UN_SILU) return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * x));
  return act_eval(act, x);
}
template <int N>
__device__ __forceinline__ void act_n(int act, float (&x)[N], int n, int from) {
#define RAI_ACT_CASE(K)                                     \
  case K:                                                   \
    _Pragma("unroll") for (int e = 0; e < N; ++e)           \
      if (n + e >= from) x[e] = act_eval_bf16_out(K, x[e]); \
    break;
  switch (act) {
    RAI_ACT_CASE(RAI_UN_GELU)
    RAI_ACT_CASE(RAI_UN_NEW_GELU)
    RAI_ACT_CASE(RAI_UN_SILU)
    RAI_ACT_CASE(RAI_UN_RELU)
    RAI_ACT_CASE(RAI_UN_TANH)
    default: break;
  }
#undef RAI_ACT_CASE
}
__device__ __forceinline__ void act8(int act, float (&x)[8], int n, int from) { act_n<8>(act, x, n, from); }
__device__ __forceinline__ void unpack8(const u32x4 &p, float (&f)[8]) {
#pragma unroll
  for (int e = 0; e < 8; ++e) f[e] = bf16_bits_to_f32((uint16_t)(p[e >> 1] >> (16 * (e & 1))));
}

// Tile epilogue shared by the tile kernels: every wave stages 32 x WN accumulators at a time in
// LDS (the tile buffers are free by then) and writes 16-byte rows with bias / activation /
// residual applied, or raw f32 partial sums when K is split over several blocks.
// (WGM x WGN = waves along M and N; WGM = 2 except for the 256 x 192 tile.)
template <int BM, int BN, int LDS_BYTES, int WGN = 2, int WGM = 2>
__device__ __forceinline__ void gemm_tile_epilogue(const LinearArgs &a, f32x16 (&acc)[BM / (32 * WGM)][BN / (32 * WGN)],
                                                   uint16_t *lds, int m0, int n0, int wave, int lane, int split,
                                                   float *partial) {
  constexpr int WM = BM / WGM, WN = BN / WGN;
  constexpr int MT = WM / 32, NT = WN / 32;
  constexpr int EP = WN + 4;                // epilogue staging pitch (floats)
  const int wm = wave / WGN, wn = wave % WGN;
  // ---- epilogue: stage 32 x WN accumulators per wave in LDS, write 8 columns per lane
  float *stage = reinterpret_cast<float *>(lds) + wave * 32 * EP;
  static_assert(WGM * WGN * 32 * EP * 4 <= LDS_BYTES, "epilogue staging does not fit the tile buffers");
  constexpr int CG = WN / 8;                 // 8-column groups per staged row
  // rows per pass: a lane keeps its column group from pass to pass, so a pass covers a power-of-two number of whole
  // rows (CG = 12, the 96-column wave tile, leaves 16 of the 64 lanes idle)
  constexpr int RP = 64 / CG >= 16 ? 16 : 64 / CG >= 8 ? 8 : 64 / CG >= 4 ? 4 : 2;
  constexpr int ITEMS = 32 / RP;             // passes
  const uint16_t *bias = (const uint16_t *)a.bias;
  const uint16_t *bias2 = (const uint16_t *)a.bias2;
  const uint16_t *res = (const uint16_t *)a.residual;
  const bool vec_out = (a.ld1 % 8 == 0) && (a.n_split % 8 == 0) && (a.n_split == a.N || a.ld2 % 8 == 0) &&
                       ((uintptr_t)a.out1 % 16 == 0) && (a.n_split == a.N || (uintptr_t)a.out2 % 16 == 0) &&
                       (!res || (a.ldr % 8 == 0 && (uintptr_t)res % 16 == 0)) && a.N % 8 == 0;
  // A lane serves the same 8 columns in every pass: their bias values are fetched once, ahead of the passes, not
  // inside each of them, where the load's latency (about a microsecond under load) sat between the LDS read and the
  // store of every pass.
  static_assert(RP * CG <= 64 && 32 % RP == 0, "a pass is RP whole rows of CG column groups");
  const int n = n0 + wn * WN + (lane % CG) * 8;
  const bool whole = n + 8 <= a.N;
  float bv[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) bv[e] = 0.f;
  if (bias && !partial && n < a.N) {
    if (whole && ((uintptr_t)(bias + n) & 15) == 0) unpack8(*reinterpret_cast<const u32x4 *>(bias + n), bv);
    else {
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (n + e < a.N) bv[e] = bf16_bits_to_f32(bias[n + e]);
    }
  }
  if (bias2 && !partial && n < a.N) {
    float b2[8];
    if (whole && ((uintptr_t)(bias2 + n) & 15) == 0) {
      unpack8(*reinterpret_cast<const u32x4 *>(bias2 + n), b2);
#pragma unroll
      for (int e = 0; e < 8; ++e) bv[e] += b2[e];
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (n + e < a.N) bv[e] += bf16_bits_to_f32(bias2[n + e]);
    }
  }
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
      const int row = lane / CG + it * RP, cg = lane % CG;
      const int m = m0 + wm * WM + i * 32 + row;
      if (lane >= RP * CG || m >= a.M || n >= a.N) continue;
      const f32x4 v0 = *reinterpret_cast<const f32x4 *>(stage + row * EP + cg * 8);
      const f32x4 v1 = *reinterpret_cast<const f32x4 *>(stage + row * EP + cg * 8 + 4);
      float v[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
      if (partial) {
        float *p = partial + ((int64_t)split * a.M + m) * a.N + n;
        if (a.N % 4 == 0) {
          *reinterpret_cast<f32x4 *>(p) = v0;
          if (n + 4 < a.N) *reinterpret_cast<f32x4 *>(p + 4) = v1;
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (n + e < a.N) p[e] = v[e];
        }
        continue;
      }
      if (a.glu) {  // columns n..n+7 are four (gate, up) pairs -> four outputs at column n/2
        uint16_t *dst = (uint16_t *)a.out1 + (int64_t)m * a.ld1 + (n >> 1);
        float gr[8], ga[4];
#pragma unroll
        for (int e = 0; e < 8; ++e) gr[e] = bf16_bits_to_f32(f32_to_bf16_bits(v[e] + bv[e]));  // gate / up rounded to bf16 as the reference does
#pragma unroll
        for (int e = 0; e < 4; ++e) ga[e] = gr[2 * e];
        act_n<4>(a.act, ga, 0, 0);   // the four gates
        float gl[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) gl[e] = bf16_bits_to_f32(f32_to_bf16_bits(ga[e])) * gr[2 * e + 1];
        if (whole && a.ld1 % 4 == 0 && (uintptr_t)a.out1 % 8 == 0) {
          typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
          u32x2 o = {pack_bf16x2(gl[0], gl[1]), pack_bf16x2(gl[2], gl[3])};
          *reinterpret_cast<u32x2 *>(dst) = o;
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + 2 * e + 1 < a.N) dst[e] = f32_to_bf16_bits(gl[e]);
        }
        continue;
      }
      // compile-time element indices throughout: a loop bounded by a run-time count would index v[]
      // dynamically, which the compiler lowers to a chain of selects per access
      const int lim = a.N - n < 8 ? a.N - n : 8;
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] += bv[e];
      if (a.act >= 0) act8(a.act, v, n, a.act_from);
      if (res) {
        if (vec_out) {
          float rv[8];
          unpack8(*reinterpret_cast<const u32x4 *>(res + (int64_t)m * a.ldr + n), rv);
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] += rv[e];
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (e < lim) v[e] += bf16_bits_to_f32(res[(int64_t)m * a.ldr + n + e]);
        }
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
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          if (e < lim) {
            const int nn = n + e;
            if (nn < a.n_split) ((uint16_t *)a.out1)[(int64_t)m * a.ld1 + nn] = f32_to_bf16_bits(v[e]);
            else ((uint16_t *)a.out2)[(int64_t)m * a.ld2 + (nn - a.n_split)] = f32_to_bf16_bits(v[e]);
          }
        }
      }
    }
  }
}

template <int BM, int BN, int BK, int SH = 0>
__global__ void __launch_bounds__(256) k_gemm_bf16_mfma(LinearArgs a, int splits, int k_per_split, float *partial) {
  // SH == 0: rows padded by 16 bytes.  SH > 0: unpadded rows, the 16-byte chunk c of row r stored at
  // chunk c ^ ((r >> SH) & (BK/8 - 1)), so that both the row-wise stores and the column-wise
  // fragment reads spread over the banks.
  constexpr int PITCH = SH ? BK : BK + 8;
  constexpr int CMASK = BK / 8 - 1;
  constexpr int WM = BM / 2, WN = BN / 2;
  constexpr int MT = WM / 32, NT = WN / 32;
  constexpr int CPR = BK / 8;               // 16-byte chunks per tile row
  constexpr int A_CH = BM * CPR / 256;      // chunks per thread
  constexpr int B_CH = BN * CPR / 256;
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
  int tile_m, tile_n;
  tile_coords(tile, tiles_m, tiles_n, &tile_m, &tile_n);
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
    sa[i] = row * PITCH + (SH ? (((kc >> 3) ^ ((row >> SH) & CMASK)) << 3) : kc);
  }
#pragma unroll
  for (int i = 0; i < B_CH; ++i) {
    const int c = tid + i * 256, row = c / CPR, kc = (c % CPR) * 8;
    int n = n0 + row;
    n = n < a.N ? n : a.N - 1;
    gb[i] = (const uint16_t *)a.W + (int64_t)n * a.ldw + k_begin + kc;
    sb[i] = row * PITCH + (SH ? (((kc >> 3) ^ ((row >> SH) & CMASK)) << 3) : kc);
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

  const int frag = (lane & 31) * PITCH + (SH ? 0 : (lane >> 5) * 8);
  const int rsw = SH ? (((lane & 31) >> SH) & CMASK) : 0;
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
      for (int i = 0; i < MT; ++i)
        fa[i] = *reinterpret_cast<const bf16x8 *>(as + i * 32 * PITCH + (SH ? (((ks * 2 + (lane >> 5)) ^ rsw) << 3) : ks * 16));
#pragma unroll
      for (int j = 0; j < NT; ++j)
        fb[j] = *reinterpret_cast<const bf16x8 *>(bs + j * 32 * PITCH + (SH ? (((ks * 2 + (lane >> 5)) ^ rsw) << 3) : ks * 16));
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

  gemm_tile_epilogue<BM, BN, gemm_lds_bytes<BM, BN, PITCH>()>(a, acc, lds, m0, n0, wave, lane, split, partial);
}

// Tile kernel with direct global -> LDS loads (global_load_lds_dwordx4): no registers and no
// ds_write instructions are spent on staging, so NS LDS stages are cheap and the loads run
// NS-1 K tiles ahead of the multiplies, which is what hides HBM/L2 latency at 2-3 blocks per CU.
//   - one load instruction moves 64 lanes x 16 bytes into 1 KB of consecutive LDS, i.e. 16
//     unpadded tile rows of BK = 32 bf16; bank spreading comes from a swizzle instead of padding:
//     the 16-byte chunk c of row r lives at chunk position c ^ ((r >> SH) & 3), applied by choosing
//     which global chunk each lane fetches;
//   - every wave issues (BM + BN) / 64 loads per K tile; `s_waitcnt vmcnt(loads * (NS - 3))` then a
//     bare s_barrier make tile t+1 visible to the block (and retire stage t-1 for refilling) with one
//     barrier per K tile.  The barrier carries no fence: a fence would wait for every outstanding
//     LDS load, i.e. drain the pipeline.
// K loop of the LDS-DMA tile kernels: acc = A[m0.., k_begin..] . W[n0.., k_begin..]^T over KT tiles of 32, with the
// software pipeline described above.  Ends with every load landed and the block synchronised, so the caller may reuse
// the LDS stages.
template <int BM, int BN, int NS, int SH, int WGN>
__device__ __forceinline__ void dma_tile_mainloop(const LinearArgs &a, uint16_t *lds, int m0, int n0, int k_begin, int KT,
                                                  int wave, int lane, f32x16 (&acc)[BM / 64][BN / (32 * WGN)]) {
  constexpr int BK = 32, PITCH = BK;
  constexpr int WM = BM / 2, WN = BN / WGN;
  constexpr int MT = WM / 32, NT = WN / 32;
  constexpr int LA = BM / (32 * WGN), LB = BN / (32 * WGN);   // loads per wave per K tile (16 rows each)
  constexpr int STAGE = (BM + BN) * BK;              // elements per stage: A rows then B rows
  const int wm = wave / WGN, wn = wave % WGN;
  // lane -> (row within the 16-row group, swizzled chunk)
  const int lrow = lane >> 2;
  const uint16_t *gpa[LA], *gpb[LB];
#pragma unroll
  for (int j = 0; j < LA; ++j) {
    const int r = (wave * LA + j) * 16 + lrow;   // row within the tile
    int m = m0 + r;
    m = m < a.M ? m : a.M - 1;
    gpa[j] = (const uint16_t *)a.A + (int64_t)m * a.lda + k_begin + (((lane & 3) ^ ((r >> SH) & 3)) << 3);
  }
#pragma unroll
  for (int j = 0; j < LB; ++j) {
    const int r = (wave * LB + j) * 16 + lrow;
    int n = n0 + r;
    n = n < a.N ? n : a.N - 1;
    gpb[j] = (const uint16_t *)a.W + (int64_t)n * a.ldw + k_begin + (((lane & 3) ^ ((r >> SH) & 3)) << 3);
  }
  typedef __attribute__((address_space(3))) void *lds_ptr;
  auto issue = [&](int kt, int stage) {
    kt = kt < KT ? kt : KT - 1;   // past the end: refetch the last tile into a stage nobody reads again
    uint16_t *sa = lds + stage * STAGE + wave * LA * 16 * BK;
    uint16_t *sb = lds + stage * STAGE + BM * BK + wave * LB * 16 * BK;
#pragma unroll
    for (int j = 0; j < LA; ++j)
      __builtin_amdgcn_global_load_lds((const void *)(gpa[j] + kt * BK), (lds_ptr)(sa + j * 16 * BK), 16, 0, 0);
#pragma unroll
    for (int j = 0; j < LB; ++j)
      __builtin_amdgcn_global_load_lds((const void *)(gpb[j] + kt * BK), (lds_ptr)(sb + j * 16 * BK), 16, 0, 0);
  };

#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

#pragma unroll
  for (int t = 0; t < NS - 1; ++t) issue(t, t);

  // Software pipeline of one K tile (BK = 32 = two MFMA K steps, fragment sets F0 and F1):
  //   top:  read F1 (tile t, step 1)            | multiply F0 (tile t, step 0)
  //   mid:  wait for tile t+1, barrier, issue the loads of tile t+NS-1, read F0 (tile t+1, step 0)
  //                                             | multiply F1
  // so LDS reads always run one fragment set ahead of the MFMAs, the barrier sits between two
  // batches of multiplies that are already in the pipe, and global loads are NS-2 tiles ahead.
  const int frow = (lane & 31) * PITCH;
  const int rsw = ((lane & 31) >> SH) & 3;
  const int coff0 = ((0 + (lane >> 5)) ^ rsw) << 3, coff1 = ((2 + (lane >> 5)) ^ rsw) << 3;
  const int a_off = wm * WM * PITCH + frow, b_off = BM * BK + wn * WN * PITCH + frow;
  bf16x8 fa0[MT], fb0[NT], fa1[MT], fb1[NT];
#define RAI_DMA_WAIT(n)                                                                        \
  do {                                                                                         \
    if constexpr ((n) == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");                   \
    else if constexpr ((n) == 4) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");              \
    else if constexpr ((n) == 6) asm volatile("s_waitcnt vmcnt(6)" ::: "memory");              \
    else if constexpr ((n) == 8) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");              \
    else if constexpr ((n) == 12) asm volatile("s_waitcnt vmcnt(12)" ::: "memory");            \
    else if constexpr ((n) == 16) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");            \
    else static_assert((n) < 0, "add the vmcnt immediate for this configuration");             \
  } while (0)
  RAI_DMA_WAIT((LA + LB) * (NS - 2));   // tile 0 has landed (this wave's part)
  __builtin_amdgcn_s_barrier();
  {
    const uint16_t *as = lds + a_off, *bs = lds + b_off;
#pragma unroll
    for (int i = 0; i < MT; ++i) fa0[i] = *reinterpret_cast<const bf16x8 *>(as + i * 32 * PITCH + coff0);
#pragma unroll
    for (int j = 0; j < NT; ++j) fb0[j] = *reinterpret_cast<const bf16x8 *>(bs + j * 32 * PITCH + coff0);
  }
  int cur = 0, nxt = NS - 1;
  // A wave issues in order and an MFMA issue blocks until the matrix pipe is free, so anything placed
  // between two batches of MFMAs runs with the pipe idle.  The LDS reads and the load issues are
  // therefore interleaved one by one between the MFMAs of each half (sched_group_barrier patterns).
  for (int kt = 0; kt < KT; ++kt) {
    {
      const uint16_t *as = lds + cur * STAGE + a_off, *bs = lds + cur * STAGE + b_off;
#pragma unroll
      for (int i = 0; i < MT; ++i) fa1[i] = *reinterpret_cast<const bf16x8 *>(as + i * 32 * PITCH + coff1);
#pragma unroll
      for (int j = 0; j < NT; ++j) fb1[j] = *reinterpret_cast<const bf16x8 *>(bs + j * 32 * PITCH + coff1);
    }
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int j = 0; j < NT; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa0[i], fb0[j], acc[i][j], 0, 0, 0);
#pragma unroll
    for (int g = 0; g < MT + NT; ++g) {
      __builtin_amdgcn_sched_group_barrier(0x008, MT * NT / (MT + NT) > 0 ? MT * NT / (MT + NT) : 1, 0);  // MFMA
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                                                  // one LDS read
    }
    __builtin_amdgcn_sched_barrier(0);
    RAI_DMA_WAIT((LA + LB) * (NS - 3));  // tile kt+1 has landed; NS-3 younger tiles stay in flight
    __builtin_amdgcn_s_barrier();
    issue(kt + NS - 1, nxt);               // into the stage of tile kt-1, which every wave has left
    cur = cur + 1 == NS ? 0 : cur + 1;
    nxt = nxt + 1 == NS ? 0 : nxt + 1;
    {
      const uint16_t *as = lds + cur * STAGE + a_off, *bs = lds + cur * STAGE + b_off;
#pragma unroll
      for (int i = 0; i < MT; ++i) fa0[i] = *reinterpret_cast<const bf16x8 *>(as + i * 32 * PITCH + coff0);
#pragma unroll
      for (int j = 0; j < NT; ++j) fb0[j] = *reinterpret_cast<const bf16x8 *>(bs + j * 32 * PITCH + coff0);
    }
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int j = 0; j < NT; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa1[i], fb1[j], acc[i][j], 0, 0, 0);
#pragma unroll
    for (int g = 0; g < MT + NT; ++g) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // MFMA
      __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);   // one global -> LDS load
      __builtin_amdgcn_sched_group_barrier(0x008, MT * NT / (MT + NT) > 1 ? MT * NT / (MT + NT) - 1 : 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // one LDS read
    }
    __builtin_amdgcn_sched_barrier(0);
  }
#undef RAI_DMA_WAIT
  // the refetches issued past the end must land before the stages are reused for the epilogue
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
}

// The same K loop with K tiles of 64: a tile row is 128 bytes in LDS and one load instruction moves 8 rows x 128 bytes,
// so every request the L1 sends to L2 is a whole 128-byte line instead of half of one (the L2s deliver 1.7x the bytes
// per clock that way with all CUs asking, measured with the loads alone), and there is one barrier per 64 of K.  Two
// stages (the same 128 KB for a 256 x 256 tile as four stages of 32): stage s+1 is requested when stage s-1 has been
// left by every wave, a whole stage of multiplies before it is needed.
//   - 16-byte chunk c (0..7) of row r lives at chunk position c ^ ((r >> 1) & 7): the 8 lanes that fetch one row swap
//     places within their 128-byte line, and a fragment read's 16 lanes per LDS cycle (16 rows at one chunk index; two
//     rows span the 64 banks) land on 16 different 16-byte slots.  (Swizzling by r & 7 left rows r and r + 8 on the
//     same banks: SQ_LDS_BANK_CONFLICT at 23 % of the kernel's cycles.)
//   - fragment sets alternate F0 / F1 over the four K steps of a stage; the reads run one set ahead of the multiplies.
template <int BM, int BN, int WGN, int WGM = 2>
__device__ __forceinline__ void dma_tile_mainloop_k64(const LinearArgs &a, uint16_t *lds, int m0, int n0, int k_begin, int KT,
                                                      int wave, int lane, f32x16 (&acc)[BM / (32 * WGM)][BN / (32 * WGN)]) {
  constexpr int BK = 64;
  constexpr int WM = BM / WGM, WN = BN / WGN;
  constexpr int MT = WM / 32, NT = WN / 32;
  constexpr int NW = WGM * WGN;
  constexpr int LA = BM / (8 * NW), LB = BN / (8 * NW);   // loads per wave per stage (8 rows each)
  constexpr int STAGE = (BM + BN) * BK;
  static_assert(BM % (8 * NW) == 0 && BN % (8 * NW) == 0, "every wave loads whole groups of 8 rows");
  static_assert(LA + LB <= 16, "the wait counts one stage of loads");
  const int wm = wave / WGN, wn = wave % WGN;
  const int lrow = lane >> 3;
  const uint16_t *gpa[LA], *gpb[LB];
#pragma unroll
  for (int j = 0; j < LA; ++j) {
    const int r = (wave * LA + j) * 8 + lrow;     // row within the tile
    int m = m0 + r;
    m = m < a.M ? m : a.M - 1;
    gpa[j] = (const uint16_t *)a.A + (int64_t)m * a.lda + k_begin + (((lane & 7) ^ ((r >> 1) & 7)) << 3);
  }
#pragma unroll
  for (int j = 0; j < LB; ++j) {
    const int r = (wave * LB + j) * 8 + lrow;
    int n = n0 + r;
    n = n < a.N ? n : a.N - 1;
    gpb[j] = (const uint16_t *)a.W + (int64_t)n * a.ldw + k_begin + (((lane & 7) ^ ((r >> 1) & 7)) << 3);
  }
  typedef __attribute__((address_space(3))) void *lds_ptr;
  auto issue = [&](int st, int buf) {
    uint16_t *sa = lds + buf * STAGE + wave * LA * 8 * BK;
    uint16_t *sb = lds + buf * STAGE + BM * BK + wave * LB * 8 * BK;
#pragma unroll
    for (int j = 0; j < LA; ++j)
      __builtin_amdgcn_global_load_lds((const void *)(gpa[j] + st * BK), (lds_ptr)(sa + j * 8 * BK), 16, 0, 0);
#pragma unroll
    for (int j = 0; j < LB; ++j)
      __builtin_amdgcn_global_load_lds((const void *)(gpb[j] + st * BK), (lds_ptr)(sb + j * 8 * BK), 16, 0, 0);
  };

#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  issue(0, 0);
  if (KT > 1) {
    issue(1, 1);
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LA + LB) : "memory");   // stage 0 has landed (this wave's part)
  } else {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }
  __builtin_amdgcn_s_barrier();

  const int frow = (lane & 31) * BK, sw = (lane >> 1) & 7, hi = lane >> 5;   // fragment rows start at multiples of 32
  int coff[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) coff[ks] = ((ks * 2 + hi) ^ sw) << 3;
  const int a_off = wm * WM * BK + frow, b_off = BM * BK + wn * WN * BK + frow;
  bf16x8 fa0[MT], fb0[NT], fa1[MT], fb1[NT];
#define RAI_K64_READ(FA, FB, BUF, KS)                                                                     \
  do {                                                                                                    \
    const uint16_t *as_ = lds + (BUF) * STAGE + a_off + coff[KS], *bs_ = lds + (BUF) * STAGE + b_off + coff[KS]; \
    _Pragma("unroll") for (int i = 0; i < MT; ++i) FA[i] = *reinterpret_cast<const bf16x8 *>(as_ + i * 32 * BK); \
    _Pragma("unroll") for (int j = 0; j < NT; ++j) FB[j] = *reinterpret_cast<const bf16x8 *>(bs_ + j * 32 * BK); \
  } while (0)
#define RAI_K64_MUL(FA, FB)                                                                    \
  do {                                                                                         \
    _Pragma("unroll") for (int i = 0; i < MT; ++i)                                             \
      _Pragma("unroll") for (int j = 0; j < NT; ++j)                                           \
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(FA[i], FB[j], acc[i][j], 0, 0, 0); \
  } while (0)
  // one LDS read between every MT*NT/(MT+NT) multiplies: a wave issues in order, so whatever sits between two
  // batches of MFMAs runs with the matrix pipe idle
#define RAI_K64_MIX_READS()                                                                                \
  do {                                                                                                     \
    _Pragma("unroll") for (int g = 0; g < MT + NT; ++g) {                                                  \
      __builtin_amdgcn_sched_group_barrier(0x008, MT * NT / (MT + NT) > 0 ? MT * NT / (MT + NT) : 1, 0);   \
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                                                   \
    }                                                                                                      \
    __builtin_amdgcn_sched_barrier(0);                                                                     \
  } while (0)
  RAI_K64_READ(fa0, fb0, 0, 0);
  // Every stage but the last in one straight-line block (a branch around the multiplies would split the
  // scheduling region and leave copies of the accumulators at the join).
  for (int st = 0; st + 1 < KT; ++st) {
    const int cur = st & 1;
    RAI_K64_READ(fa1, fb1, cur, 1);
    RAI_K64_MUL(fa0, fb0);
    RAI_K64_MIX_READS();
    RAI_K64_READ(fa0, fb0, cur, 2);
    RAI_K64_MUL(fa1, fb1);
    RAI_K64_MIX_READS();
    RAI_K64_READ(fa1, fb1, cur, 3);
    RAI_K64_MUL(fa0, fb0);
    RAI_K64_MIX_READS();
    // stage st+1 has landed (requested a stage ago) and this wave's reads of stage st are done: after the barrier
    // stage st belongs to the loads of stage st+2 (past the end: the last stage once more, into a buffer nobody reads)
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    issue(st + 2 < KT ? st + 2 : KT - 1, cur);
    RAI_K64_READ(fa0, fb0, cur ^ 1, 0);
    RAI_K64_MUL(fa1, fb1);
#pragma unroll
    for (int g = 0; g < MT + NT; ++g) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // MFMA
      __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);   // one global -> LDS load
      __builtin_amdgcn_sched_group_barrier(0x008, MT * NT / (MT + NT) > 1 ? MT * NT / (MT + NT) - 1 : 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // one LDS read
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  {
    const int cur = (KT - 1) & 1;
    RAI_K64_READ(fa1, fb1, cur, 1);
    RAI_K64_MUL(fa0, fb0);
    RAI_K64_MIX_READS();
    RAI_K64_READ(fa0, fb0, cur, 2);
    RAI_K64_MUL(fa1, fb1);
    RAI_K64_MIX_READS();
    RAI_K64_READ(fa1, fb1, cur, 3);
    RAI_K64_MUL(fa0, fb0);
    RAI_K64_MIX_READS();
    RAI_K64_MUL(fa1, fb1);
  }
#undef RAI_K64_READ
#undef RAI_K64_MUL
#undef RAI_K64_MIX_READS
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
}

template <int BM, int BN, int NS, int SH, int WGN = 2, int WGM = 2>
__global__ void __launch_bounds__(64 * WGM * WGN) k_gemm_bf16_mfma_dma(LinearArgs a, int splits, int k_per_split, float *partial) {
  // block = 2 x WGN waves.  WGN = 4 (eight waves, wave tile (BM/2) x (BN/4)) keeps two waves on every SIMD: one
  // multiplies while the other sits in its wait for the next tile, and twice as many waves issue loads.
  constexpr int BK = 32, PITCH = BK;
  extern __shared__ __attribute__((aligned(16))) uint16_t lds[];

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int tiles_m = (a.M + BM - 1) / BM, tiles_n = (a.N + BN - 1) / BN;
  const int total = tiles_m * tiles_n;
  const int tile = xcd_remap(blockIdx.x, total);
  if (tile >= total) return;
  int tile_m, tile_n;
  tile_coords(tile, tiles_m, tiles_n, &tile_m, &tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int split = blockIdx.y;
  const int k_begin = split * k_per_split;
  const int k_end = k_begin + k_per_split < a.K ? k_begin + k_per_split : a.K;
  const int KT = (k_end - k_begin) / BK;

  f32x16 acc[BM / (32 * WGM)][BN / (32 * WGN)];
  if constexpr (NS == 2) {   // two stages of 64 (the launcher sends K % 64 == 0 and splits of whole stages here)
    dma_tile_mainloop_k64<BM, BN, WGN, WGM>(a, lds, m0, n0, k_begin, KT / 2, wave, lane, acc);
  } else {
    static_assert(WGM == 2, "the K-32 loop is written for two waves along M");
    dma_tile_mainloop<BM, BN, NS, SH, WGN>(a, lds, m0, n0, k_begin, KT, wave, lane, acc);
  }
  gemm_tile_epilogue<BM, BN, dma_lds_bytes<BM, BN, NS, WGN, WGM>(), WGN, WGM>(a, acc, lds, m0, n0, wave, lane, split, partial);
}

// ---- stream-K form of the eight-wave 256x256 tile kernel ---------------------------------------------------------
// One block per CU.  When the tile count is not a multiple of the CU count, the last partial round would leave CUs
// idle for a whole tile time (140 tiles on 256 CUs: 45 % of the machine).  Here the K tiles of those `sk_tiles` tiles
// are dealt out evenly instead: block p (in XCD order, so neighbours share an L2) takes units [start(p), start(p+1))
// of the sk_tiles * KT (tile, K tile) units, i.e. the tail of one tile and the head of the next.  A tile is then the
// work of two or three blocks: each stores its f32 accumulators to its slot of the workspace in register order
// with device-scope stores and counts itself in; the block that arrives
// last adds the slots in slot order (so the sum does not depend on who was last) and runs the epilogue.  Nobody
// waits for anybody.  The remaining tiles follow in whole rounds, one tile per block as before.
struct StreamKArgs {
  int sk_tiles;   // tiles 0 .. sk_tiles-1 are shared out by K tile; the rest run whole
  int q, rem;     // units per block: blocks 0 .. rem-1 take q + 1, the others q
  int max_parts;  // slots per tile in the workspace
  float *ws;      // [sk_tiles][max_parts][BM * BN] f32
  int *counters;  // [sk_tiles][2] (tickets, stored shares), zero between launches
  int *fault;     // host-visible word: RAI_FAULT_STREAMK is stored here when a wait for shares expires
  int spin_limit; // polls of the stored-shares counter before the wait is given up
  int drop_tile;  // test hook: the stored shares of this tile are never counted (-1: none), so its wait must expire
};

__device__ __forceinline__ int sk_start(const StreamKArgs &k, int p) { return p * k.q + (p < k.rem ? p : k.rem); }
__device__ __forceinline__ int sk_block_of(const StreamKArgs &k, int u) {
  const int big = k.rem * (k.q + 1);
  return u < big ? u / (k.q + 1) : k.rem + (u - big) / k.q;
}

template <int BM, int BN, int NS, int SH, int WGN>
__global__ void __launch_bounds__(128 * WGN) k_gemm_bf16_mfma_dma_streamk(LinearArgs a, StreamKArgs sk) {
  constexpr int BK = NS == 2 ? 64 : 32;   // the unit of sharing is one K tile of the main loop
  constexpr int MT = BM / 64, NT = BN / (32 * WGN);
  constexpr int LDS_BYTES = dma_lds_bytes<BM, BN, NS, WGN>();
  extern __shared__ __attribute__((aligned(16))) uint16_t lds[];
  __shared__ int s_ticket;

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int tiles_m = (a.M + BM - 1) / BM, tiles_n = (a.N + BN - 1) / BN;
  const int total = tiles_m * tiles_n;
  const int KT = a.K / BK;
  const int P = gridDim.x;
  const int p = xcd_remap(blockIdx.x, P);   // P is a multiple of the XCD count
  f32x16 acc[MT][NT];

  // one loop over this block's segments (shares of tiles first, then whole tiles), so that the K loop and the
  // epilogue are instantiated once
  int u = sk_start(sk, p);
  const int u_end = sk_start(sk, p + 1);
  int whole = sk.sk_tiles + p;
  for (;;) {
    int tile, kt0, kt1;
    if (u < u_end) {
      tile = u / KT;
      kt0 = u - tile * KT;
      kt1 = kt0 + (u_end - u) < KT ? kt0 + (u_end - u) : KT;
      u += kt1 - kt0;
    } else if (whole < total) {
      tile = whole;
      kt0 = 0;
      kt1 = KT;
      whole += P;
    } else {
      break;
    }
    int tile_m, tile_n;
    tile_coords(tile, tiles_m, tiles_n, &tile_m, &tile_n);
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    __syncthreads();   // the previous segment's epilogue staging is done with the LDS
    if constexpr (NS == 2) {
      dma_tile_mainloop_k64<BM, BN, WGN>(a, lds, m0, n0, kt0 * BK, kt1 - kt0, wave, lane, acc);
    } else {
      dma_tile_mainloop<BM, BN, NS, SH, WGN>(a, lds, m0, n0, kt0 * BK, kt1 - kt0, wave, lane, acc);
    }
    if (kt1 - kt0 != KT) {
      // a share of the tile: which slot is ours, and how many there are
      const int first = sk_block_of(sk, tile * KT), last = sk_block_of(sk, tile * KT + KT - 1);
      const int parts = last - first + 1, slot = p - first;
      // Slot layout [wave][accumulator register][lane]: one store or load instruction covers 256 consecutive bytes.
      // The shares cross XCDs, whose L2s are not coherent with each other: they are written and read with
      // device-scope accesses (write-through stores, loads that miss L2) instead of a release / acquire fence pair
      // -- the fences write back and invalidate a whole L2 each and, issued by every block of an XCD at about the
      // same time, queue up behind one another (measured: +130 us per launch).
      float *tile_ws = sk.ws + (int64_t)tile * sk.max_parts * (BM * BN) + wave * (MT * NT * 16 * 64) + lane;
      // Two counters per tile: `arrived` hands out tickets when a share has been computed, `stored` counts the
      // shares that have reached memory.  The block with the last ticket keeps its share in registers and sums; the
      // others store theirs.  Its wait is for blocks that already hold a ticket, i.e. are running and have nothing
      // left to do but their stores, and it is bounded all the same.
      int *arrived = sk.counters + 2 * tile, *stored = arrived + 1;
      if (tid == 0) s_ticket = __hip_atomic_fetch_add(arrived, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __syncthreads();
      if (s_ticket != parts - 1) {
        float *mine = tile_ws + (int64_t)slot * (BM * BN);
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
          for (int j = 0; j < NT; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r)
              __hip_atomic_store(mine + ((i * NT + j) * 16 + r) * 64, acc[i][j][r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this wave's share has left for memory
        __syncthreads();
        if (tid == 0 && tile != sk.drop_tile) __hip_atomic_fetch_add(stored, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        continue;
      }
      if (tid == 0) {
        bool complete = false;
        for (int spin = 0; spin < sk.spin_limit && !complete; ++spin) {
          complete = __hip_atomic_load(stored, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == parts - 1;
          if (!complete) __builtin_amdgcn_s_sleep(2);
        }
        if (complete) {
          __hip_atomic_store(arrived, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __hip_atomic_store(stored, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else {
          // A share is missing.  Nothing is summed and nothing written for this tile, the counters stay as they are
          // (a late block may still count itself in; the host zeroes them all before the next launch), and the
          // host learns of it at its next synchronisation.
          __hip_atomic_store(sk.fault, (int)RAI_FAULT_STREAMK, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
          s_ticket = -1;
        }
      }
      __syncthreads();
      if (s_ticket < 0) continue;
      // the other slots are complete.  Sum in slot order, our registers standing in for our slot, so the result does
      // not depend on who came last.
#pragma unroll
      for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j) {
          f32x16 sum = acc[i][j];
          for (int s = 0; s < parts; ++s) {
            if (s == slot) {
              if (s > 0) {
#pragma unroll
                for (int r = 0; r < 16; ++r) sum[r] += acc[i][j][r];
              }
              continue;
            }
            const float *src = tile_ws + (int64_t)s * (BM * BN) + ((i * NT + j) * 16) * 64;
            f32x16 v;
#pragma unroll
            for (int r = 0; r < 16; ++r) v[r] = __hip_atomic_load(src + r * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (s == 0) sum = v;
            else {
#pragma unroll
              for (int r = 0; r < 16; ++r) sum[r] += v[r];
            }
          }
          acc[i][j] = sum;
        }
    }
    gemm_tile_epilogue<BM, BN, LDS_BYTES, WGN>(a, acc, lds, m0, n0, wave, lane, 0, nullptr);
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

// The same pass for a Linear whose output rows are normalised next.  A block of four waves owns a row (N <= 512 *
// ITEMS columns).  The sums over the partial products, bias / activation / residual and the bf16 store are element
// by element, so they are shared out: every wave takes a quarter of the row's 16-byte packs (512 rows are then eight
// waves per CU with one round of loads each, instead of two waves with two rounds).  The stored (rounded) row goes
// through LDS to the first wave, which runs LayerNorm on it with the arithmetic of the stand-alone norm kernel -- same
// per-lane order, same wave reductions -- so fusing changes no bit (rai-nn/src/layer_norm.rs:32-42).
template <int ITEMS>
__global__ void __launch_bounds__(256) k_splitk_epilogue_ln(LinearArgs a, int splits, const float *partial) {
  constexpr int NWV = 4;                                 // waves per row
  constexpr int JT = (ITEMS * 64 / NWV + 63) / 64;       // packs per lane in the summing part
  __shared__ u32x4 rowbuf[64 * ITEMS];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int row = blockIdx.x;
  const int packs = a.N / 8;
  const int quarter = (packs + NWV - 1) / NWV;
  const int64_t total = (int64_t)a.M * a.N;
  const uint16_t *bias = (const uint16_t *)a.bias, *bias2 = (const uint16_t *)a.bias2;
  const uint16_t *res = (const uint16_t *)a.residual;
  {
    // loads are issued as early and as many at a time as the registers allow: bias and residual first, then the
    // partial products of all the lane's packs (six splits each), while every element's additions stay in split order
    int pk[JT];
    bool on[JT];
    u32x4 braw[JT], b2raw[JT], rraw[JT];
    float x[JT][8];
#pragma unroll
    for (int j = 0; j < JT; ++j) {
      const int q = lane + j * 64;
      pk[j] = wv * quarter + q;
      on[j] = q < quarter && pk[j] < packs;
      if (!on[j]) pk[j] = 0;   // a clamped pack is loaded and never used
      const int n = pk[j] * 8;
      braw[j] = b2raw[j] = rraw[j] = u32x4{0u, 0u, 0u, 0u};
      if (bias) braw[j] = *reinterpret_cast<const u32x4 *>(bias + n);
      if (bias2) b2raw[j] = *reinterpret_cast<const u32x4 *>(bias2 + n);
      if (res) rraw[j] = *reinterpret_cast<const u32x4 *>(res + (int64_t)row * a.ldr + n);
#pragma unroll
      for (int e = 0; e < 8; ++e) x[j][e] = 0.f;
    }
    for (int s0 = 0; s0 < splits; s0 += 6) {
      f32x4 p0[JT][6], p1[JT][6];
#pragma unroll
      for (int j = 0; j < JT; ++j)
#pragma unroll
        for (int u = 0; u < 6; ++u) {
          const int sp = s0 + u < splits ? s0 + u : splits - 1;
          const float *pp = partial + (int64_t)sp * total + (int64_t)row * a.N + pk[j] * 8;
          p0[j][u] = *reinterpret_cast<const f32x4 *>(pp);
          p1[j][u] = *reinterpret_cast<const f32x4 *>(pp + 4);
        }
#pragma unroll
      for (int j = 0; j < JT; ++j)
#pragma unroll
        for (int u = 0; u < 6; ++u) {
          if (s0 + u < splits) {
            x[j][0] += p0[j][u].x; x[j][1] += p0[j][u].y; x[j][2] += p0[j][u].z; x[j][3] += p0[j][u].w;
            x[j][4] += p1[j][u].x; x[j][5] += p1[j][u].y; x[j][6] += p1[j][u].z; x[j][7] += p1[j][u].w;
          }
        }
    }
#pragma unroll
    for (int j = 0; j < JT; ++j) {
      if (on[j]) {
        const int n = pk[j] * 8;
        float b1[8], b2[8];
        unpack8(braw[j], b1);     // zero bits where there is no bias: +0.0
        unpack8(b2raw[j], b2);
#pragma unroll
        for (int e = 0; e < 8; ++e) x[j][e] += b1[e] + b2[e];
        if (a.act >= 0) act8(a.act, x[j], n, a.act_from);
        if (res) {
          float rv[8];
          unpack8(rraw[j], rv);
#pragma unroll
          for (int e = 0; e < 8; ++e) x[j][e] += rv[e];
        }
        u32x4 o;
        o.x = (uint32_t)f32_to_bf16_bits(x[j][0]) | ((uint32_t)f32_to_bf16_bits(x[j][1]) << 16);
        o.y = (uint32_t)f32_to_bf16_bits(x[j][2]) | ((uint32_t)f32_to_bf16_bits(x[j][3]) << 16);
        o.z = (uint32_t)f32_to_bf16_bits(x[j][4]) | ((uint32_t)f32_to_bf16_bits(x[j][5]) << 16);
        o.w = (uint32_t)f32_to_bf16_bits(x[j][6]) | ((uint32_t)f32_to_bf16_bits(x[j][7]) << 16);
        *reinterpret_cast<u32x4 *>((uint16_t *)a.out1 + (int64_t)row * a.ld1 + n) = o;
        rowbuf[pk[j]] = o;
      }
    }
  }
  __syncthreads();
  if (wv != 0) return;
  // ---- LayerNorm of the stored row, one wave, pack p = lane + 64 it
  float v[ITEMS][8];
  float s = 0.f;
#pragma unroll
  for (int it = 0; it < ITEMS; ++it) {
    const int p = lane + it * 64;
    if (p < packs) {
      unpack8(rowbuf[p], v[it]);
#pragma unroll
      for (int e = 0; e < 8; ++e) s += v[it][e];
    }
  }
  s = wave_sum(s);
  const float mean = s / (float)a.N;
  float q = 0.f;
#pragma unroll
  for (int it = 0; it < ITEMS; ++it) {
    const int p = lane + it * 64;
    if (p < packs) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float d = v[it][e] - mean;
        q += d * d;
      }
    }
  }
  q = wave_sum(q);
  const float scale = 1.0f / sqrtf(q / (float)a.N + a.post_ln_eps);
  const uint16_t *lw = (const uint16_t *)a.post_ln_w, *lb = (const uint16_t *)a.post_ln_b;
#pragma unroll
  for (int it = 0; it < ITEMS; ++it) {
    const int p = lane + it * 64;
    if (p < packs) {
      const int n = p * 8;
      float wv[8], bv[8];
      if (lw) unpack8(*reinterpret_cast<const u32x4 *>(lw + n), wv);
      if (lb) unpack8(*reinterpret_cast<const u32x4 *>(lb + n), bv);
      uint32_t h[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float y = (v[it][e] - mean) * scale;
        if (lw) y *= wv[e];
        if (lb) y += bv[e];
        h[e] = f32_to_bf16_bits(y);
      }
      u32x4 o = {h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16)};
      *reinterpret_cast<u32x4 *>((uint16_t *)a.post_ln_out + (int64_t)row * a.N + n) = o;
    }
  }
}

// Whether the pass over the partial sums can also normalise the rows: one ungated output, whole 16-byte packs.
static bool post_norm_fits(const LinearArgs &a) {
  auto al16 = [](const void *p) { return ((uintptr_t)p & 15) == 0; };
  return a.post_ln_out && !a.glu && a.n_split >= a.N && a.N % 8 == 0 && a.N <= 4096 && a.ld1 % 8 == 0 && al16(a.out1) &&
         al16(a.post_ln_out) && (!a.bias || al16(a.bias)) && (!a.bias2 || al16(a.bias2)) &&
         (!a.residual || (a.ldr % 8 == 0 && al16(a.residual))) && (!a.post_ln_w || al16(a.post_ln_w)) &&
         (!a.post_ln_b || al16(a.post_ln_b)) && a.splitk_ws && ((uintptr_t)a.splitk_ws & 15) == 0;
}
// Sums the partial products of a tile GEMM that split K (and normalises the rows when asked to and possible).
static int launch_splitk_epilogue(hipStream_t st, const LinearArgs &a, int splits, const float *partial) {
  if (post_norm_fits(a)) {
    const int items = (a.N / 8 + 63) / 64;
    const dim3 grid(a.M), block(256);
    if (items <= 2) hipLaunchKernelGGL(k_splitk_epilogue_ln<2>, grid, block, 0, st, a, splits, partial);
    else if (items <= 5) hipLaunchKernelGGL(k_splitk_epilogue_ln<5>, grid, block, 0, st, a, splits, partial);
    else hipLaunchKernelGGL(k_splitk_epilogue_ln<8>, grid, block, 0, st, a, splits, partial);
    return launch_check("splitk_epilogue_ln");
  }
  const int64_t total = (int64_t)a.M * a.N;
  const int blocks = (int)((total + 255) / 256 < 4096 ? (total + 255) / 256 : 4096);
  hipLaunchKernelGGL(k_splitk_epilogue, dim3(blocks), dim3(256), 0, st, a, splits, partial);
  return launch_check("splitk_epilogue");
}

template <int BM, int BN, int BK, int SH = 0> static int launch_cfg(hipStream_t st, const LinearArgs &a, int splits) {
  constexpr size_t lds = gemm_lds_bytes<BM, BN, (SH ? BK : BK + 8)>();
  static bool attr_set = false;
  if (lds > 64 * 1024 && !attr_set) {
    RAI_HIP_TRY(hipFuncSetAttribute((const void *)k_gemm_bf16_mfma<BM, BN, BK, SH>,
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
  hipLaunchKernelGGL((k_gemm_bf16_mfma<BM, BN, BK, SH>), dim3(grid_x, splits), dim3(256), lds, st, a, splits, k_per_split,
                     partial);
  RAI_TRY(launch_check("gemm_bf16_mfma"));
  if (splits > 1) RAI_TRY(launch_splitk_epilogue(st, a, splits, (const float *)partial));
  return RAI_OK;
}

template <int BM, int BN, int NS, int SH, int WGN = 2, int WGM = 2>
static int launch_cfg_dma(hipStream_t st, const LinearArgs &a, int splits) {
  constexpr size_t lds = dma_lds_bytes<BM, BN, NS, WGN, WGM>();
  static bool attr_set = false;
  if (lds > 64 * 1024 && !attr_set) {
    RAI_HIP_TRY(hipFuncSetAttribute((const void *)k_gemm_bf16_mfma_dma<BM, BN, NS, SH, WGN, WGM>,
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attr_set = true;
  }
  const int tiles = ((a.M + BM - 1) / BM) * ((a.N + BN - 1) / BN);
  const int grid_x = ((tiles + kXcds - 1) / kXcds) * kXcds;
  int k_per_split = a.K;
  float *partial = nullptr;
  if (splits > 1) {
    constexpr int KU = NS == 2 ? 64 : 32;   // K tile of the main loop
    const int k_tiles = a.K / KU, per = (k_tiles + splits - 1) / splits;
    splits = (k_tiles + per - 1) / per;
    k_per_split = per * KU;
    partial = (float *)a.splitk_ws;
  }
  hipLaunchKernelGGL((k_gemm_bf16_mfma_dma<BM, BN, NS, SH, WGN, WGM>), dim3(grid_x, splits), dim3(64 * WGM * WGN), lds, st, a,
                     splits, k_per_split, partial);
  RAI_TRY(launch_check("gemm_bf16_mfma_dma"));
  if (splits > 1) RAI_TRY(launch_splitk_epilogue(st, a, splits, (const float *)partial));
  return RAI_OK;
}

// Arrival counters of the stream-K kernel, one per shared tile; every launch leaves them at zero.
static __device__ int g_streamk_counters[4 * kNumCU];

// How the stream-K kernel would share out an M x N x K product: false when it does not apply (tile count a multiple
// of the CU count, too few tiles, or a tile would be the work of more than three blocks).
struct StreamKPlan {
  StreamKArgs k;
  size_t ws_bytes;
};
static bool streamk_plan(int M, int N, int K, int bk, StreamKPlan *plan, bool forced = false) {
  const int P = kNumCU, KT = K / bk;
  const int T = ((M + 255) / 256) * ((N + 255) / 256);
  const int full = T / P, left = T % P;
  if (left == 0 || K / 32 < 8) return false;
  int sk_tiles = left;
  if (left < P / 2) {
    if (full == 0) return false;
    sk_tiles = left + P;   // a whole round joins the shared part: every block then works on two tiles at most
  }
  const long long units = (long long)sk_tiles * KT;
  StreamKArgs k;
  k.sk_tiles = sk_tiles;
  k.q = (int)(units / P);
  k.rem = (int)(units % P);
  if (k.q < 1) return false;
  auto block_of = [&](int u) {
    const int big = k.rem * (k.q + 1);
    return u < big ? u / (k.q + 1) : k.rem + (u - big) / k.q;
  };
  int max_parts = 1;
  for (int t = 0; t < sk_tiles; ++t) {
    const int parts = block_of(t * KT + KT - 1) - block_of(t * KT) + 1;
    if (parts > max_parts) max_parts = parts;
  }
  if (max_parts > 3 || sk_tiles > 2 * kNumCU) return false;
  // Worth it when the CU time saved exceeds what the exchange of the shares costs.  Measured with cold weights, bias
  // and gelu_new: 4096 x 10240 x 2560 (two shares per tile, 40 K tiles of a round saved) 237 -> 215 us, i.e. ~18 us
  // for the exchange; 512 x 17920 x 2560 (three shares, 36 saved) 81 -> 84 us, i.e. ~39 us: every block ends on a
  // read of the other shares plus the epilogue, with nothing left to hide them behind.  One K tile of a 256 x 256
  // tile takes ~1 us with all CUs busy.
  const float saved_us = (float)(P - left) / P * (K / 32) * 1.0f;
  const float exchange_us = max_parts <= 2 ? 18.f : 39.f;
  if (!forced && saved_us < 1.3f * exchange_us) return false;
  k.max_parts = max_parts;
  k.ws = nullptr;
  k.counters = nullptr;
  plan->k = k;
  plan->ws_bytes = (size_t)sk_tiles * max_parts * 256 * 256 * sizeof(float);
  return true;
}

size_t linear_streamk_workspace_bytes(int M, int N, int K) {
  StreamKPlan plan;
  return streamk_plan(M, N, K, 32, &plan) ? plan.ws_bytes : 0;
}

static int linear_device(const LinearArgs &a, int *dev) {
  *dev = a.dev;
  if (*dev < 0) RAI_HIP_TRY(hipGetDevice(dev));
  RAI_REQUIRE(*dev >= 0 && *dev < 64, RAI_ERR_BAD_ARG, "device %d out of range", *dev);
  return RAI_OK;
}

// True when the stream-K kernel serves this Linear (plain tile epilogue, workspace large enough, not switched off).
static bool streamk_applies(const LinearArgs &a, int bk, StreamKPlan *plan, bool forced = false) {
  const char *off = getenv("RAI_HIP_NO_STREAMK");   // read per call: tests compare both forms in one process
  if (off && *off && *off != '0') return false;
  if (!a.splitk_ws || ((uintptr_t)a.splitk_ws & 15) || a.post_ln_out) return false;
  // one block per CU of a 256-CU part: the plan, the counter array and the XCD order are laid out for that grid
  int dev = -1;
  if (linear_device(a, &dev) != RAI_OK || device_cu_count(dev) != kNumCU) return false;
  return a.K % bk == 0 && streamk_plan(a.M, a.N, a.K, bk, plan, forced) && plan->ws_bytes <= a.splitk_ws_bytes;
}

// every GPU holds its own copy of a __device__ array at its own address: looked up once per device
template <typename Sym> static int *device_ints_of(int dev, int *(&cache)[64], const Sym &symbol) {
  if (dev < 0 || dev >= 64) return nullptr;
  if (!cache[dev]) {
    int cur = -1;
    void *p = nullptr;
    if (hipGetDevice(&cur) != hipSuccess || (cur != dev && hipSetDevice(dev) != hipSuccess)) return nullptr;
    if (hipGetSymbolAddress(&p, symbol) == hipSuccess) cache[dev] = (int *)p;
    if (cur != dev) (void)hipSetDevice(cur);
  }
  return cache[dev];
}
static int *streamk_counters_of(int dev) {
  static int *counters[64];
  return device_ints_of(dev, counters, HIP_SYMBOL(g_streamk_counters));
}
// Tickets of the small-M streaming Linear's K split, one per group of weight tiles; zero between launches (the block
// that takes a group's last ticket puts it back).  Launches that overlap on one GPU would share them: the library
// runs a device's work on one stream.
constexpr int kSplitTickets = 16384;
static __device__ int g_splitk_tickets[kSplitTickets];
static int *splitk_tickets_of(int dev) {
  static int *tickets[64];
  return device_ints_of(dev, tickets, HIP_SYMBOL(g_splitk_tickets));
}

int streamk_counters_reset(int dev, hipStream_t st) {
  int *c = streamk_counters_of(dev), *t = splitk_tickets_of(dev);
  RAI_REQUIRE(c && t, RAI_ERR_HIP, "stream-K counters of device %d not found", dev);
  RAI_HIP_TRY(hipMemsetAsync(c, 0, sizeof(int) * 4 * kNumCU, st));
  RAI_HIP_TRY(hipMemsetAsync(t, 0, sizeof(int) * kSplitTickets, st));
  return RAI_OK;
}

template <int NS>
static int launch_streamk(hipStream_t st, const LinearArgs &a, StreamKPlan plan) {
  constexpr int BM = 256, BN = 256, SH = 2, WGN = 4;
  constexpr size_t lds = dma_lds_bytes<BM, BN, NS, WGN>();
  int dev = 0;
  RAI_TRY(linear_device(a, &dev));
  static bool attr_set[64];
  if (!attr_set[dev]) {
    RAI_HIP_TRY(hipFuncSetAttribute((const void *)k_gemm_bf16_mfma_dma_streamk<BM, BN, NS, SH, WGN>,
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attr_set[dev] = true;
  }
  plan.k.ws = (float *)a.splitk_ws;
  plan.k.counters = streamk_counters_of(dev);
  plan.k.fault = kernel_fault_word(dev);
  RAI_REQUIRE(plan.k.counters && plan.k.fault, RAI_ERR_HIP, "stream-K: device %d has no counters / fault word", dev);
  plan.k.spin_limit = 1 << 20;
  plan.k.drop_tile = -1;
  // RAI_HIP_STREAMK_TEST="<spin limit>,<tile>": a tiny wait and one tile whose shares are never counted, so that the
  // expiry path runs with every wave still exiting normally (read per launch; the tests set it around one call)
  if (const char *t = getenv("RAI_HIP_STREAMK_TEST")) {
    int lim = 0, tile = -1;
    if (sscanf(t, "%d,%d", &lim, &tile) == 2 && lim > 0) { plan.k.spin_limit = lim; plan.k.drop_tile = tile; }
  }
  hipLaunchKernelGGL((k_gemm_bf16_mfma_dma_streamk<BM, BN, NS, SH, WGN>), dim3(kNumCU), dim3(128 * WGN), lds, st, a, plan.k);
  return launch_check("gemm_bf16_mfma_dma_streamk");
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
// Fragment-major copy of W: element j of lane l of (row tile t, K step s) is W[16 t + l % 16][32 s + 8 (l / 16) + j].
__global__ void __launch_bounds__(256) k_linear_fragment_layout(bf16x8 *out, const uint16_t *W, int64_t ldw, int N, int ksteps,
                                                                int64_t total) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int lane = (int)(i & 63);
    const int64_t ts = i >> 6;
    const int s = (int)(ts % ksteps);
    const int64_t t = ts / ksteps;
    const int64_t n = t * 16 + (lane & 15);
    bf16x8 v = {};
    if (n < N) v = *reinterpret_cast<const bf16x8 *>(W + n * ldw + s * 32 + (lane >> 4) * 8);
    out[i] = v;
  }
}
size_t linear_fragment_elems(int N, int K) { return (size_t)((N + 15) / 16) * 16 * (size_t)K; }
int launch_linear_fragment_layout(hipStream_t st, const void *W, int64_t ldw, int N, int K, void *Wfrag) {
  RAI_REQUIRE(K % 32 == 0 && ldw % 8 == 0 && (uintptr_t)W % 16 == 0 && (uintptr_t)Wfrag % 16 == 0, RAI_ERR_BAD_STRIDE,
              "fragment layout: K must be a multiple of 32 and the operands 16-byte aligned");
  const int64_t total = (int64_t)((N + 15) / 16) * (K / 32) * 64;
  const int64_t blocks = (total + 255) / 256;
  hipLaunchKernelGGL(k_linear_fragment_layout, dim3((unsigned)(blocks < 65535 ? blocks : 65535)), dim3(256), 0, st,
                     (bf16x8 *)Wfrag, (const uint16_t *)W, ldw, N, K / 32, total);
  return launch_check("linear_fragment_layout");
}

// 16 bytes to or from memory past the (per-XCD, mutually incoherent) L2s: for data that another block of the same
// launch reads or wrote (p is 16-byte aligned)
__device__ __forceinline__ void store_f32x4_device(float *p, f32x4 v) {
  unsigned long long *q = reinterpret_cast<unsigned long long *>(p);
  __hip_atomic_store(q, (unsigned long long)__float_as_uint(v.x) | ((unsigned long long)__float_as_uint(v.y) << 32), __ATOMIC_RELAXED,
                     __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store(q + 1, (unsigned long long)__float_as_uint(v.z) | ((unsigned long long)__float_as_uint(v.w) << 32), __ATOMIC_RELAXED,
                     __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ f32x4 load_f32x4_device(const float *p) {
  const unsigned long long *q = reinterpret_cast<const unsigned long long *>(p);
  const unsigned long long lo = __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const unsigned long long hi = __hip_atomic_load(q + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return f32x4{__uint_as_float((uint32_t)lo), __uint_as_float((uint32_t)(lo >> 32)), __uint_as_float((uint32_t)hi),
               __uint_as_float((uint32_t)(hi >> 32))};
}

template <int MT, int KS, int G, bool FRAG>
__global__ void __launch_bounds__(512) k_linear_bf16_mfma_stream(LinearArgs a, int tiles, float *partial, int *tickets) {
  __shared__ int s_ticket;
  constexpr int NW = 8;
  extern __shared__ __attribute__((aligned(16))) uint16_t lds[];
  constexpr int PCH = 4 * G + 1;                       // row pitch of the parked accumulators, in f32x4
  f32x4 *red = reinterpret_cast<f32x4 *>(lds);        // [NW][MT * 16 rows][PCH]
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lrow = lane & 15, lq = lane >> 4;
  const int split = blockIdx.y;
  const int k0 = (split * NW + wave) * KS * 32;

  int koff[KS];   // K steps beyond K read column 0 (their activation fragments are zero)
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) koff[ks] = k0 + ks * 32 < a.K ? k0 + ks * 32 : 0;
  const uint16_t *wbase = (const uint16_t *)a.W + lq * 8;
  const bf16x8 *fbase = reinterpret_cast<const bf16x8 *>(a.Wfrag) + lane;
  const int ksteps = a.K / 32;

  // A ring of tile buffers: while tile t is multiplied, the next RING-1 tiles are in flight.  Long streams (four
  // tiles per group, i.e. at least four tiles per block) take three buffers and loads that bypass the caches
  // (measured on a 1 GB matrix: 232 -> 193 us); short ones keep two buffers and cached loads, which a 10 MB matrix on
  // 160 blocks prefers by 1-2 us.  The ring turns by G positions per group, so the group body exists in RING rotations.
  constexpr int RING = G >= 4 ? 3 : 2;
  constexpr bool NT = G >= 4;
  bf16x8 w[RING][KS];
  auto load_tile = [&](bf16x8 (&wt)[KS], int tile) {
    tile = tile < tiles ? tile : tiles - 1;
    if constexpr (FRAG) {   // one instruction reads 1 KB of consecutive memory
      const bf16x8 *p = fbase + (int64_t)tile * ksteps * 64;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) wt[ks] = NT ? __builtin_nontemporal_load(p + (koff[ks] >> 5) * 64) : p[(koff[ks] >> 5) * 64];
    } else {
      int n = tile * 16 + lrow;
      n = n < a.N ? n : a.N - 1;
      const uint16_t *p = wbase + (int64_t)n * a.ldw;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        wt[ks] = NT ? __builtin_nontemporal_load(reinterpret_cast<const bf16x8 *>(p + koff[ks])) : *reinterpret_cast<const bf16x8 *>(p + koff[ks]);
    }
    // keep the whole tile's loads together and ahead of the multiplies that follow: left alone,
    // the scheduler sinks each load to just before its use and the prefetch distance collapses
    __builtin_amdgcn_sched_barrier(0);
  };
  const int stride = gridDim.x * G;
  // tile at position pos (0 .. G + RING - 2) counted from the start of the group that begins at tile g0
  auto tile_at = [&](int g0, int pos) { return g0 + (pos / G) * stride + pos % G; };
  // The block's first tiles are asked for behind the activation fragments (which come from the L2 and are needed
  // first: loads return in order) and, with a fused norm, before its statistics go round the block.
  int g0 = blockIdx.x * G;
  auto first_tiles = [&]() {
#pragma unroll
    for (int pos = 0; pos + 1 < RING; ++pos) load_tile(w[pos], tile_at(g0, pos));
  };
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
  // Optional RMSNorm of the activation rows (ln_kind 1: x * w / rms, 2: x * (1 + w) / rms), K not split
  // over blocks: the sum of squares of a row is gathered from the four lanes and eight waves that hold
  // its pieces, then every fragment is scaled and rounded to bf16 exactly as the stand-alone kernel does.
  if (a.ln_kind > 0) {
    float *rs = reinterpret_cast<float *>(lds);   // [8 waves][MT * 16 rows]; the accumulator area is not in use yet
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
    first_tiles();   // on their way while the row statistics go round the block
    // the widened values of the statistics pass are not kept for the scaling pass (256 registers: they would spill)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+v"(xf[mt][ks]));
    __syncthreads();
    const uint16_t *lw = (const uint16_t *)a.ln_w;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      float tot = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) tot += rs[w * (MT * 16) + mt * 16 + lrow];
      const float scale = 1.0f / sqrtf(tot / (float)a.K + a.ln_eps);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const int k = k0 + ks * 32;
        if (k < a.K) {
          const bf16x8 wv = *reinterpret_cast<const bf16x8 *>(lw + k + lq * 8);
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const float wf = (float)wv[j];
            xf[mt][ks][j] = (__bf16)((float)xf[mt][ks][j] * scale * (a.ln_kind == 2 ? 1.0f + wf : wf));
          }
        }
      }
    }
    __syncthreads();   // the statistics have been read before the area is reused
  } else {
    first_tiles();
  }
  const uint16_t *bias = (const uint16_t *)a.bias;
  const uint16_t *bias2 = (const uint16_t *)a.bias2;
  const uint16_t *res = (const uint16_t *)a.residual;
  // bias, activation / gated pair, residual and the bf16 store of four consecutive columns n .. n+3 of row m
  auto finish = [&](int m, int n, f32x4 s4) __attribute__((always_inline)) {
    const float x[4] = {s4.x, s4.y, s4.z, s4.w};
    const int lim = a.N - n < 4 ? a.N - n : 4;
    if (a.glu) {   // columns (n, n+1) and (n+2, n+3) are (gate, up) pairs (N is a multiple of 8)
      uint16_t o[2];
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const float gt = x[2 * e] + (bias ? bf16_bits_to_f32(bias[n + 2 * e]) : 0.f);
        const float up = x[2 * e + 1] + (bias ? bf16_bits_to_f32(bias[n + 2 * e + 1]) : 0.f);
        o[e] = f32_to_bf16_bits(glu_bf16(a.act, gt, up));
      }
      uint16_t *dst = (uint16_t *)a.out1 + (int64_t)m * a.ld1 + (n >> 1);
      if (((uintptr_t)dst & 3) == 0) *reinterpret_cast<uint32_t *>(dst) = (uint32_t)o[0] | ((uint32_t)o[1] << 16);
      else { dst[0] = o[0]; dst[1] = o[1]; }
      return;
    }
    uint16_t o[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int nn = e < lim ? n + e : n;
      float y = x[e] + ((bias ? bf16_bits_to_f32(bias[nn]) : 0.f) + (bias2 ? bf16_bits_to_f32(bias2[nn]) : 0.f));
      if (a.act >= 0 && nn >= a.act_from) y = act_eval(a.act, y);
      if (res) y += bf16_bits_to_f32(res[(int64_t)m * a.ldr + nn]);
      o[e] = f32_to_bf16_bits(y);
    }
    // all four columns in one output and the destination 8-byte aligned: one store
    const bool first = n + 3 < a.n_split, second = n >= a.n_split;
    uint16_t *dst = second ? (uint16_t *)a.out2 + (int64_t)m * a.ld2 + (n - a.n_split) : (uint16_t *)a.out1 + (int64_t)m * a.ld1 + n;
    if (lim == 4 && (first || second) && ((uintptr_t)dst & 7) == 0) {
      typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
      const u32x2 pk = {(uint32_t)o[0] | ((uint32_t)o[1] << 16), (uint32_t)o[2] | ((uint32_t)o[3] << 16)};
      *reinterpret_cast<u32x2 *>(dst) = pk;
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (e < lim) {
          const int nn = n + e;
          if (nn < a.n_split) ((uint16_t *)a.out1)[(int64_t)m * a.ld1 + nn] = o[e];
          else ((uint16_t *)a.out2)[(int64_t)m * a.ld2 + (nn - a.n_split)] = o[e];
        }
      }
    }
  };
  auto group = [&](auto rot, const int g0) {
    constexpr int R = decltype(rot)::value;
    f32x4 acc[G][MT];
#pragma unroll
    for (int j = 0; j < G; ++j)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[j][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < G; ++j) {
      load_tile(w[(R + j + RING - 1) % RING], tile_at(g0, j + RING - 1));
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[j][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[(R + j) % RING][ks], xf[mt][ks], acc[j][mt], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    // ---- sum the eight K slices and write G tiles of 16 columns x 16*MT rows.
    // Every wave parks its accumulators as [row m][G tiles x 4 column quads] (pitch PCH = 4 G + 1 chunks of 16 bytes,
    // odd, so that the 16 lanes of a quad, one row each, hit distinct banks); a thread then owns four consecutive
    // columns of one row: eight 16-byte reads, one store of four bf16, and 16 neighbouring threads cover 64 columns of
    // a row.  (One 4-byte read per wave and element and 2-byte stores a row apart took as long as streaming the
    // group's weights.)
    __syncthreads();   // the previous group's sums have been read
#pragma unroll
    for (int j = 0; j < G; ++j)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) red[(wave * MT * 16 + mt * 16 + lrow) * PCH + j * 4 + lq] = acc[j][mt];
    __syncthreads();
    for (int v = tid; v < MT * G * 64; v += 512) {
      const int m = v / (G * 4), c = v - m * (G * 4);
      const int tile = g0 + (c >> 2);
      const int n = tile * 16 + 4 * (c & 3);
      if (tile >= tiles || n >= a.N || m >= a.M) continue;
      f32x4 s4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int w = 0; w < NW; ++w) {
        const f32x4 t = red[(w * MT * 16 + m) * PCH + c];
        s4.x += t.x; s4.y += t.y; s4.z += t.z; s4.w += t.w;
      }
      if (partial) {
        float *p = partial + ((int64_t)split * a.M + m) * a.N + n;
        if (tickets) {   // read by another block of this launch: past the L2 (N is a multiple of 4, checked on the host)
          store_f32x4_device(p, s4);
        } else if (a.N - n >= 4 && a.N % 4 == 0) {
          *reinterpret_cast<f32x4 *>(p) = s4;
        } else {
          const float x[4] = {s4.x, s4.y, s4.z, s4.w};
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + e < a.N) p[e] = x[e];
        }
        continue;
      }
      finish(m, n, s4);
    }
    if (partial && tickets) {
      // K split over blocks without a second launch: a block counts itself in once its partial sums have reached
      // memory, and the block that counts last -- whichever it is -- adds all of them in split order (the order of
      // the separate summing pass, so the result is the same bit for bit) and runs the epilogue.  Nobody waits.
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      int *ticket = tickets + g0 / G;
      if (tid == 0) s_ticket = __hip_atomic_fetch_add(ticket, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __syncthreads();
      if (s_ticket == (int)gridDim.y - 1) {
        if (tid == 0) __hip_atomic_store(ticket, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // for the next launch
        for (int v = tid; v < MT * G * 64; v += 512) {
          const int m = v / (G * 4), c = v - m * (G * 4);
          const int tile = g0 + (c >> 2);
          const int n = tile * 16 + 4 * (c & 3);
          if (tile >= tiles || n >= a.N || m >= a.M) continue;
          f32x4 s4 = {0.f, 0.f, 0.f, 0.f};
          for (int sp = 0; sp < (int)gridDim.y; ++sp) {
            const f32x4 t = load_f32x4_device(partial + ((int64_t)sp * a.M + m) * a.N + n);
            s4.x += t.x; s4.y += t.y; s4.z += t.z; s4.w += t.w;
          }
          finish(m, n, s4);
        }
      }
    }
  };
  for (;;) {
    group(std::integral_constant<int, 0>{}, g0);
    if ((g0 += stride) >= tiles) break;
    group(std::integral_constant<int, G % RING>{}, g0);
    if ((g0 += stride) >= tiles) break;
    if constexpr (RING == 3) {
      group(std::integral_constant<int, (2 * G) % RING>{}, g0);
      if ((g0 += stride) >= tiles) break;
    }
  }
}

template <int MT, int KS, int G, bool FRAG = false>
static int launch_mfma_stream_cfg(hipStream_t st, const LinearArgs &a, int splits) {
  if constexpr (!FRAG) {
    if (a.Wfrag) return launch_mfma_stream_cfg<MT, KS, G, true>(st, a, splits);
  }
  const int tiles = (a.N + 15) / 16;
  const int groups = (tiles + G - 1) / G;
  int blocks_x = kNumCU / splits;
  if (blocks_x < 1) blocks_x = 1;
  if (blocks_x > groups) blocks_x = groups;
  const size_t lds = (size_t)8 * MT * 16 * (4 * G + 1) * sizeof(f32x4);
  static bool attr_set = false;
  if (lds > 64 * 1024 && !attr_set) {
    RAI_HIP_TRY(hipFuncSetAttribute((const void *)k_linear_bf16_mfma_stream<MT, KS, G, FRAG>,
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attr_set = true;
  }
  float *partial = splits > 1 ? (float *)a.splitk_ws : nullptr;
  // K split: the block that finishes a group last sums the partial products and runs the epilogue itself (no second
  // launch) when the tickets reach and the partial rows are 16-byte aligned; RAI_HIP_NO_FUSED_SPLITK=1 keeps the
  // separate summing pass (the tests compare the two: same bits).
  int *tickets = nullptr;
  if (splits > 1 && groups <= kSplitTickets && a.N % 4 == 0 && ((uintptr_t)partial & 15) == 0 && !getenv("RAI_HIP_NO_FUSED_SPLITK")) {
    int dev = -1;
    if (linear_device(a, &dev) == RAI_OK) tickets = splitk_tickets_of(dev);
  }
  hipLaunchKernelGGL((k_linear_bf16_mfma_stream<MT, KS, G, FRAG>), dim3(blocks_x, splits), dim3(512), lds, st, a, tiles,
                     partial, tickets);
  RAI_TRY(launch_check("linear_bf16_mfma_stream"));
  if (splits > 1 && !tickets) {
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

// True when the small-M streaming kernel can apply the RMSNorm of the activation rows itself.
bool linear_mfma_fuses_norm(int M, int K, int ln_kind) {
  // read per call (three getenv are nothing next to a launch): tests force the fallback kernels within one process
  const bool off = getenv("RAI_HIP_NO_MFMA_STREAM") != nullptr || getenv("RAI_HIP_NO_MFMA_SKINNY") != nullptr ||
                   getenv("RAI_HIP_NO_FUSED_NORM") != nullptr;
  if (off || (ln_kind != 1 && ln_kind != 2) || M <= 8 || M > 64 || K % 32) return false;
  return K <= (M <= 32 ? 8 * 8 * 32 : 8 * 4 * 32);   // one block's K span: no split over blocks
}

// Split K when the tile count alone cannot fill the GPU and a workspace was provided.
static int tile_splits(const LinearArgs &a) {
  const int tiles = ((a.M + 127) / 128) * ((a.N + 127) / 128);
  int splits = 1;
  if (a.force_splits > 0) {
    const int kt = a.K / 32;
    int s = a.force_splits < kt ? a.force_splits : kt;
    while (s > 1 && (!a.splitk_ws || (size_t)s * a.M * a.N * sizeof(float) > a.splitk_ws_bytes)) --s;
    return s < 1 ? 1 : s;
  }
  if (a.splitk_ws && tiles < kNumCU) {
    // Cost model in units of one K tile of one block: blocks go round-robin over the CUs, a CU holds up to three,
    // n co-resident blocks share a CU at a combined rate of 0.5 / 0.85 / 1 (one block alone cannot hide its own
    // barriers and memory latency), each block pays ~8 units of prologue + epilogue, and every split adds a pass over
    // the f32 partial sums (~7 units at 512 x 2560).  Measured at 512 x 2560 x 12800: 3, 4, 6, 9, 12 splits give
    // 6.69, 6.64, 6.28, 6.44, 6.79 ms per 32-layer prefill, the order this model predicts.
    const int kt = a.K / 32;
    float best = 0.f;
    for (int s = 1; s <= 12; ++s) {
      if (s > 1 && (kt / s < 8 || (size_t)s * a.M * a.N * sizeof(float) > a.splitk_ws_bytes)) break;
      const float per_block = (float)((kt + s - 1) / s) + 8.f;
      int left = (tiles * s + kNumCU - 1) / kNumCU;   // blocks on the busiest CU
      float cost = (s > 1 ? 7.f * s : 0.f) * ((float)a.M * a.N / (512.f * 2560.f));
      while (left > 0) {
        const int n = left < 3 ? left : 3;
        cost += n * per_block / (n == 1 ? 0.5f : n == 2 ? 0.85f : 1.f);
        left -= n;
      }
      if (s == 1 || cost < best) { best = cost; splits = s; }
    }
  }
  return splits;
}

bool linear_fuses_post_norm(const LinearArgs &a) {
  // the tile kernels serve more than 64 rows; their split-K pass is the one that can normalise
  // (RAI_HIP_NO_POST_NORM: run the norm as its own launch, for comparison)
  const char *off = getenv("RAI_HIP_NO_POST_NORM");   // read per call: the test switches it within one process
  if (off && *off) return false;
  return a.M > 64 && post_norm_fits(a) && tile_splits(a) > 1;
}

static bool no_k64() {   // read per call: tests compare both forms in one process
  const char *e = getenv("RAI_HIP_NO_K64");
  return e && *e && *e != '0';
}

int launch_linear_bf16_mfma(hipStream_t st, const LinearArgs &a) {
  RAI_REQUIRE(a.M > 0 && a.N > 0 && a.K > 0, RAI_ERR_BAD_SHAPE, "linear: empty problem %dx%dx%d", a.M, a.N, a.K);
  RAI_REQUIRE(a.A && a.W && a.out1, RAI_ERR_BAD_ARG, "linear: null operand");
  RAI_REQUIRE(a.n_split >= 0 && a.n_split <= a.N && (a.n_split == a.N || a.out2), RAI_ERR_BAD_ARG,
              "linear: bad output split");
  RAI_REQUIRE(a.ln_kind < 0 || linear_mfma_fuses_norm(a.M, a.K, a.ln_kind), RAI_ERR_UNSUPPORTED,
              "linear: fused norm needs M <= 8, or an RMS norm with M <= 64 and K within one block's span");
  if (a.glu) RAI_REQUIRE(a.N % 8 == 0 && !a.residual && a.n_split == a.N && a.act >= 0, RAI_ERR_BAD_ARG,
                         "linear mfma: bad gated-MLP arguments");
  RAI_REQUIRE(a.K % 32 == 0, RAI_ERR_UNSUPPORTED, "linear mfma: K=%d must be a multiple of 32", a.K);
  RAI_REQUIRE(a.lda % 8 == 0 && a.ldw % 8 == 0 && (uintptr_t)a.A % 16 == 0 && (uintptr_t)a.W % 16 == 0,
              RAI_ERR_BAD_STRIDE, "linear mfma: operands must be 16-byte aligned with row strides multiple of 8");
  const bool no_skinny = getenv("RAI_HIP_NO_MFMA_SKINNY") != nullptr;
  const bool no_stream = getenv("RAI_HIP_NO_MFMA_STREAM") != nullptr;
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
  const int tiles = ((a.M + 127) / 128) * ((a.N + 127) / 128);
  const int splits = tile_splits(a);
  // Tile choice.  The LDS-DMA kernels stream K tiles straight into LDS; the 256x128 tile halves the
  // L2 -> LDS traffic per flop for one operand and is used once there are enough tiles of that size
  // to give every CU two; smaller products keep the 128x128 tile (three blocks per CU).
  // RAI_HIP_GEMM_TILE = "128x128" | "128x128k64" | "256x128" | "256x192" | "256x256" | "256x256x8w" | "256x256x8wk64" |
  // "streamk" | "streamk64" | "classic" overrides (tuning aid; a form that does not apply to the shape is an error).
  const char *knob = getenv("RAI_HIP_GEMM_TILE");
  if (knob) {
    if (!strcmp(knob, "128x128")) return launch_cfg_dma<128, 128, 3, 2>(st, a, splits);
    if (!strcmp(knob, "256x128")) return launch_cfg_dma<256, 128, 3, 2>(st, a, splits);
    if (!strcmp(knob, "256x256")) return launch_cfg_dma<256, 256, 4, 2>(st, a, splits);
    if (!strcmp(knob, "classic")) return launch_cfg<128, 128, 32>(st, a, splits);
    if (!strcmp(knob, "256x256x8w")) return launch_cfg_dma<256, 256, 4, 2, 4>(st, a, splits);
    if (!strcmp(knob, "128x128k64")) {
      RAI_REQUIRE(a.K % 64 == 0, RAI_ERR_UNSUPPORTED, "linear: RAI_HIP_GEMM_TILE=%s needs K %% 64 == 0 (%dx%dx%d)", knob, a.M, a.N, a.K);
      return launch_cfg_dma<128, 128, 2, 0, 2>(st, a, splits);
    }
    if (!strcmp(knob, "256x192")) {
      RAI_REQUIRE(a.K % 64 == 0, RAI_ERR_UNSUPPORTED, "linear: RAI_HIP_GEMM_TILE=%s needs K %% 64 == 0 (%dx%dx%d)", knob, a.M, a.N, a.K);
      return launch_cfg_dma<256, 192, 2, 0, 2, 4>(st, a, splits);
    }
    if (!strcmp(knob, "256x256x8wk64")) {
      RAI_REQUIRE(splits == 1 && a.K % 64 == 0, RAI_ERR_UNSUPPORTED,
                  "linear: RAI_HIP_GEMM_TILE=256x256x8wk64 needs K %% 64 == 0 and no K split (%dx%dx%d)", a.M, a.N, a.K);
      return launch_cfg_dma<256, 256, 2, 0, 4>(st, a, splits);
    }
    if (!strcmp(knob, "streamk") || !strcmp(knob, "streamk64")) {
      const int bk = knob[7] ? 64 : 32;
      StreamKPlan plan;
      RAI_REQUIRE(splits == 1 && streamk_applies(a, bk, &plan, true), RAI_ERR_UNSUPPORTED,
                  "linear: RAI_HIP_GEMM_TILE=%s does not apply to %dx%dx%d", knob, a.M, a.N, a.K);
      return bk == 64 ? launch_streamk<2>(st, a, plan) : launch_streamk<4>(st, a, plan);
    }
  }
  const int big_tiles = ((a.M + 255) / 256) * ((a.N + 127) / 128);
  const int huge_tiles = ((a.M + 255) / 256) * ((a.N + 255) / 256);
  // 256x256 in its eight-wave form (one block per CU, 4 LDS stages, two waves per SIMD) once its tiles cover a good
  // half of the CUs: the tile with the most flops per byte drawn from L2, which is what bounds these kernels.
  // Measured against the smaller tiles: 16384 x 8960 x 1536 845 against 736 TFLOP/s, 16384 x 2048 x 1536 983 against
  // 834, 4096 x 10240 x 2560 896 against 789, 4096 x 2560 x 10240 (160 tiles) 837 against 650, 512 x 17920 x 2560
  // (140 tiles) 689 against 621; with 128 tiles or fewer the smaller tiles win (4096 x 2048 x 2048: 618 against 760).
  // The four-wave 256x256 form is 3-9 % behind the eight-wave one everywhere.
  if (splits == 1 && 32 * huge_tiles >= 17 * kNumCU) {
    // K tiles of 64 (whole 128-byte lines per request) where K allows; RAI_HIP_NO_K64 keeps the tiles of 32
    const bool k64 = a.K % 64 == 0 && !no_k64();
    StreamKPlan plan;
    const int tiles_192 = ((a.M + 255) / 256) * ((a.N + 191) / 192);
    const int rounds_192 = (tiles_192 + kNumCU - 1) / kNumCU;
    if (streamk_applies(a, k64 ? 64 : 32, &plan)) {
      // Whole rounds of 256 x 192 tiles against stream-K over 256 x 256 ones, in us per tile from the two kernels'
      // measured times (K = 1536 and 8960, all CUs busy): short K makes the exchange of the shares expensive next
      // to the tiles themselves (16384 x 1536 x 1536: 512 tiles of 256 x 192 in 80 us, stream-K over 384 in 90 us;
      // at K = 8960 stream-K wins, 433 against 456 us).
      const float st64 = (float)(a.K / 64);
      const float t256 = 5.8f + 1.69f * st64, t192 = 1.1f + 1.62f * st64;
      const float est_sk = (float)huge_tiles / kNumCU * t256 + (plan.k.max_parts <= 2 ? 18.f : 39.f);
      if (k64 && rounds_192 * t192 < 0.95f * est_sk) return launch_cfg_dma<256, 192, 2, 0, 2, 4>(st, a, splits);
      return k64 ? launch_streamk<2>(st, a, plan) : launch_streamk<4>(st, a, plan);
    }
    // 256 x 192 (eight waves as 4 x 2, 64 x 96 each) where its tiles need no more rounds over the CUs than the
    // 256 x 256 ones: the same round then holds three quarters of the work per CU, spread over more of them
    // (512 x 17920 x 2560 with cold weights: 188 tiles in 64.7 us against 140 tiles in 71.2 us)
    if (k64 && rounds_192 <= (huge_tiles + kNumCU - 1) / kNumCU)
      return launch_cfg_dma<256, 192, 2, 0, 2, 4>(st, a, splits);
    return k64 ? launch_cfg_dma<256, 256, 2, 0, 4>(st, a, splits) : launch_cfg_dma<256, 256, 4, 2, 4>(st, a, splits);
  }
  if (splits == 1 && big_tiles >= 2 * kNumCU) return launch_cfg_dma<256, 128, 3, 2>(st, a, splits);
  // 128 x 128 with two stages of K 64 (two blocks per CU) where K allows: 12-22 % over three stages of 32 on the
  // prefill shapes with cold weights (512 x 10240 x 2560: 66 -> 55 us, 2048^3: 33 -> 26 us)
  if (a.K % 64 == 0 && !no_k64()) return launch_cfg_dma<128, 128, 2, 0, 2>(st, a, splits);
  return launch_cfg_dma<128, 128, 3, 2>(st, a, splits);
}

}  // namespace rai
