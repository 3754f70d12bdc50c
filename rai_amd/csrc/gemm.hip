// Dense contractions.
//   (the bf16 MFMA tile kernel lives in gemm_mfma.hip)
//   k_linear_bf16_skinny weight-streaming kernel for M <= 8 rows (decode): each wave
//                        streams whole weight rows with 16-byte loads; HBM-bound.
//   k_linear_f32         f32 NT tile kernel (FMA) with the same epilogue.
//   k_matmul_generic     any strides / batch broadcast, f32 or f64 accumulate.
//
// Reference semantics: rai-core/src/backend/candle.rs:327-443 (MatMul, stride rule),
// rai-core/src/shape.rs:130-160 (batch broadcast), rai-nn/src/linear.rs:59-69.
#include <cstdlib>

#include "gemm.h"

namespace rai {


// ============================================================ bf16 skinny (decode) kernel
// M <= MROWS rows of A.  Each wave owns R consecutive weight rows at a time and
// streams them with one 16-byte non-temporal load per lane per 512-element K
// chunk; the (optionally normalised) activations live in LDS as bf16 and the
// products are formed with v_dot2_f32_bf16 (two bf16 products per lane-op,
// accumulated in f32).
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

// acc + dot(a[0..8), b[0..8)) over eight bf16 pairs packed in two 16-byte words.
// The vector elements are named explicitly: indexing an ext_vector with a loop
// variable inside __builtin_bit_cast made hipcc read element 0 four times.
__device__ __forceinline__ float dot2_bf16(uint32_t a, uint32_t b, float c) {
  bf16x2 p, q;
  __builtin_memcpy(&p, &a, 4);
  __builtin_memcpy(&q, &b, 4);
  return __builtin_amdgcn_fdot2_f32_bf16(p, q, c, false);
}
__device__ __forceinline__ float dot8_bf16(u32x4 a, u32x4 b, float c) {
  c = dot2_bf16(a.x, b.x, c);
  c = dot2_bf16(a.y, b.y, c);
  c = dot2_bf16(a.z, b.z, c);
  return dot2_bf16(a.w, b.w, c);
}

// Every wave owns `rows_per_wave` consecutive weight rows (so all waves stream
// the same number of bytes and are co-resident: no tail), R rows at a time, with
// U 16-byte loads per row in flight per lane.
template <int MROWS, int R, int U, int NWV>
__global__ void __launch_bounds__(NWV * 64) k_linear_bf16_skinny(LinearArgs a, int rows_per_wave) {
  constexpr int NT = NWV * 64;
  extern __shared__ __attribute__((aligned(16))) uint16_t xs[];  // [MROWS][K]
  __shared__ float red[2 * NWV];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint16_t *A = (const uint16_t *)a.A;
  const uint16_t *W = (const uint16_t *)a.W;
  // With a second product (M == 1) the K axis is the first product's K followed by the second's: position k < K1 is
  // column k of (A, W), position k >= K1 column k - K1 of (A2, W2); a 16-byte chunk never straddles (K1 % 8 == 0).
  const int K1 = a.K, K = a.K + a.K2;
  const uint16_t *A2 = a.K2 ? (const uint16_t *)a.A2 - K1 : nullptr;   // indexed by the position on the joint axis
  const uint16_t *W2 = a.K2 ? (const uint16_t *)a.W2 - K1 : nullptr;
  auto x_at = [&](const uint16_t *row, int k) { return k < K1 ? row + k : A2 + k; };
  auto w_at = [&](int n, int k) { return k < K1 ? W + (int64_t)n * a.ldw + k : W2 + (int64_t)n * a.ldw2 + k; };

  // Loads return in issue order: the activation rows (L2-resident) are requested
  // first, the first set of weight loads right behind them, so the staging into
  // LDS completes while the weights are still in flight.
  constexpr int XCH = 8;  // staged 16-byte chunks per thread per row that are prefetched in registers
  const int n_begin = (blockIdx.x * NWV + wave) * rows_per_wave;
  const int n_end = n_begin + rows_per_wave < a.N ? n_begin + rows_per_wave : a.N;
  u32x4 xpre[XCH];
#pragma unroll
  for (int i = 0; i < XCH; ++i) {
    const int k = (tid + i * NT) * 8;
    xpre[i] = k < K ? *reinterpret_cast<const u32x4 *>(x_at(A, k)) : u32x4{0u, 0u, 0u, 0u};
  }
  u32x4 wv[U][R];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int k = lane * 8 + u * 512;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      int n = n_begin + r < n_end ? n_begin + r : n_end - 1;
      if (k < K && n_begin < a.N) wv[u][r] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(w_at(n, k)));
      else wv[u][r] = u32x4{0u, 0u, 0u, 0u};
    }
  }

  // ---- stage activations, optionally normalising each row over K
  for (int m = 0; m < MROWS; ++m) {
    if (m >= a.M) break;
    const uint16_t *xr = A + (int64_t)m * a.lda;
    uint16_t *xd = xs + m * K;
    if (m == 0) {
#pragma unroll
      for (int i = 0; i < XCH; ++i) {
        const int k = (tid + i * NT) * 8;
        if (k < K) *reinterpret_cast<u32x4 *>(xd + k) = xpre[i];
      }
      for (int k = (tid + XCH * NT) * 8; k < K; k += NT * 8)
        *reinterpret_cast<u32x4 *>(xd + k) = *reinterpret_cast<const u32x4 *>(x_at(xr, k));
    } else {
      for (int k = tid * 8; k < K; k += NT * 8)
        *reinterpret_cast<u32x4 *>(xd + k) = *reinterpret_cast<const u32x4 *>(xr + k);
    }
    if (a.ln_kind >= 0) {
      __syncthreads();
      float s = 0.f;
      for (int k = tid; k < K; k += NT) {
        float v = bf16_bits_to_f32(xd[k]);
        s += a.ln_kind == 0 ? v : v * v;
      }
      s = wave_sum(s);
      if (lane == 0) red[wave] = s;
      __syncthreads();
      s = 0.f;
#pragma unroll
      for (int w = 0; w < NWV; ++w) s += red[w];
      float mean = 0.f, scale;
      if (a.ln_kind == 0) {
        mean = s / (float)K;
        float q = 0.f;
        for (int k = tid; k < K; k += NT) { float d = bf16_bits_to_f32(xd[k]) - mean; q += d * d; }
        q = wave_sum(q);
        if (lane == 0) red[NWV + wave] = q;
        __syncthreads();
        q = 0.f;
#pragma unroll
        for (int w = 0; w < NWV; ++w) q += red[NWV + w];
        scale = 1.0f / sqrtf(q / (float)K + a.ln_eps);
      } else {
        scale = 1.0f / sqrtf(s / (float)K + a.ln_eps);
      }
      const uint16_t *lw = (const uint16_t *)a.ln_w, *lb = (const uint16_t *)a.ln_b;
      for (int k = tid; k < K; k += NT) {
        float y = (bf16_bits_to_f32(xd[k]) - mean) * scale;
        float wv = bf16_bits_to_f32(lw[k]);
        y *= a.ln_kind == 2 ? 1.0f + wv : wv;
        if (lb) y += bf16_bits_to_f32(lb[k]);
        // the reference materialises the normalised activations in bf16 too
        xd[k] = f32_to_bf16_bits(y);
      }
      __syncthreads();
    }
  }
  __syncthreads();

  const uint16_t *bias = (const uint16_t *)a.bias;
  const uint16_t *bias2 = (const uint16_t *)a.bias2;
  const uint16_t *res = (const uint16_t *)a.residual;
  // Flattened (row group, K step) loop in rotated form: multiply the set in
  // registers, then fetch the next set.
  if (n_begin >= n_end) return;
  float acc[R][MROWS];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int m = 0; m < MROWS; ++m) acc[r][m] = 0.f;
  int n_base = n_begin, k0 = lane * 8;
  while (true) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = k0 + u * 512;
      if (k < K) {
#pragma unroll
        for (int m = 0; m < MROWS; ++m) {
          const u32x4 xv = *reinterpret_cast<const u32x4 *>(xs + m * K + k);
#pragma unroll
          for (int r = 0; r < R; ++r) acc[r][m] = dot8_bf16(wv[u][r], xv, acc[r][m]);
        }
      }
    }
    k0 += 64 * 8 * U;
    const bool row_done = k0 >= K;
    const int n_cur = n_base;
    if (row_done) {
      n_base += R;
      k0 = lane * 8;
    }
    const bool more = n_base < n_end;
    if (more) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int k = k0 + u * 512;
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const int n = n_base + r < n_end ? n_base + r : n_end - 1;  // tail rows re-read the last row; never stored
          if (k < K) wv[u][r] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(w_at(n, k)));
        }
      }
    }
    if (row_done) {
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int m = 0; m < MROWS; ++m) acc[r][m] = wave_sum(acc[r][m]);
      if (lane == 0 && a.glu) {
        if constexpr (R % 2 == 0) {
#pragma unroll
          for (int r = 0; r < R; r += 2) {
            const int n = n_cur + r;
            if (n + 1 >= n_end) break;
            const float bg = bias ? bf16_bits_to_f32(bias[n]) : 0.f, bu = bias ? bf16_bits_to_f32(bias[n + 1]) : 0.f;
#pragma unroll
            for (int m = 0; m < MROWS; ++m) {
              if (m >= a.M) break;
              ((uint16_t *)a.out1)[(int64_t)m * a.ld1 + (n >> 1)] =
                  f32_to_bf16_bits(glu_bf16(a.act, acc[r][m] + bg, acc[r + 1][m] + bu));
            }
          }
        }
      } else if (lane == 0) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const int n = n_cur + r;
          if (n >= n_end) break;
          const float bv = (bias ? bf16_bits_to_f32(bias[n]) : 0.f) + (bias2 ? bf16_bits_to_f32(bias2[n]) : 0.f);
          const bool do_act = a.act >= 0 && n >= a.act_from;
          uint16_t *dst;
          int64_t ld;
          int col;
          if (n < a.n_split) { dst = (uint16_t *)a.out1; ld = a.ld1; col = n; }
          else { dst = (uint16_t *)a.out2; ld = a.ld2; col = n - a.n_split; }
#pragma unroll
          for (int m = 0; m < MROWS; ++m) {
            if (m >= a.M) break;
            float v = acc[r][m] + bv;
            if (do_act) v = act_eval(a.act, v);
            if (res) v += bf16_bits_to_f32(res[(int64_t)m * a.ldr + n]);
            dst[(int64_t)m * ld + col] = f32_to_bf16_bits(v);
          }
        }
      }
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int m = 0; m < MROWS; ++m) acc[r][m] = 0.f;
    }
    if (!more) break;
  }
}

// ============================================================ bf16 GEMV with the activation vector in registers (M == 1)
// One wave streams R weight rows at a time.  Lane l owns the K positions
// l*8 + 512*u (u < KC), the same positions of the activation vector, which it
// keeps in registers as packed bf16 pairs: no LDS, no block barriers, waves are
// independent.  The weight loads of the first row group are issued before the
// activation vector is fetched and normalised, so the fused LayerNorm/RMSNorm
// prologue overlaps the first HBM round trip.
template <int KC, int R>
__device__ __forceinline__ void gemv_reg_rows(const LinearArgs &a, int n_begin, int rows_per_wave) {
  const int lane = threadIdx.x & 63;
  const int K = a.K;
  const uint16_t *W = (const uint16_t *)a.W;
  if (n_begin >= a.N) return;
  const int n_end = n_begin + rows_per_wave < a.N ? n_begin + rows_per_wave : a.N;

  u32x4 wv[R][KC];
  auto load_group = [&](int n_base) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int n = n_base + r < n_end ? n_base + r : n_end - 1;
      const uint16_t *wr = W + (int64_t)n * a.ldw + lane * 8;
#pragma unroll
      for (int u = 0; u < KC; ++u) {
        if (lane * 8 + u * 512 < K) wv[r][u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(wr + u * 512));
        else wv[r][u] = u32x4{0u, 0u, 0u, 0u};
      }
    }
  };
  // Loads return in issue order, so the small L2-resident vectors (activations,
  // norm parameters) are requested first and the weight stream right after: the
  // norm prologue then runs while the weights are still in flight.
  u32x4 xv[KC], lwv[KC], lbv[KC];
  {
    const uint16_t *xr = (const uint16_t *)a.A + lane * 8;
    const uint16_t *lw = a.ln_kind >= 0 ? (const uint16_t *)a.ln_w + lane * 8 : nullptr;
    const uint16_t *lb = (a.ln_kind >= 0 && a.ln_b) ? (const uint16_t *)a.ln_b + lane * 8 : nullptr;
#pragma unroll
    for (int u = 0; u < KC; ++u) {
      const bool in = lane * 8 + u * 512 < K;
      xv[u] = in ? *reinterpret_cast<const u32x4 *>(xr + u * 512) : u32x4{0u, 0u, 0u, 0u};
      lwv[u] = (in && lw) ? *reinterpret_cast<const u32x4 *>(lw + u * 512) : u32x4{0u, 0u, 0u, 0u};
      lbv[u] = (in && lb) ? *reinterpret_cast<const u32x4 *>(lb + u * 512) : u32x4{0u, 0u, 0u, 0u};
    }
  }
  load_group(n_begin);

  // ---- fused LayerNorm / RMSNorm of the activation vector, kept as packed bf16 in registers.
  // Sum and sum of squares come from v_dot2_f32_bf16 on the packed pairs (exact
  // products, f32 accumulation); the variance is E[x^2] - mean^2.
  if (a.ln_kind >= 0) {
    const uint32_t ones = 0x3f803f80u;  // (1.0bf16, 1.0bf16)
    float s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int u = 0; u < KC; ++u) {
      const uint32_t w4[4] = {xv[u].x, xv[u].y, xv[u].z, xv[u].w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        s1 = dot2_bf16(w4[j], ones, s1);
        s2 = dot2_bf16(w4[j], w4[j], s2);
      }
    }
    if (a.ln_kind == 0) s1 = wave_sum(s1);
    s2 = wave_sum(s2);
    float mean = 0.f, scale;
    if (a.ln_kind == 0) {
      mean = s1 / (float)K;
      float var = s2 / (float)K - mean * mean;
      var = var > 0.f ? var : 0.f;
      scale = 1.0f / sqrtf(var + a.ln_eps);
    } else {
      scale = 1.0f / sqrtf(s2 / (float)K + a.ln_eps);
    }
    const float shift = -mean * scale;
#pragma unroll
    for (int u = 0; u < KC; ++u) {
      if (lane * 8 + u * 512 < K) {
        const uint32_t xx[4] = {xv[u].x, xv[u].y, xv[u].z, xv[u].w};
        const uint32_t ww[4] = {lwv[u].x, lwv[u].y, lwv[u].z, lwv[u].w};
        const uint32_t bb[4] = {lbv[u].x, lbv[u].y, lbv[u].z, lbv[u].w};
        uint32_t o[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          float w0 = __uint_as_float(ww[j] << 16), w1 = __uint_as_float(ww[j] & 0xffff0000u);
          if (a.ln_kind == 2) { w0 += 1.0f; w1 += 1.0f; }
          // ((x - mean) * scale) * w + b
          const float y0 = fmaf(fmaf(__uint_as_float(xx[j] << 16), scale, shift), w0, __uint_as_float(bb[j] << 16));
          const float y1 = fmaf(fmaf(__uint_as_float(xx[j] & 0xffff0000u), scale, shift), w1,
                                __uint_as_float(bb[j] & 0xffff0000u));
          // the reference materialises the normalised activations in bf16 too
          o[j] = pack_bf16x2(y0, y1);
        }
        xv[u] = u32x4{o[0], o[1], o[2], o[3]};
      }
    }
  }

  const uint16_t *bias = (const uint16_t *)a.bias;
  const uint16_t *bias2 = (const uint16_t *)a.bias2;
  const uint16_t *res = (const uint16_t *)a.residual;
  for (int n_base = n_begin; n_base < n_end; n_base += R) {
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      acc[r] = 0.f;
#pragma unroll
      for (int u = 0; u < KC; ++u) acc[r] = dot8_bf16(wv[r][u], xv[u], acc[r]);
    }
    // the next group's loads go out before this group's reduction and stores
    if (n_base + R < n_end) load_group(n_base + R);
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = wave_sum(acc[r]);
    if (lane == 0 && a.glu) {
      if constexpr (R % 2 == 0) {
#pragma unroll
        for (int r = 0; r < R; r += 2) {
          const int n = n_base + r;
          if (n + 1 >= a.N || n >= n_end) break;
          const float bg = bias ? bf16_bits_to_f32(bias[n]) : 0.f, bu = bias ? bf16_bits_to_f32(bias[n + 1]) : 0.f;
          ((uint16_t *)a.out1)[n >> 1] = f32_to_bf16_bits(glu_bf16(a.act, acc[r] + bg, acc[r + 1] + bu));
        }
      }
    } else if (lane == 0) {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int n = n_base + r;
        if (n >= n_end) break;
        float v = acc[r] + (bias ? bf16_bits_to_f32(bias[n]) : 0.f) + (bias2 ? bf16_bits_to_f32(bias2[n]) : 0.f);
        if (a.act >= 0 && n >= a.act_from) v = act_eval(a.act, v);
        if (res) v += bf16_bits_to_f32(res[n]);
        if (n < a.n_split) ((uint16_t *)a.out1)[n] = f32_to_bf16_bits(v);
        else ((uint16_t *)a.out2)[n - a.n_split] = f32_to_bf16_bits(v);
      }
    }
  }
}

template <int KC, int R>
__global__ void __launch_bounds__(256) k_gemv_bf16_reg(LinearArgs a, int rows_per_wave) {
  gemv_reg_rows<KC, R>(a, (blockIdx.x * 4 + (threadIdx.x >> 6)) * rows_per_wave, rows_per_wave);
}

// Up to four Linears of one activation vector in one launch (the q, k, v projections and the first MLP Linear of a
// decoder block, each with its own weight, bias, activation and output): wave gw serves rows of the member whose
// wave range [wave_base[s], wave_base[s + 1]) holds it.  The fused norm is every member's.
template <int KC, int R>
__global__ void __launch_bounds__(256) k_gemv_bf16_reg_group(GemvGroupArgs g, int rows_per_wave) {
  const int gw = __builtin_amdgcn_readfirstlane(blockIdx.x * 4 + (threadIdx.x >> 6));
  if (gw >= g.wave_base[g.count]) return;
  int s = 0;
#pragma unroll
  for (int i = 1; i < kGemvGroupMax; ++i)
    if (i < g.count && gw >= g.wave_base[i]) s = i;
  LinearArgs a;
  a.A = g.x; a.lda = g.K;
  a.W = g.W[0]; a.ldw = g.ldw[0]; a.bias = g.bias[0]; a.out1 = g.out[0]; a.N = g.N[0]; a.act = g.act[0];
  int base = g.wave_base[0];
#pragma unroll
  for (int i = 1; i < kGemvGroupMax; ++i)
    if (s == i) { a.W = g.W[i]; a.ldw = g.ldw[i]; a.bias = g.bias[i]; a.out1 = g.out[i]; a.N = g.N[i]; a.act = g.act[i]; base = g.wave_base[i]; }
  a.bias2 = nullptr; a.residual = nullptr; a.ldr = 0; a.ld1 = a.N; a.out2 = nullptr; a.ld2 = 0;
  a.M = 1; a.K = g.K; a.n_split = a.N; a.act_from = 0; a.glu = 0;
  a.ln_w = g.ln_w; a.ln_b = g.ln_b; a.ln_eps = g.ln_eps; a.ln_kind = g.ln_kind;
  a.A2 = nullptr; a.W2 = nullptr; a.ldw2 = 0; a.K2 = 0;
  gemv_reg_rows<KC, R>(a, (gw - base) * rows_per_wave, rows_per_wave);
}

// ============================================================ f32 NT tile kernel
// 64x64 tile, BK=16, 256 threads each computing a 4x4 micro-tile with FMA.
__global__ void __launch_bounds__(256) k_linear_f32(LinearArgs a) {
  constexpr int BM = 64, BN = 64, BK = 16;
  __shared__ float As[BK][BM + 4];
  __shared__ float Bs[BK][BN + 4];
  const int tid = threadIdx.x;
  const int tiles_m = (a.M + BM - 1) / BM;
  const int tile_n = blockIdx.x / tiles_m, tile_m = blockIdx.x % tiles_m;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const float *A = (const float *)a.A;
  const float *W = (const float *)a.W;
  const int tx = tid & 15, ty = tid >> 4;  // 16 x 16 threads
  float acc[4][4] = {};
  const int lrow = tid >> 2, lk = (tid & 3) * 4;  // each thread loads 4 consecutive k of one row
  const bool vec_ok = (a.lda % 4 == 0) && (a.ldw % 4 == 0) && ((uintptr_t)A % 16 == 0) && ((uintptr_t)W % 16 == 0);
  for (int k0 = 0; k0 < a.K; k0 += BK) {
    float va[4] = {0.f, 0.f, 0.f, 0.f}, vb[4] = {0.f, 0.f, 0.f, 0.f};
    {
      int m = m0 + lrow, k = k0 + lk;
      if (m < a.M) {
        const float *p = A + (int64_t)m * a.lda + k;
        if (vec_ok && k + 3 < a.K) { float4 t = *reinterpret_cast<const float4 *>(p); va[0] = t.x; va[1] = t.y; va[2] = t.z; va[3] = t.w; }
        else { for (int j = 0; j < 4; ++j) if (k + j < a.K) va[j] = p[j]; }
      }
      int n = n0 + lrow;
      if (n < a.N) {
        const float *p = W + (int64_t)n * a.ldw + k;
        if (vec_ok && k + 3 < a.K) { float4 t = *reinterpret_cast<const float4 *>(p); vb[0] = t.x; vb[1] = t.y; vb[2] = t.z; vb[3] = t.w; }
        else { for (int j = 0; j < 4; ++j) if (k + j < a.K) vb[j] = p[j]; }
      }
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 4; ++j) { As[lk + j][lrow] = va[j]; Bs[lk + j][lrow] = vb[j]; }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < BK; ++k) {
      float4 av = *reinterpret_cast<const float4 *>(&As[k][ty * 4]);
      float4 bv = *reinterpret_cast<const float4 *>(&Bs[k][tx * 4]);
      float af[4] = {av.x, av.y, av.z, av.w}, bf[4] = {bv.x, bv.y, bv.z, bv.w};
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(af[i], bf[j], acc[i][j]);
    }
  }
  const float *bias = (const float *)a.bias;
  const float *bias2 = (const float *)a.bias2;
  const float *res = (const float *)a.residual;
  if (a.glu) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int m = m0 + ty * 4 + i;
      if (m >= a.M) continue;
#pragma unroll
      for (int j = 0; j < 4; j += 2) {
        int n = n0 + tx * 4 + j;
        if (n + 1 >= a.N) continue;
        float g = acc[i][j] + (bias ? bias[n] : 0.f), u = acc[i][j + 1] + (bias ? bias[n + 1] : 0.f);
        ((float *)a.out1)[(int64_t)m * a.ld1 + (n >> 1)] = act_eval(a.act, g) * u;
      }
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    int m = m0 + ty * 4 + i;
    if (m >= a.M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      int n = n0 + tx * 4 + j;
      if (n >= a.N) continue;
      float v = acc[i][j] + (bias ? bias[n] : 0.f) + (bias2 ? bias2[n] : 0.f);
      if (a.act >= 0 && n >= a.act_from) v = act_eval(a.act, v);
      if (res) v += res[(int64_t)m * a.ldr + n];
      if (n < a.n_split) ((float *)a.out1)[(int64_t)m * a.ld1 + n] = v;
      else ((float *)a.out2)[(int64_t)m * a.ld2 + (n - a.n_split)] = v;
    }
  }
}

// ============================================================ generic strided batched matmul
struct MatmulArgs {
  int64_t M, N, K;
  int64_t a_rs, a_cs, b_rs, b_cs;  // element strides of the last two dims
  int batch_rank;
  int64_t batch_shape[RAI_HIP_MAX_RANK];
  int64_t a_bs[RAI_HIP_MAX_RANK], b_bs[RAI_HIP_MAX_RANK];
};

template <typename T>
__global__ void __launch_bounds__(256) k_matmul_generic(T *out, const T *A, const T *B, MatmulArgs g) {
  typedef typename Scalar<T>::compute C;
  constexpr int BM = 64, BN = 64, BK = 16;
  __shared__ C As[BK][BM + 1];
  __shared__ C Bs[BK][BN + 1];
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  int64_t rem = blockIdx.z, aoff = 0, boff = 0;
  for (int d = g.batch_rank - 1; d >= 0; --d) {
    int64_t q = rem / g.batch_shape[d], i = rem - q * g.batch_shape[d];
    rem = q;
    aoff += i * g.a_bs[d];
    boff += i * g.b_bs[d];
  }
  A += aoff;
  B += boff;
  out += (int64_t)blockIdx.z * g.M * g.N;
  const int64_t m0 = (int64_t)blockIdx.y * BM, n0 = (int64_t)blockIdx.x * BN;
  C acc[4][4] = {};
  for (int64_t k0 = 0; k0 < g.K; k0 += BK) {
    // 64x16 elements of A and of B: 4 per thread each
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int e = tid + i * 256;
      int kk, mm;
      // pick the traversal that makes consecutive threads touch consecutive memory
      if (g.a_cs == 1) { kk = e & 15; mm = e >> 4; } else { mm = e & 63; kk = e >> 6; }
      int64_t m = m0 + mm, k = k0 + kk;
      As[kk][mm] = (m < g.M && k < g.K) ? Scalar<T>::load(A + m * g.a_rs + k * g.a_cs) : C(0);
      int nn;
      if (g.b_cs == 1) { nn = e & 63; kk = e >> 6; } else { kk = e & 15; nn = e >> 4; }
      int64_t n = n0 + nn;
      k = k0 + kk;
      Bs[kk][nn] = (n < g.N && k < g.K) ? Scalar<T>::load(B + k * g.b_rs + n * g.b_cs) : C(0);
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < BK; ++k) {
      C af[4], bf[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) { af[i] = As[k][ty * 4 + i]; bf[i] = Bs[k][tx * 4 + i]; }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] += af[i] * bf[j];
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    int64_t m = m0 + ty * 4 + i;
    if (m >= g.M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      int64_t n = n0 + tx * 4 + j;
      if (n < g.N) Scalar<T>::store(out + m * g.N + n, acc[i][j]);
    }
  }
}

// ============================================================ launchers
static int check_linear_args(const LinearArgs &a, size_t es) {
  RAI_REQUIRE(a.M > 0 && a.N > 0 && a.K > 0, RAI_ERR_BAD_SHAPE, "linear: empty problem %dx%dx%d", a.M, a.N, a.K);
  RAI_REQUIRE(a.A && a.W && a.out1, RAI_ERR_BAD_ARG, "linear: null operand");
  RAI_REQUIRE(a.n_split >= 0 && a.n_split <= a.N && (a.n_split == a.N || a.out2), RAI_ERR_BAD_ARG,
              "linear: bad output split");
  const int v = (int)(16 / es);
  RAI_REQUIRE(a.K % v == 0 && a.lda % v == 0 && a.ldw % v == 0, RAI_ERR_BAD_STRIDE,
              "linear: K and row strides must be multiples of %d elements", v);
  RAI_REQUIRE((uintptr_t)a.A % 16 == 0 && (uintptr_t)a.W % 16 == 0, RAI_ERR_BAD_STRIDE,
              "linear: operands must be 16-byte aligned");
  return RAI_OK;
}

template <int MROWS, int R, int U, int NWV = 4>
static int launch_skinny_cfg(hipStream_t st, const LinearArgs &a, int rows_per_wave) {
  const size_t lds = (size_t)MROWS * (a.K + a.K2) * sizeof(uint16_t);
  static size_t attr_bytes = 0;
  if (lds > 64 * 1024 && lds > attr_bytes) {
    RAI_HIP_TRY(hipFuncSetAttribute((const void *)k_linear_bf16_skinny<MROWS, R, U, NWV>,
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attr_bytes = lds;
  }
  const int waves = (a.N + rows_per_wave - 1) / rows_per_wave;
  const int blocks = (waves + NWV - 1) / NWV;
  hipLaunchKernelGGL((k_linear_bf16_skinny<MROWS, R, U, NWV>), dim3(blocks), dim3(NWV * 64), lds, st, a, rows_per_wave);
  return launch_check("linear_bf16_skinny");
}

template <int KC, int R>
static int launch_gemv_reg(hipStream_t st, const LinearArgs &a, int waves_per_cu, int rows_per_wave = 0) {
  // every wave co-resident (waves_per_cu follows the kernel's register budget),
  // each with a whole number of R-row groups
  int rpw = rows_per_wave;
  if (rpw <= 0) {
    const int target_waves = kNumCU * waves_per_cu;
    rpw = (a.N + target_waves - 1) / target_waves;
    rpw = ((rpw + R - 1) / R) * R;
  }
  const int waves = (a.N + rpw - 1) / rpw;
  hipLaunchKernelGGL((k_gemv_bf16_reg<KC, R>), dim3((waves + 3) / 4), dim3(256), 0, st, a, rpw);
  return launch_check("gemv_bf16_reg");
}

bool gemv_group_serves(int K, int count) { return count >= 1 && count <= kGemvGroupMax && K % 8 == 0 && K >= 8 && K <= 4096; }

int launch_gemv_group(hipStream_t st, GemvGroupArgs g) {
  RAI_REQUIRE(gemv_group_serves(g.K, g.count) && g.x && ((uintptr_t)g.x & 15) == 0, RAI_ERR_UNSUPPORTED, "linear group: K=%d x %d members not served",
              g.K, g.count);
  if (g.ln_kind >= 0) RAI_REQUIRE(g.ln_w && ((uintptr_t)g.ln_w & 15) == 0 && ((uintptr_t)g.ln_b & 15) == 0, RAI_ERR_BAD_STRIDE, "linear group: norm parameters");
  // short-lived waves, one or two groups of two rows each (what the single Linear of these widths takes);
  // RAI_HIP_GEMV_GROUP_ROWS overrides (tuning aid, read per launch)
  int total = 0;
  for (int i = 0; i < g.count; ++i) total += g.N[i];
  int rpw = total >= 8192 ? 8 : 2;
  if (const char *e = getenv("RAI_HIP_GEMV_GROUP_ROWS")) {
    const int v = atoi(e);
    if (v >= 2 && v <= 64 && v % 2 == 0) rpw = v;
  }
  int waves = 0;
  for (int i = 0; i < g.count; ++i) {
    RAI_REQUIRE(g.W[i] && g.out[i] && g.N[i] >= 1 && g.ldw[i] % 8 == 0 && ((uintptr_t)g.W[i] & 15) == 0, RAI_ERR_BAD_STRIDE,
                "linear group: member %d not served", i);
    g.wave_base[i] = waves;
    waves += (g.N[i] + rpw - 1) / rpw;
  }
  g.wave_base[g.count] = waves;
  const dim3 grid((waves + 3) / 4), block(256);
  if (g.K <= 2048) hipLaunchKernelGGL((k_gemv_bf16_reg_group<4, 2>), grid, block, 0, st, g, rpw);
  else if (g.K <= 2560) hipLaunchKernelGGL((k_gemv_bf16_reg_group<5, 2>), grid, block, 0, st, g, rpw);
  else hipLaunchKernelGGL((k_gemv_bf16_reg_group<8, 2>), grid, block, 0, st, g, rpw);
  return launch_check("gemv_bf16_reg_group");
}

int launch_linear_bf16_skinny(hipStream_t st, const LinearArgs &a) {
  RAI_TRY(check_linear_args(a, 2));
  RAI_REQUIRE(a.M <= 8, RAI_ERR_BAD_SHAPE, "linear skinny: M=%d > 8", a.M);
  RAI_REQUIRE((size_t)a.M * (a.K + a.K2) * 2 <= 150 * 1024, RAI_ERR_UNSUPPORTED, "linear skinny: activations exceed LDS");
  const bool dual = a.K2 > 0;
  if (dual)
    RAI_REQUIRE(a.M == 1 && a.A2 && a.W2 && a.K2 % 8 == 0 && a.ldw2 % 8 == 0 && (uintptr_t)a.A2 % 16 == 0 && (uintptr_t)a.W2 % 16 == 0 &&
                    a.ln_kind < 0 && !a.glu,
                RAI_ERR_UNSUPPORTED, "linear: second product not served (one row, no norm, no gate)");
  if (a.glu) RAI_REQUIRE(a.N % 2 == 0 && !a.residual && a.n_split == a.N && a.act >= 0, RAI_ERR_BAD_ARG,
                         "linear: bad gated-MLP arguments");
  if (a.M == 1 && a.K <= 4096 && a.N >= 1024 && !dual) {
    // activation vector in registers (at most 8 chunks of 16 bytes per lane)
    if (a.K <= 2048) return launch_gemv_reg<4, 4>(st, a, 8);
    if (a.K <= 2560) {
      static const char *gk = getenv("RAI_HIP_GEMV");  // tuning aid: "R,rows_per_wave"
      if (gk) {
        int r = 0, rp = 0;
        if (sscanf(gk, "%d,%d", &r, &rp) == 2 && rp > 0) {
          if (r == 4) return launch_gemv_reg<5, 4>(st, a, 0, rp);
          if (r == 2) return launch_gemv_reg<5, 2>(st, a, 0, rp);
        }
      }
      return launch_gemv_reg<5, 2>(st, a, 0, a.N >= 8192 ? 4 : 2);  // short-lived waves, two row groups each
    }
    return launch_gemv_reg<8, 2>(st, a, 8);
  }
  // About 10 waves per CU, all co-resident, each with the same number of rows.
  const int target_waves = kNumCU * 10;
  int rpw = (a.N + target_waves - 1) / target_waves;
  if (a.glu) {  // gate/up row pairs must stay inside one row group
    RAI_REQUIRE(a.N % 2 == 0 && !a.residual && a.n_split == a.N, RAI_ERR_BAD_ARG, "linear: bad gated-MLP arguments");
    rpw = rpw < 2 ? 2 : (rpw / 2) * 2;
    if (a.M == 1) return launch_skinny_cfg<1, 2, 8>(st, a, rpw);
    if (a.M == 2) return launch_skinny_cfg<2, 2, 8>(st, a, rpw);
    if (a.M <= 4) return launch_skinny_cfg<4, 2, 4>(st, a, rpw);
    return launch_skinny_cfg<8, 2, 4>(st, a, rpw);
  }
  if (a.M == 1) {
    static const char *knob = getenv("RAI_HIP_SKINNY");  // tuning aid: "R,NWV,rows_per_wave,U"
    if (knob) {
      int r = 0, nwv = 0, rp = 0, u = 0;
      if (sscanf(knob, "%d,%d,%d,%d", &r, &nwv, &rp, &u) == 4 && rp > 0) {
        if (r == 1 && nwv == 4 && u == 8) return launch_skinny_cfg<1, 1, 8, 4>(st, a, rp);
        if (r == 1 && nwv == 4 && u == 13) return launch_skinny_cfg<1, 1, 13, 4>(st, a, rp);
        if (r == 1 && nwv == 4 && u == 25) return launch_skinny_cfg<1, 1, 25, 4>(st, a, rp);
        if (r == 1 && nwv == 8 && u == 25) return launch_skinny_cfg<1, 1, 25, 8>(st, a, rp);
        if (r == 1 && nwv == 16 && u == 25) return launch_skinny_cfg<1, 1, 25, 16>(st, a, rp);
        if (r == 2 && nwv == 4 && u == 13) return launch_skinny_cfg<1, 2, 13, 4>(st, a, rp);
        if (r == 2 && nwv == 4 && u == 8) return launch_skinny_cfg<1, 2, 8, 4>(st, a, rp);
      }
    }
    // one row per wave with the whole row in flight when it fits the register budget
    if (a.N <= kNumCU * 16 && a.K + a.K2 <= 25 * 512) return launch_skinny_cfg<1, 1, 25>(st, a, 1);
    if (rpw >= 4) { rpw = (rpw / 4) * 4; return launch_skinny_cfg<1, 4, 5>(st, a, rpw); }
    if (rpw >= 2) { rpw = 2; return launch_skinny_cfg<1, 2, 8>(st, a, rpw); }
    return launch_skinny_cfg<1, 1, 8>(st, a, 1);
  }
  if (a.M == 2) {
    if (rpw >= 4) { rpw = (rpw / 4) * 4; return launch_skinny_cfg<2, 4, 4>(st, a, rpw); }
    if (rpw >= 2) return launch_skinny_cfg<2, 2, 8>(st, a, 2);
    return launch_skinny_cfg<2, 1, 8>(st, a, 1);
  }
  if (a.M <= 4) {
    if (rpw >= 2) { rpw = (rpw / 2) * 2; return launch_skinny_cfg<4, 2, 4>(st, a, rpw); }
    return launch_skinny_cfg<4, 1, 8>(st, a, 1);
  }
  if (rpw >= 2) { rpw = (rpw / 2) * 2; return launch_skinny_cfg<8, 2, 4>(st, a, rpw); }
  return launch_skinny_cfg<8, 1, 4>(st, a, 1);
}

int launch_linear_dual_row(hipStream_t st, int dev, const void *x1, int K1, const void *W1, int64_t ldw1, const void *bias1, const void *x2, int K2,
                           const void *W2, int64_t ldw2, const void *bias2, const void *residual, void *out, int N) {
  LinearArgs a = linear_args_default();
  a.dev = dev;
  a.A = x1; a.lda = K1; a.W = W1; a.ldw = ldw1; a.K = K1;
  a.A2 = x2; a.W2 = W2; a.ldw2 = ldw2; a.K2 = K2;
  a.bias = bias1; a.bias2 = bias2;
  a.residual = residual; a.ldr = N;
  a.out1 = out; a.ld1 = N;
  a.M = 1; a.N = N; a.n_split = N;
  return launch_linear_bf16_skinny(st, a);
}

int launch_linear_bf16(hipStream_t st, const LinearArgs &a) {
  if (a.M <= 8 && (size_t)a.M * a.K * 2 <= 150 * 1024) return launch_linear_bf16_skinny(st, a);
  return launch_linear_bf16_mfma(st, a);
}

// dst[N][K] = src[K][N]^T through a 64x64 LDS tile: both the reads (rows of src) and the
// writes (rows of dst) are contiguous runs of 64 elements.
template <typename T>
__global__ void __launch_bounds__(256) k_transpose_2d(T *dst, const T *src, int K, int N) {
  __shared__ T tile[64][64 + 2];
  const int n0 = blockIdx.x * 64, k0 = blockIdx.y * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int i = ty; i < 64; i += 4) {
    const int k = k0 + i, n = n0 + tx;
    if (k < K && n < N) tile[i][tx] = src[(int64_t)k * N + n];
  }
  __syncthreads();
  for (int i = ty; i < 64; i += 4) {
    const int n = n0 + i, k = k0 + tx;
    if (n < N && k < K) dst[(int64_t)n * K + k] = tile[tx][i];
  }
}

// The same transposition with 16-byte accesses on both sides (N, K multiples of 16 / sizeof(T), 16-byte aligned
// operands): a 64 x 64 tile is read as rows of 16-byte chunks, and every thread then gathers the 16 bytes of one
// output chunk (consecutive k for one n) from LDS.  The odd pitch in 32-bit words keeps the column gathers off a
// single bank.
template <typename T>
__global__ void __launch_bounds__(256) k_transpose_2d_vec(T *dst, const T *src, int K, int N) {
  constexpr int V = 16 / sizeof(T), CPR = 64 / V;      // elements per chunk, chunks per tile row
  constexpr int PITCH = sizeof(T) == 2 ? 66 : 65;      // 33 resp. 65 words per row
  struct alignas(16) Pack { T v[V]; };
  __shared__ T tile[64][PITCH];
  const int n0 = blockIdx.x * 64, k0 = blockIdx.y * 64;
  for (int c = threadIdx.x; c < 64 * CPR; c += 256) {
    const int i = c / CPR, j = (c % CPR) * V;
    const int k = k0 + i, n = n0 + j;
    if (k < K && n < N) {
      const Pack p = *reinterpret_cast<const Pack *>(src + (int64_t)k * N + n);
#pragma unroll
      for (int e = 0; e < V; ++e) tile[i][j + e] = p.v[e];
    }
  }
  __syncthreads();
  for (int c = threadIdx.x; c < 64 * CPR; c += 256) {
    const int i = c / CPR, j = (c % CPR) * V;            // output row n0 + i, k chunk at k0 + j
    const int n = n0 + i, k = k0 + j;
    if (n < N && k < K) {
      Pack p;
#pragma unroll
      for (int e = 0; e < V; ++e) p.v[e] = tile[j + e][i];
      *reinterpret_cast<Pack *>(dst + (int64_t)n * K + k) = p;
    }
  }
}

template <typename T> static void launch_transpose_2d(hipStream_t st, T *dst, const T *src, int K, int N) {
  const dim3 grid((unsigned)((N + 63) / 64), (unsigned)((K + 63) / 64));
  constexpr int V = 16 / sizeof(T);
  if (N % V == 0 && K % V == 0 && (uintptr_t)dst % 16 == 0 && (uintptr_t)src % 16 == 0)
    hipLaunchKernelGGL(k_transpose_2d_vec<T>, grid, dim3(256), 0, st, dst, src, K, N);
  else
    hipLaunchKernelGGL(k_transpose_2d<T>, grid, dim3(256), 0, st, dst, src, K, N);
}

int launch_linear_f32(hipStream_t st, const LinearArgs &a) {
  RAI_REQUIRE(a.M > 0 && a.N > 0 && a.K > 0, RAI_ERR_BAD_SHAPE, "linear: empty problem");
  RAI_REQUIRE(a.ln_kind < 0, RAI_ERR_UNSUPPORTED, "linear f32: no fused norm");
  const int tiles = ((a.M + 63) / 64) * ((a.N + 63) / 64);
  hipLaunchKernelGGL(k_linear_f32, dim3(tiles), dim3(256), 0, st, a);
  return launch_check("linear_f32");
}

// Lends the device's scratch block to a tile GEMM that may split K.
static int splitk_workspace(int dev, LinearArgs *la) {
  const size_t want = (size_t)8 * la->M * la->N * sizeof(float);
  const size_t cap = (size_t)256 << 20;
  const size_t bytes = want < cap ? want : cap;
  void *ws = nullptr;
  RAI_TRY(workspace(dev, bytes, &ws));
  la->splitk_ws = ws;
  la->splitk_ws_bytes = bytes;
  return RAI_OK;
}

}  // namespace rai

using namespace rai;

extern "C" {

int rai_hip_matmul(int dev, const rai_hip_tensor *a, const rai_hip_tensor *b, const rai_hip_tensor *out) {
  RAI_TRY(validate(a, "a"));
  RAI_TRY(validate(b, "b"));
  RAI_TRY(validate(out, "out"));
  RAI_REQUIRE(a->dtype == b->dtype && a->dtype == out->dtype, RAI_ERR_BAD_DTYPE, "matmul: dtypes differ (%s, %s, %s)",
              dtype_name(a->dtype), dtype_name(b->dtype), dtype_name(out->dtype));
  RAI_REQUIRE(is_float(a->dtype), RAI_ERR_BAD_DTYPE, "matmul: float dtype required");
  RAI_REQUIRE(a->rank >= 2 && b->rank == a->rank && out->rank == a->rank, RAI_ERR_BAD_SHAPE,
              "matmul: operands must have equal rank >= 2 (got %d, %d, %d)", a->rank, b->rank, out->rank);
  const int r = a->rank;
  const int64_t M = a->shape[r - 2], K = a->shape[r - 1], N = b->shape[r - 1];
  RAI_REQUIRE(b->shape[r - 2] == K, RAI_ERR_BAD_SHAPE, "matmul: inner dims %lld vs %lld", (long long)K,
              (long long)b->shape[r - 2]);
  RAI_REQUIRE(out->shape[r - 2] == M && out->shape[r - 1] == N, RAI_ERR_BAD_SHAPE, "matmul: output is not [%lld,%lld]",
              (long long)M, (long long)N);
  int64_t batch = 1;
  for (int i = 0; i < r - 2; ++i) {
    RAI_REQUIRE(a->shape[i] == out->shape[i] && b->shape[i] == out->shape[i], RAI_ERR_BAD_SHAPE,
                "matmul: batch dims must be broadcast to the output's");
    batch *= out->shape[i];
  }
  RAI_REQUIRE(is_contiguous(out), RAI_ERR_BAD_STRIDE, "matmul: output must be contiguous");
  hipStream_t st = stream_of(dev);
  if (!st) return RAI_ERR_HIP;
  if (numel(out) == 0) return RAI_OK;
  if (K == 0) return rai_hip_fill(dev, out, 0.0);

  // Fast path: one weight matrix shared by every batch (stride-0 batch dims) in
  // NT layout with K-contiguous activations whose rows share one stride -> the
  // batch folds into M.
  if ((a->dtype == RAI_BF16 || a->dtype == RAI_F32) && b->stride[r - 2] == 1 && (a->stride[r - 1] == 1 || K == 1)) {
    bool b_shared = true;
    for (int i = 0; i < r - 2; ++i)
      if (b->shape[i] != 1 && b->stride[i] != 0) b_shared = false;
    rai_hip_tensor rows = *a;
    rows.rank = r - 1;
    const rai_hip_tensor *ts[1] = {&rows};
    StridedArgs ca;
    coalesce(1, ts, &ca);
    const size_t es = dtype_size(a->dtype);
    const int v = (int)(16 / es);
    int64_t lda = (batch * M == 1) ? K : ca.stride[0][0];
    int64_t ldw = N == 1 ? K : b->stride[r - 1];
    bool aligned = K % v == 0 && lda % v == 0 && ldw % v == 0 && (uintptr_t)base_ptr(a) % 16 == 0 &&
                   (uintptr_t)base_ptr(b) % 16 == 0;
    if (b_shared && ca.rank == 1 && batch * M < (1LL << 31) && (a->dtype == RAI_F32 || aligned) && ldw >= K) {
      LinearArgs la = linear_args_default();
  la.dev = dev;
      la.A = base_ptr(a);
      la.lda = lda;
      la.W = base_ptr(b);
      la.ldw = ldw;
      la.out1 = base_ptr(out);
      la.ld1 = N;
      la.M = (int)(batch * M);
      la.N = (int)N;
      la.K = (int)K;
      la.n_split = (int)N;
      if (a->dtype == RAI_BF16 && la.M > 8 && la.K % 32 != 0) goto generic;
      if (a->dtype == RAI_BF16 && la.M > 8) RAI_TRY(splitk_workspace(dev, &la));
      return a->dtype == RAI_BF16 ? launch_linear_bf16(st, la) : launch_linear_f32(st, la);
    }
  }

  // NN layout with one shared right operand (B[K,N] row-major): transpose B once into a
  // scratch [N,K] (one pass over B) and run the NT tile kernel on the batch folded into M.
  if ((a->dtype == RAI_BF16 || a->dtype == RAI_F32) && b->stride[r - 1] == 1 && b->stride[r - 2] == N && N > 1 && K > 1 &&
      (double)batch * M * N * K >= 1e8) {
    bool b_shared = true;
    for (int i = 0; i < r - 2; ++i)
      if (b->shape[i] != 1 && b->stride[i] != 0) b_shared = false;
    if (b_shared) {
      void *tmp = nullptr;
      RAI_TRY(rai_hip_alloc(dev, (size_t)N * K * dtype_size(b->dtype), &tmp));
      hipStream_t tst = stream_of(dev);
      if (b->dtype == RAI_BF16)
        launch_transpose_2d<uint16_t>(tst, (uint16_t *)tmp, (const uint16_t *)base_ptr(b), (int)K, (int)N);
      else
        launch_transpose_2d<float>(tst, (float *)tmp, (const float *)base_ptr(b), (int)K, (int)N);
      int rc = launch_check("transpose_2d");
      if (rc == RAI_OK) {
        rai_hip_tensor b2 = *b;  // [.., K, N] view of the transposed copy: strides (1, K), batch strides 0
        b2.data = tmp; b2.offset = 0;
        for (int i = 0; i < r - 2; ++i) b2.stride[i] = 0;
        b2.stride[r - 2] = 1; b2.stride[r - 1] = K;
        rc = rai_hip_matmul(dev, a, &b2, out);
      }
      (void)rai_hip_release(tmp);  // stream-ordered reuse: later work on this stream runs after the product
      return rc;
    }
  }

generic:
  MatmulArgs g;
  g.M = M; g.N = N; g.K = K;
  g.a_rs = a->stride[r - 2]; g.a_cs = a->stride[r - 1];
  g.b_rs = b->stride[r - 2]; g.b_cs = b->stride[r - 1];
  g.batch_rank = r - 2;
  for (int i = 0; i < RAI_HIP_MAX_RANK; ++i) {
    bool in = i < r - 2;
    g.batch_shape[i] = in ? out->shape[i] : 1;
    g.a_bs[i] = in ? a->stride[i] : 0;
    g.b_bs[i] = in ? b->stride[i] : 0;
  }
  RAI_REQUIRE(batch <= 65535, RAI_ERR_UNSUPPORTED, "matmul: batch %lld exceeds grid limit", (long long)batch);
  dim3 grid((unsigned)((N + 63) / 64), (unsigned)((M + 63) / 64), (unsigned)batch);
  RAI_DISPATCH_FLOAT(a->dtype, T,
                     hipLaunchKernelGGL((k_matmul_generic<T>), grid, dim3(256), 0, st, (T *)base_ptr(out),
                                        (const T *)base_ptr(a), (const T *)base_ptr(b), g));
  return launch_check("matmul_generic");
}

int rai_hip_linear(int dev, const rai_hip_tensor *x, const rai_hip_tensor *w, const rai_hip_tensor *bias, int32_t act,
                   const rai_hip_tensor *residual, const rai_hip_tensor *out) {
  RAI_TRY(validate(x, "x"));
  RAI_TRY(validate(w, "w"));
  RAI_TRY(validate(out, "out"));
  RAI_REQUIRE(x->dtype == RAI_BF16 || x->dtype == RAI_F32, RAI_ERR_BAD_DTYPE, "linear: bf16 or f32 required");
  RAI_REQUIRE(w->dtype == x->dtype && out->dtype == x->dtype, RAI_ERR_BAD_DTYPE, "linear: dtype mismatch");
  RAI_REQUIRE(w->rank == 2 && x->rank >= 1 && out->rank == x->rank, RAI_ERR_BAD_SHAPE, "linear: bad ranks");
  const int64_t N = w->shape[0], K = w->shape[1];
  RAI_REQUIRE(x->shape[x->rank - 1] == K && out->shape[out->rank - 1] == N, RAI_ERR_BAD_SHAPE,
              "linear: x[..,%lld] w[%lld,%lld] out[..,%lld]", (long long)x->shape[x->rank - 1], (long long)N,
              (long long)K, (long long)out->shape[out->rank - 1]);
  for (int i = 0; i < x->rank - 1; ++i)
    RAI_REQUIRE(x->shape[i] == out->shape[i], RAI_ERR_BAD_SHAPE, "linear: leading dims differ");
  RAI_REQUIRE(is_contiguous(out), RAI_ERR_BAD_STRIDE, "linear: output must be contiguous");
  RAI_REQUIRE((w->stride[1] == 1 || K == 1) && (x->stride[x->rank - 1] == 1 || K == 1), RAI_ERR_BAD_STRIDE,
              "linear: x and w must be K-contiguous");
  RAI_REQUIRE(act == -1 || act == RAI_UN_GELU || act == RAI_UN_NEW_GELU || act == RAI_UN_SILU || act == RAI_UN_RELU ||
                  act == RAI_UN_TANH,
              RAI_ERR_BAD_ARG, "linear: unsupported activation %d", act);
  const int64_t M = K ? numel(x) / K : 0;
  if (numel(out) == 0) return RAI_OK;
  RAI_REQUIRE(M < (1LL << 31) && K > 0, RAI_ERR_BAD_SHAPE, "linear: bad problem size");
  rai_hip_tensor rows = *x;
  rows.rank = x->rank - 1;
  const rai_hip_tensor *ts[1] = {&rows};
  StridedArgs ca;
  coalesce(1, ts, &ca);
  RAI_REQUIRE(ca.rank == 1, RAI_ERR_BAD_STRIDE, "linear: rows of x must share one stride");
  LinearArgs la = linear_args_default();
  la.dev = dev;
  la.A = base_ptr(x);
  la.lda = M == 1 ? K : ca.stride[0][0];
  la.W = base_ptr(w);
  la.ldw = N == 1 ? K : w->stride[0];
  if (bias) {
    RAI_TRY(validate(bias, "bias"));
    RAI_REQUIRE(bias->dtype == x->dtype && bias->rank == 1 && bias->shape[0] == N && (bias->stride[0] == 1 || N == 1),
                RAI_ERR_BAD_SHAPE, "linear: bias must be a contiguous [%lld] vector of x's dtype", (long long)N);
    la.bias = base_ptr(bias);
  }
  if (residual) {
    RAI_TRY(validate(residual, "residual"));
    RAI_REQUIRE(residual->dtype == x->dtype && same_shape(residual, out) && is_contiguous(residual), RAI_ERR_BAD_SHAPE,
                "linear: residual must be contiguous with the output's shape");
    la.residual = base_ptr(residual);
    la.ldr = N;
  }
  la.out1 = base_ptr(out);
  la.ld1 = N;
  la.M = (int)M;
  la.N = (int)N;
  la.K = (int)K;
  la.n_split = (int)N;
  la.act = act;
  la.act_from = 0;
  hipStream_t st = stream_of(dev);
  if (!st) return RAI_ERR_HIP;
  if (x->dtype == RAI_BF16 && la.M > 8) {
    RAI_REQUIRE(K % 32 == 0, RAI_ERR_UNSUPPORTED, "linear: bf16 with M > 8 needs K %% 32 == 0 (K=%lld)", (long long)K);
    RAI_TRY(splitk_workspace(dev, &la));
  }
  return x->dtype == RAI_BF16 ? launch_linear_bf16(st, la) : launch_linear_f32(st, la);
}

int rai_hip_linear_packed(int dev, const rai_hip_tensor *x, const rai_hip_tensor *w, const rai_hip_tensor *bias,
                          const rai_hip_tensor *bias2, int32_t act, int32_t act_from, const rai_hip_tensor *residual,
                          int32_t glu, int32_t k_splits, const rai_hip_tensor *out1, const rai_hip_tensor *out2) {
  RAI_TRY(validate(x, "x"));
  RAI_TRY(validate(w, "w"));
  RAI_TRY(validate(out1, "out1"));
  RAI_REQUIRE(x->dtype == RAI_BF16, RAI_ERR_BAD_DTYPE, "linear_packed: bf16 required");
  RAI_REQUIRE(w->dtype == x->dtype && out1->dtype == x->dtype, RAI_ERR_BAD_DTYPE, "linear_packed: dtype mismatch");
  RAI_REQUIRE(w->rank == 2 && x->rank == 2 && out1->rank == 2, RAI_ERR_BAD_SHAPE, "linear_packed: x, w, out1 must be rank 2");
  const int64_t M = x->shape[0], N = w->shape[0], K = w->shape[1];
  RAI_REQUIRE(x->shape[1] == K && out1->shape[0] == M, RAI_ERR_BAD_SHAPE, "linear_packed: x[%lld,%lld] w[%lld,%lld] out1[%lld,..]",
              (long long)M, (long long)x->shape[1], (long long)N, (long long)K, (long long)out1->shape[0]);
  RAI_REQUIRE(M > 0 && N > 0 && K > 0 && M < (1LL << 31) && N < (1LL << 31), RAI_ERR_BAD_SHAPE, "linear_packed: bad problem size");
  RAI_REQUIRE(x->stride[1] == 1 && w->stride[1] == 1 && is_contiguous(out1), RAI_ERR_BAD_STRIDE,
              "linear_packed: x and w must be K-contiguous, outputs contiguous");
  RAI_REQUIRE(act == -1 || act == RAI_UN_GELU || act == RAI_UN_NEW_GELU || act == RAI_UN_SILU || act == RAI_UN_RELU ||
                  act == RAI_UN_TANH,
              RAI_ERR_BAD_ARG, "linear_packed: unsupported activation %d", act);
  RAI_REQUIRE(act_from >= 0 && act_from <= N && k_splits >= 0, RAI_ERR_BAD_ARG, "linear_packed: bad act_from / k_splits");
  const int64_t n1 = out1->shape[1];
  LinearArgs la = linear_args_default();
  la.dev = dev;
  if (glu) {
    RAI_REQUIRE(N % 2 == 0 && n1 == N / 2 && !out2 && !residual && !bias2 && act >= 0 && act_from == 0, RAI_ERR_BAD_ARG,
                "linear_packed: a gated product writes N/2 columns to out1 and takes an activation, no residual, "
                "no second bias and no second output");
    la.n_split = (int)N;
  } else {
    RAI_REQUIRE(n1 >= 1 && n1 <= N, RAI_ERR_BAD_SHAPE, "linear_packed: out1 has %lld of %lld columns", (long long)n1, (long long)N);
    la.n_split = (int)n1;
    if (n1 < N) {
      RAI_REQUIRE(out2, RAI_ERR_BAD_ARG, "linear_packed: out2 missing for columns [%lld, %lld)", (long long)n1, (long long)N);
      RAI_TRY(validate(out2, "out2"));
      RAI_REQUIRE(out2->dtype == x->dtype && out2->rank == 2 && out2->shape[0] == M && out2->shape[1] == N - n1 &&
                      is_contiguous(out2),
                  RAI_ERR_BAD_SHAPE, "linear_packed: out2 must be a contiguous [%lld,%lld]", (long long)M, (long long)(N - n1));
      RAI_REQUIRE(!residual, RAI_ERR_BAD_ARG, "linear_packed: a residual needs a single output");
      la.out2 = base_ptr(out2);
      la.ld2 = N - n1;
    } else {
      RAI_REQUIRE(!out2, RAI_ERR_BAD_ARG, "linear_packed: out1 takes every column, out2 must be null");
    }
  }
  la.A = base_ptr(x);
  la.lda = M == 1 ? K : x->stride[0];
  la.W = base_ptr(w);
  la.ldw = N == 1 ? K : w->stride[0];
  const rai_hip_tensor *bs[2] = {bias, bias2};
  for (int i = 0; i < 2; ++i) {
    if (!bs[i]) continue;
    RAI_TRY(validate(bs[i], "bias"));
    RAI_REQUIRE(bs[i]->dtype == x->dtype && bs[i]->rank == 1 && bs[i]->shape[0] == N && (bs[i]->stride[0] == 1 || N == 1),
                RAI_ERR_BAD_SHAPE, "linear_packed: a bias must be a contiguous [%lld] vector of x's dtype", (long long)N);
    (i ? la.bias2 : la.bias) = base_ptr(bs[i]);
  }
  if (residual) {
    RAI_TRY(validate(residual, "residual"));
    RAI_REQUIRE(residual->dtype == x->dtype && same_shape(residual, out1) && is_contiguous(residual), RAI_ERR_BAD_SHAPE,
                "linear_packed: residual must be contiguous with the output's shape");
    la.residual = base_ptr(residual);
    la.ldr = N;
  }
  la.out1 = base_ptr(out1);
  la.ld1 = n1;
  la.M = (int)M;
  la.N = (int)N;
  la.K = (int)K;
  la.act = act;
  la.act_from = act_from;
  la.glu = glu ? 1 : 0;
  la.force_splits = k_splits;
  hipStream_t st = stream_of(dev);
  if (!st) return RAI_ERR_HIP;
  if (la.M > 8) {
    RAI_REQUIRE(K % 32 == 0, RAI_ERR_UNSUPPORTED, "linear_packed: M > 8 needs K %% 32 == 0 (K=%lld)", (long long)K);
    RAI_TRY(splitk_workspace(dev, &la));
  }
  return launch_linear_bf16(st, la);
}

}  // extern "C"
