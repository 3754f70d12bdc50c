// LayerNorm, RMSNorm and rotary-embedding kernels (HBM-bound, one read and one
// write of the activation).  A wave64 owns a row: the row is loaded once into
// registers with 16-byte accesses, reduced with shuffles, and written back.
//
// Reference compositions: rai-nn/src/layer_norm.rs:32-42 (mean hlops/mean.rs:4-7,
// population var hlops/var.rs:33-38, rsqrt = 1/sqrt candle.rs:545-553),
// rai-nn/src/rms_norm.rs:18-22, rai-models/src/llm/gemma.rs:42-54,
// rotary: rai-models/src/llm/phi2.rs:44-78, qwen2.rs:33-72.
#include "common.h"

namespace rai {

template <typename T, int V> struct alignas(sizeof(T) * V) NPack { T v[V]; };

enum NormKind { kLayerNorm = 0, kRmsNorm = 1, kRmsNormAddOne = 2 };

// rows x n, unit stride inside a row.  blockDim = 256 = 4 waves = 4 rows.
template <typename T, int V, int ITEMS>
__global__ void __launch_bounds__(256)
k_norm_wave(T *out, const T *x, const T *w, const T *b, int64_t rows, int64_t n, int64_t x_row_stride, float eps,
            int kind) {
  const int lane = threadIdx.x & 63;
  const int64_t packs = n / V;
  for (int64_t row = blockIdx.x * 4 + (threadIdx.x >> 6); row < rows; row += (int64_t)gridDim.x * 4) {
    const T *xr = x + row * x_row_stride;
    float v[ITEMS][V];
    float s = 0.f;
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
      int64_t p = lane + it * 64;
      if (p < packs) {
        NPack<T, V> pk = *reinterpret_cast<const NPack<T, V> *>(xr + p * V);
#pragma unroll
        for (int j = 0; j < V; ++j) {
          v[it][j] = (float)Scalar<T>::load(&pk.v[j]);
          s += kind == kLayerNorm ? v[it][j] : v[it][j] * v[it][j];
        }
      }
    }
    s = wave_sum(s);
    float mean = 0.f, scale;
    if (kind == kLayerNorm) {
      mean = s / (float)n;
      float q = 0.f;
#pragma unroll
      for (int it = 0; it < ITEMS; ++it) {
        int64_t p = lane + it * 64;
        if (p < packs) {
#pragma unroll
          for (int j = 0; j < V; ++j) {
            float d = v[it][j] - mean;
            q += d * d;
          }
        }
      }
      q = wave_sum(q);
      scale = 1.0f / sqrtf(q / (float)n + eps);
    } else {
      scale = 1.0f / sqrtf(s / (float)n + eps);
    }
    T *yr = out + row * n;
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
      int64_t p = lane + it * 64;
      if (p < packs) {
        NPack<T, V> wk, bk, ok;
        if (w) wk = *reinterpret_cast<const NPack<T, V> *>(w + p * V);
        if (b) bk = *reinterpret_cast<const NPack<T, V> *>(b + p * V);
#pragma unroll
        for (int j = 0; j < V; ++j) {
          float y = (v[it][j] - mean) * scale;
          if (w) {
            float wf = (float)Scalar<T>::load(&wk.v[j]);
            y *= (kind == kRmsNormAddOne) ? (1.0f + wf) : wf;
          }
          if (b) y += (float)Scalar<T>::load(&bk.v[j]);
          Scalar<T>::store(&ok.v[j], y);
        }
        *reinterpret_cast<NPack<T, V> *>(yr + p * V) = ok;
      }
    }
  }
}

// Fallback for rows that do not fit the register budget or are unaligned: one
// block per row, the row is re-read from L2 for each pass.
template <typename T>
__global__ void __launch_bounds__(256)
k_norm_block(T *out, const T *x, const T *w, const T *b, int64_t rows, int64_t n, int64_t x_row_stride, double eps_d,
             int kind) {
  typedef typename Scalar<T>::compute C;
  __shared__ C sh[4];
  auto block_sum = [&](C v) -> C {
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = v;
    __syncthreads();
    return sh[0] + sh[1] + sh[2] + sh[3];
  };
  const C eps = (C)eps_d;
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const T *xr = x + row * x_row_stride;
    C s = 0;
    for (int64_t i = threadIdx.x; i < n; i += 256) {
      C v = Scalar<T>::load(xr + i);
      s += kind == kLayerNorm ? v : v * v;
    }
    s = block_sum(s);
    C mean = 0, scale;
    if (kind == kLayerNorm) {
      mean = s / (C)n;
      C q = 0;
      for (int64_t i = threadIdx.x; i < n; i += 256) {
        C d = Scalar<T>::load(xr + i) - mean;
        q += d * d;
      }
      q = block_sum(q);
      scale = C(1) / sqrt(q / (C)n + eps);
    } else {
      scale = C(1) / sqrt(s / (C)n + eps);
    }
    T *yr = out + row * n;
    for (int64_t i = threadIdx.x; i < n; i += 256) {
      C y = (Scalar<T>::load(xr + i) - mean) * scale;
      if (w) {
        C wf = Scalar<T>::load(w + i);
        y *= (kind == kRmsNormAddOne) ? (C(1) + wf) : wf;
      }
      if (b) y += Scalar<T>::load(b + i);
      Scalar<T>::store(yr + i, y);
    }
  }
}

// ---------------------------------------------------------------- rope
struct RopeArgs {
  int64_t B, H, S, D;
  int64_t xs[4];  // input strides
  int64_t rot, half, offset;
  int64_t tab_row_stride;
};

// A value rounded to storage type T and widened again: the rounding every node of the reference's rotary chain
// (x * cos, rotate_half(x) * sin, their sum: rai-models/src/llm/phi2.rs:66-77) applies to its result.
template <typename T> __device__ __forceinline__ float rope_round(float v) {
  T tmp;
  Scalar<T>::store(&tmp, (typename Scalar<T>::compute)v);
  return (float)Scalar<T>::load(&tmp);
}

template <typename T, typename TT>
__global__ void __launch_bounds__(256) k_rope(T *out, const T *x, const TT *cos_t, const TT *sin_t, RopeArgs a) {
#pragma clang fp contract(off)   // two products and a sum, each rounded on its own: no fused multiply-add

  const int64_t total = a.B * a.H * a.S * a.D;
  for (int64_t e = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; e < total; e += (int64_t)gridDim.x * blockDim.x) {
    int64_t d = e % a.D;
    int64_t r = e / a.D;
    int64_t s = r % a.S;
    r /= a.S;
    int64_t h = r % a.H;
    int64_t b = r / a.H;
    const T *xp = x + b * a.xs[0] + h * a.xs[1] + s * a.xs[2];
    float v = (float)Scalar<T>::load(xp + d * a.xs[3]);
    if (d < a.rot) {
      const int64_t trow = (a.offset + s) * a.tab_row_stride;
      float c = (float)Scalar<TT>::load(cos_t + trow + d);
      float sn = (float)Scalar<TT>::load(sin_t + trow + d);
      // rotate_half = cat(-x2, x1)
      float other = d < a.half ? -(float)Scalar<T>::load(xp + (d + a.half) * a.xs[3])
                               : (float)Scalar<T>::load(xp + (d - a.half) * a.xs[3]);
      v = rope_round<T>(v * c) + rope_round<T>(other * sn);
    }
    Scalar<T>::store(out + e, v);
  }
}

// Same operation, one thread per 16 bytes of a row: requires unit inner stride, D, rot and
// rot/2 multiples of the pack width, 16-byte aligned rows, and fewer than 2^31 packs (all
// index arithmetic in 32 bits; the per-element form spends most of its time in 64-bit
// divisions).
template <typename T, typename TT>
__global__ void __launch_bounds__(256) k_rope_vec(T *out, const T *x, const TT *cos_t, const TT *sin_t, RopeArgs a) {
#pragma clang fp contract(off)
  constexpr int VEC = 16 / sizeof(T);
  struct alignas(16) Pack { T v[VEC]; };
  const uint32_t cpr = (uint32_t)(a.D / VEC), S = (uint32_t)a.S, H = (uint32_t)a.H;
  const uint32_t total = (uint32_t)(a.B * a.H * a.S) * cpr;
  const uint32_t rot = (uint32_t)a.rot, half = (uint32_t)a.half;
  for (uint32_t idx = blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += gridDim.x * blockDim.x) {
    const uint32_t row = idx / cpr, d = (idx - row * cpr) * VEC;
    const uint32_t s = row % S, r2 = row / S, h = r2 % H, b = r2 / H;
    const T *xp = x + (int64_t)b * a.xs[0] + (int64_t)h * a.xs[1] + (int64_t)s * a.xs[2];
    Pack v = *reinterpret_cast<const Pack *>(xp + d);
    if (d < rot) {
      const Pack o = *reinterpret_cast<const Pack *>(xp + (d < half ? d + half : d - half));
      const int64_t trow = (a.offset + s) * a.tab_row_stride + d;
      const float sign = d < half ? -1.f : 1.f;  // rotate_half = cat(-x2, x1)
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const float c = (float)Scalar<TT>::load(cos_t + trow + j), sn = (float)Scalar<TT>::load(sin_t + trow + j);
        const float r = rope_round<T>((float)Scalar<T>::load(&v.v[j]) * c) +
                        rope_round<T>(sign * (float)Scalar<T>::load(&o.v[j]) * sn);
        Scalar<T>::store(&v.v[j], (typename Scalar<T>::compute)r);
      }
    }
    *reinterpret_cast<Pack *>(out + (int64_t)row * a.D + d) = v;
  }
}

template <typename TT>
__global__ void __launch_bounds__(256)
k_rope_tables(TT *cos_t, TT *sin_t, int64_t max_pos, int rot, double theta, int f64_powf) {
  const int half = rot / 2;
  for (int64_t e = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; e < max_pos * rot;
       e += (int64_t)gridDim.x * blockDim.x) {
    int64_t pos = e / rot;
    int i = (int)(e % rot) % half;
    float inv_freq;
    if (f64_powf) inv_freq = (float)(1.0 / pow(theta, (double)(2 * i) / (double)rot));
    else inv_freq = 1.0f / powf((float)theta, (float)(2 * i) / (float)rot);
    float ang = (float)pos * inv_freq;
    Scalar<TT>::store(cos_t + e, (typename Scalar<TT>::compute)cosf(ang));
    Scalar<TT>::store(sin_t + e, (typename Scalar<TT>::compute)sinf(ang));
  }
}

static int norm_impl(int dev, const rai_hip_tensor *x, const rai_hip_tensor *w, const rai_hip_tensor *b, double eps,
                     int kind, const rai_hip_tensor *out, const char *what) {
  RAI_TRY(validate(x, "x"));
  RAI_TRY(validate(out, "out"));
  RAI_REQUIRE(is_float(x->dtype), RAI_ERR_BAD_DTYPE, "%s: float dtype required", what);
  RAI_REQUIRE(x->dtype == out->dtype, RAI_ERR_BAD_DTYPE, "%s: dtype mismatch", what);
  RAI_REQUIRE(x->rank >= 1, RAI_ERR_BAD_SHAPE, "%s: rank 0 input", what);
  RAI_REQUIRE(same_shape(x, out), RAI_ERR_BAD_SHAPE, "%s: shape mismatch", what);
  RAI_REQUIRE(is_contiguous(out), RAI_ERR_BAD_STRIDE, "%s: output must be contiguous", what);
  const int64_t n = x->shape[x->rank - 1];
  RAI_REQUIRE(n > 0, RAI_ERR_BAD_SHAPE, "%s: empty normalised axis", what);
  const rai_hip_tensor *params[2] = {w, b};
  for (const rai_hip_tensor *p : params) {
    if (!p) continue;
    RAI_TRY(validate(p, "param"));
    RAI_REQUIRE(p->dtype == x->dtype, RAI_ERR_BAD_DTYPE, "%s: parameter dtype must equal x dtype", what);
    RAI_REQUIRE(p->rank == 1 && p->shape[0] == n && (p->stride[0] == 1 || n == 1), RAI_ERR_BAD_SHAPE,
                "%s: parameter must be a contiguous [%lld] vector", what, (long long)n);
  }
  RAI_REQUIRE(x->stride[x->rank - 1] == 1 || n == 1, RAI_ERR_BAD_STRIDE, "%s: last dim must have unit stride", what);
  hipStream_t st = stream_of(dev);
  if (!st) return RAI_ERR_HIP;
  if (numel(out) == 0) return RAI_OK;
  // rows must be addressable with a single stride
  rai_hip_tensor rows_view = *x;
  rows_view.rank = x->rank - 1;
  const rai_hip_tensor *ts[1] = {&rows_view};
  StridedArgs ca;
  coalesce(1, ts, &ca);
  RAI_REQUIRE(ca.rank == 1, RAI_ERR_BAD_STRIDE, "%s: rows of x must share one stride (make x contiguous)", what);
  const int64_t rows = numel(x) / n;
  const int64_t row_stride = rows == 1 ? n : ca.stride[0][0];
  const size_t es = dtype_size(x->dtype);
  const int v = (int)(16 / es);
  auto al = [&](const rai_hip_tensor *t) { return !t || ((uintptr_t)base_ptr(t) % 16 == 0); };
  bool aligned = (n % v == 0) && (row_stride % v == 0) && al(x) && al(out) && al(w) && al(b);
  const int64_t packs = n / v;
  if (aligned && x->dtype != RAI_F64 && packs <= 64 * 16) {
    int64_t blocks = (rows + 3) / 4;
    int grid = (int)(blocks < kNumCU * 32 ? blocks : kNumCU * 32);
#define NORM_LAUNCH(T, V, ITEMS)                                                                                  \
  hipLaunchKernelGGL((k_norm_wave<T, V, ITEMS>), dim3(grid), dim3(256), 0, st, (T *)base_ptr(out),                \
                     (const T *)base_ptr(x), w ? (const T *)base_ptr(w) : nullptr,                                \
                     b ? (const T *)base_ptr(b) : nullptr, rows, n, row_stride, (float)eps, kind)
#define NORM_BY_ITEMS(T, V)                        \
  do {                                             \
    if (packs <= 64 * 2) NORM_LAUNCH(T, V, 2);     \
    else if (packs <= 64 * 5) NORM_LAUNCH(T, V, 5); \
    else if (packs <= 64 * 10) NORM_LAUNCH(T, V, 10); \
    else NORM_LAUNCH(T, V, 16);                    \
  } while (0)
    if (x->dtype == RAI_F32) NORM_BY_ITEMS(float, 4);
    else if (x->dtype == RAI_BF16) NORM_BY_ITEMS(bf16_raw, 8);
    else NORM_BY_ITEMS(f16_raw, 8);
#undef NORM_BY_ITEMS
#undef NORM_LAUNCH
    return launch_check(what);
  }
  int grid = (int)(rows < kNumCU * 16 ? rows : kNumCU * 16);
  RAI_DISPATCH_FLOAT(x->dtype, T,
                     hipLaunchKernelGGL((k_norm_block<T>), dim3(grid), dim3(256), 0, st, (T *)base_ptr(out),
                                        (const T *)base_ptr(x), w ? (const T *)base_ptr(w) : nullptr,
                                        b ? (const T *)base_ptr(b) : nullptr, rows, n, row_stride, eps, kind));
  return launch_check(what);
}

}  // namespace rai

using namespace rai;

extern "C" {

int rai_hip_layer_norm(int dev, const rai_hip_tensor *x, const rai_hip_tensor *w, const rai_hip_tensor *b, double eps,
                       const rai_hip_tensor *out) {
  RAI_REQUIRE((w == nullptr) == (b == nullptr), RAI_ERR_BAD_ARG, "layer_norm: weight and bias come together");
  return norm_impl(dev, x, w, b, eps, kLayerNorm, out, "layer_norm");
}

int rai_hip_rms_norm(int dev, const rai_hip_tensor *x, const rai_hip_tensor *w, double eps, int32_t add_one,
                     const rai_hip_tensor *out) {
  RAI_REQUIRE(w != nullptr, RAI_ERR_BAD_ARG, "rms_norm: weight required");
  return norm_impl(dev, x, w, nullptr, eps, add_one ? kRmsNormAddOne : kRmsNorm, out, "rms_norm");
}

int rai_hip_rope(int dev, const rai_hip_tensor *x, const rai_hip_tensor *cos_t, const rai_hip_tensor *sin_t,
                 int32_t rot_dim, int64_t offset, const rai_hip_tensor *out) {
  RAI_TRY(validate(x, "x"));
  RAI_TRY(validate(cos_t, "cos"));
  RAI_TRY(validate(sin_t, "sin"));
  RAI_TRY(validate(out, "out"));
  RAI_REQUIRE(x->rank == 4, RAI_ERR_BAD_SHAPE, "rope: x must be [B,H,S,D]");
  RAI_REQUIRE(is_float(x->dtype) && x->dtype != RAI_F64, RAI_ERR_BAD_DTYPE, "rope: f32/bf16/f16 required");
  RAI_REQUIRE(x->dtype == out->dtype, RAI_ERR_BAD_DTYPE, "rope: dtype mismatch");
  RAI_REQUIRE(same_shape(x, out) && is_contiguous(out), RAI_ERR_BAD_SHAPE, "rope: out must be contiguous, x's shape");
  const int64_t D = x->shape[3], S = x->shape[2];
  RAI_REQUIRE(rot_dim > 0 && rot_dim % 2 == 0 && rot_dim <= D, RAI_ERR_BAD_ARG, "rope: bad rot_dim %d for D=%lld",
              rot_dim, (long long)D);
  RAI_REQUIRE(cos_t->rank == 2 && sin_t->rank == 2 && cos_t->shape[1] == rot_dim && sin_t->shape[1] == rot_dim &&
                  cos_t->shape[0] == sin_t->shape[0],
              RAI_ERR_BAD_SHAPE, "rope: tables must be [max_pos, rot_dim]");
  RAI_REQUIRE(offset >= 0 && offset + S <= cos_t->shape[0], RAI_ERR_BAD_ARG,
              "rope: positions %lld..%lld exceed table rows %lld", (long long)offset, (long long)(offset + S),
              (long long)cos_t->shape[0]);
  RAI_REQUIRE(cos_t->dtype == sin_t->dtype && (cos_t->dtype == x->dtype || cos_t->dtype == RAI_F32), RAI_ERR_BAD_DTYPE,
              "rope: tables must be x's dtype or f32");
  RAI_REQUIRE(cos_t->stride[1] == 1 && sin_t->stride[1] == 1 && cos_t->stride[0] == sin_t->stride[0],
              RAI_ERR_BAD_STRIDE, "rope: tables must have unit inner stride and equal row strides");
  hipStream_t st = stream_of(dev);
  if (!st) return RAI_ERR_HIP;
  if (numel(out) == 0) return RAI_OK;
  RopeArgs a;
  a.B = x->shape[0]; a.H = x->shape[1]; a.S = S; a.D = D;
  for (int i = 0; i < 4; ++i) a.xs[i] = x->stride[i];
  a.rot = rot_dim; a.half = rot_dim / 2; a.offset = offset; a.tab_row_stride = cos_t->stride[0];
  const int vec = (int)(16 / dtype_size(x->dtype));
  const bool vec_ok = x->stride[3] == 1 && D % vec == 0 && rot_dim % vec == 0 && (rot_dim / 2) % vec == 0 &&
                      x->stride[0] % vec == 0 && x->stride[1] % vec == 0 && x->stride[2] % vec == 0 &&
                      (uintptr_t)base_ptr(x) % 16 == 0 && (uintptr_t)base_ptr(out) % 16 == 0 &&
                      numel(out) / vec < (int64_t)1 << 31;
  int64_t blocks = ((vec_ok ? numel(out) / vec : numel(out)) + 255) / 256;
  int grid = (int)(blocks < kNumCU * 32 ? blocks : kNumCU * 32);
#define ROPE_LAUNCH(T, TT)                                                                                       \
  do {                                                                                                           \
    if (vec_ok)                                                                                                  \
      hipLaunchKernelGGL((k_rope_vec<T, TT>), dim3(grid), dim3(256), 0, st, (T *)base_ptr(out),                  \
                         (const T *)base_ptr(x), (const TT *)base_ptr(cos_t), (const TT *)base_ptr(sin_t), a);   \
    else                                                                                                         \
      ROPE_LAUNCH_SCALAR(T, TT);                                                                                 \
  } while (0)
#define ROPE_LAUNCH_SCALAR(T, TT)                                                                                   \
  hipLaunchKernelGGL((k_rope<T, TT>), dim3(grid), dim3(256), 0, st, (T *)base_ptr(out), (const T *)base_ptr(x), \
                     (const TT *)base_ptr(cos_t), (const TT *)base_ptr(sin_t), a)
  if (x->dtype == RAI_F32) ROPE_LAUNCH(float, float);
  else if (x->dtype == RAI_BF16) { if (cos_t->dtype == RAI_F32) ROPE_LAUNCH(bf16_raw, float); else ROPE_LAUNCH(bf16_raw, bf16_raw); }
  else { if (cos_t->dtype == RAI_F32) ROPE_LAUNCH(f16_raw, float); else ROPE_LAUNCH(f16_raw, f16_raw); }
#undef ROPE_LAUNCH
#undef ROPE_LAUNCH_SCALAR
  return launch_check("rope");
}

int rai_hip_rope_tables(int dev, double theta, int32_t rot_dim, int32_t f64_powf, const rai_hip_tensor *cos_t,
                        const rai_hip_tensor *sin_t) {
  RAI_TRY(validate(cos_t, "cos"));
  RAI_TRY(validate(sin_t, "sin"));
  RAI_REQUIRE(rot_dim > 0 && rot_dim % 2 == 0, RAI_ERR_BAD_ARG, "rope_tables: bad rot_dim %d", rot_dim);
  RAI_REQUIRE(cos_t->rank == 2 && same_shape(cos_t, sin_t) && cos_t->shape[1] == rot_dim, RAI_ERR_BAD_SHAPE,
              "rope_tables: tables must be [max_pos, rot_dim]");
  RAI_REQUIRE(is_contiguous(cos_t) && is_contiguous(sin_t), RAI_ERR_BAD_STRIDE, "rope_tables: tables must be contiguous");
  RAI_REQUIRE(cos_t->dtype == sin_t->dtype && is_float(cos_t->dtype) && cos_t->dtype != RAI_F64, RAI_ERR_BAD_DTYPE,
              "rope_tables: f32/bf16/f16 tables");
  hipStream_t st = stream_of(dev);
  if (!st) return RAI_ERR_HIP;
  int64_t n = numel(cos_t);
  if (n == 0) return RAI_OK;
  int64_t blocks = (n + 255) / 256;
  int grid = (int)(blocks < 4096 ? blocks : 4096);
  RAI_DISPATCH_FLOAT(cos_t->dtype, T, {
    if constexpr (sizeof(T) <= 4)
      hipLaunchKernelGGL((k_rope_tables<T>), dim3(grid), dim3(256), 0, st, (T *)base_ptr(cos_t), (T *)base_ptr(sin_t),
                         cos_t->shape[0], (int)rot_dim, theta, (int)f64_powf);
  });
  return launch_check("rope_tables");
}

}  // extern "C"
