// Creation, cast, strided copy, unary, broadcast-binary and where kernels.
// HBM-bound: every kernel moves 16 bytes per lane per access when the innermost
// dimension allows it, and decomposes the outer index once per 16-byte pack.
//
// Reference semantics: rai-core/src/backend/candle.rs:197-325 (creation, arith),
// :445-473,525-553,608-656,947-978 (unary), :658-774 (compare, max/min, cast),
// :901-915 (where), :980-988 (contiguous).
#include "common.h"
#include "fused.h"

namespace rai {

template <typename T, int V> struct alignas(sizeof(T) * V) Pack { T v[V]; };

struct IterSpace {
  int rank;
  int64_t shape[RAI_HIP_MAX_RANK];
  int64_t stride[3][RAI_HIP_MAX_RANK];  // operand 0 is the output
  int64_t n_packs;                      // total / V
};

// Splits the linear index of a pack into per-operand element offsets.
template <int NOPS, int V>
__device__ __forceinline__ void decompose(const IterSpace &s, int64_t pack, int64_t *off) {
#pragma unroll
  for (int k = 0; k < NOPS; ++k) off[k] = 0;
  int64_t inner_packs = s.shape[s.rank - 1] / V;
  int64_t rem = pack / inner_packs;
  int64_t in = (pack - rem * inner_packs) * V;
#pragma unroll
  for (int k = 0; k < NOPS; ++k) off[k] = in * s.stride[k][s.rank - 1];
  for (int d = s.rank - 2; d >= 0; --d) {
    int64_t q = rem / s.shape[d];
    int64_t i = rem - q * s.shape[d];
    rem = q;
#pragma unroll
    for (int k = 0; k < NOPS; ++k) off[k] += i * s.stride[k][d];
  }
}

template <typename T, int V>
__device__ __forceinline__ void load_pack(const T *base, int64_t off, int64_t inner_stride, T *dst) {
  if (V > 1 && inner_stride == 1) {
    *reinterpret_cast<Pack<T, V> *>(dst) = *reinterpret_cast<const Pack<T, V> *>(base + off);
  } else {
#pragma unroll
    for (int j = 0; j < V; ++j) dst[j] = base[off + j * inner_stride];
  }
}
template <typename T, int V>
__device__ __forceinline__ void store_pack(T *base, int64_t off, int64_t inner_stride, const T *src) {
  if (V > 1 && inner_stride == 1) {
    *reinterpret_cast<Pack<T, V> *>(base + off) = *reinterpret_cast<const Pack<T, V> *>(src);
  } else {
#pragma unroll
    for (int j = 0; j < V; ++j) base[off + j * inner_stride] = src[j];
  }
}

// ------------------------------------------------------------------ math
template <typename C> __device__ __forceinline__ C unary_eval(int op, C x, C p) {
  switch (op) {
    case RAI_UN_SIN: return sin(x);
    case RAI_UN_COS: return cos(x);
    case RAI_UN_NEG: return -x;
    case RAI_UN_SQUARE: return x * x;
    case RAI_UN_SQRT: return sqrt(x);
    case RAI_UN_RSQRT: return C(1) / sqrt(x);
    case RAI_UN_ABS: return fabs(x);
    case RAI_UN_EXP: return exp(x);
    case RAI_UN_LOG: return log(x);
    case RAI_UN_LOG2: return log(x) / C(0.6931471805599453);
    case RAI_UN_LOG10: return log(x) / C(2.302585092994046);
    case RAI_UN_ERF: return erf(x);
    case RAI_UN_TANH: return tanh(x);
    case RAI_UN_POWF: return pow(x, p);
    case RAI_UN_SIGN: return C(x >= C(0)) - C(x <= C(0));
    case RAI_UN_GELU: return x * C(0.5) * (C(1) + erf(x / C(1.4142135623730951)));
    case RAI_UN_NEW_GELU: {
      // sqrt(2/pi) and 0.044715 as f32 constants, like hlops/activations.rs:25-27
      const C k = C(0.7978845608028654f);
      return C(0.5) * x * (C(1) + tanh(k * (x + C(0.044715f) * x * x * x)));
    }
    case RAI_UN_SILU: return x / (exp(-x) + C(1));
    case RAI_UN_RELU: return x > C(0) ? x : C(0);
    default: return x;
  }
}
template <> __device__ __forceinline__ float unary_eval<float>(int op, float x, float p) {
  switch (op) {
    case RAI_UN_SIN: return sinf(x);
    case RAI_UN_COS: return cosf(x);
    case RAI_UN_NEG: return -x;
    case RAI_UN_SQUARE: return x * x;
    case RAI_UN_SQRT: return sqrtf(x);
    case RAI_UN_RSQRT: return 1.0f / sqrtf(x);
    case RAI_UN_ABS: return fabsf(x);
    case RAI_UN_EXP: return expf(x);
    case RAI_UN_LOG: return logf(x);
    case RAI_UN_LOG2: return logf(x) / 0.6931471805599453f;
    case RAI_UN_LOG10: return logf(x) / 2.302585092994046f;
    case RAI_UN_ERF: return erff(x);
    case RAI_UN_TANH: return tanhf(x);
    case RAI_UN_POWF: return powf(x, p);
    case RAI_UN_SIGN: return float(x >= 0.f) - float(x <= 0.f);
    case RAI_UN_GELU: return x * 0.5f * (1.0f + erff(x / 1.4142135623730951f));
    case RAI_UN_NEW_GELU: {
      const float k = 0.7978845608028654f;
      return 0.5f * x * (1.0f + tanhf(k * (x + 0.044715f * x * x * x)));
    }
    case RAI_UN_SILU: return x / (expf(-x) + 1.0f);
    case RAI_UN_RELU: return x > 0.f ? x : 0.f;
    default: return x;
  }
}

template <typename C> __device__ __forceinline__ C cmax(C a, C b) { return a > b ? a : b; }
template <typename C> __device__ __forceinline__ C cmin(C a, C b) { return a < b ? a : b; }
template <> __device__ __forceinline__ float cmax<float>(float a, float b) {
  return (a != a || b != b) ? __uint_as_float(0x7fc00000u) : (a > b ? a : b);
}
template <> __device__ __forceinline__ float cmin<float>(float a, float b) {
  return (a != a || b != b) ? __uint_as_float(0x7fc00000u) : (a < b ? a : b);
}

template <typename C> __device__ __forceinline__ C arith_eval(int op, C a, C b) {
  switch (op) {
    case RAI_BIN_ADD: return a + b;
    case RAI_BIN_SUB: return a - b;
    case RAI_BIN_MUL: return a * b;
    case RAI_BIN_DIV: return a / b;
    case RAI_BIN_MAXIMUM: return cmax<C>(a, b);
    default: return cmin<C>(a, b);
  }
}
// Integer division by zero is a panic in the reference; here it yields 0.
template <> __device__ __forceinline__ uint8_t arith_eval<uint8_t>(int op, uint8_t a, uint8_t b) {
  switch (op) {
    case RAI_BIN_ADD: return a + b;
    case RAI_BIN_SUB: return a - b;
    case RAI_BIN_MUL: return a * b;
    case RAI_BIN_DIV: return b ? a / b : 0;
    case RAI_BIN_MAXIMUM: return a > b ? a : b;
    default: return a < b ? a : b;
  }
}
template <> __device__ __forceinline__ uint32_t arith_eval<uint32_t>(int op, uint32_t a, uint32_t b) {
  switch (op) {
    case RAI_BIN_ADD: return a + b;
    case RAI_BIN_SUB: return a - b;
    case RAI_BIN_MUL: return a * b;
    case RAI_BIN_DIV: return b ? a / b : 0;
    case RAI_BIN_MAXIMUM: return a > b ? a : b;
    default: return a < b ? a : b;
  }
}
template <> __device__ __forceinline__ int64_t arith_eval<int64_t>(int op, int64_t a, int64_t b) {
  switch (op) {
    case RAI_BIN_ADD: return a + b;
    case RAI_BIN_SUB: return a - b;
    case RAI_BIN_MUL: return a * b;
    case RAI_BIN_DIV: return b ? a / b : 0;
    case RAI_BIN_MAXIMUM: return a > b ? a : b;
    default: return a < b ? a : b;
  }
}
template <typename C> __device__ __forceinline__ uint8_t cmp_eval(int op, C a, C b) {
  switch (op) {
    case RAI_BIN_EQ: return a == b;
    case RAI_BIN_NE: return a != b;
    case RAI_BIN_GT: return a > b;
    case RAI_BIN_GE: return a >= b;
    case RAI_BIN_LT: return a < b;
    default: return a <= b;
  }
}

// ------------------------------------------------------------------ kernels
template <typename T, int V>
__global__ void __launch_bounds__(256) k_unary(IterSpace s, T *out, const T *in, int op, double param) {
  typedef typename Scalar<T>::compute C;
  for (int64_t p = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; p < s.n_packs;
       p += (int64_t)gridDim.x * blockDim.x) {
    int64_t off[2];
    decompose<2, V>(s, p, off);
    T a[V], r[V];
    load_pack<T, V>(in, off[1], s.stride[1][s.rank - 1], a);
#pragma unroll
    for (int j = 0; j < V; ++j) {
      C x = Scalar<T>::load(&a[j]);
      Scalar<T>::store(&r[j], unary_eval<C>(op, x, (C)param));
    }
    store_pack<T, V>(out, off[0], s.stride[0][s.rank - 1], r);
  }
}

template <typename T, int V>
__global__ void __launch_bounds__(256) k_copy(IterSpace s, T *out, const T *in) {
  for (int64_t p = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; p < s.n_packs;
       p += (int64_t)gridDim.x * blockDim.x) {
    int64_t off[2];
    decompose<2, V>(s, p, off);
    T a[V];
    load_pack<T, V>(in, off[1], s.stride[1][s.rank - 1], a);
    store_pack<T, V>(out, off[0], s.stride[0][s.rank - 1], a);
  }
}

template <typename T, int V>
__global__ void __launch_bounds__(256) k_binary(IterSpace s, T *out, const T *lhs, const T *rhs, int op) {
  typedef typename Scalar<T>::compute C;
  for (int64_t p = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; p < s.n_packs;
       p += (int64_t)gridDim.x * blockDim.x) {
    int64_t off[3];
    decompose<3, V>(s, p, off);
    T a[V], b[V], r[V];
    load_pack<T, V>(lhs, off[1], s.stride[1][s.rank - 1], a);
    load_pack<T, V>(rhs, off[2], s.stride[2][s.rank - 1], b);
#pragma unroll
    for (int j = 0; j < V; ++j)
      Scalar<T>::store(&r[j], arith_eval<C>(op, Scalar<T>::load(&a[j]), Scalar<T>::load(&b[j])));
    store_pack<T, V>(out, off[0], s.stride[0][s.rank - 1], r);
  }
}

template <typename T>
__global__ void __launch_bounds__(256) k_compare(IterSpace s, uint8_t *out, const T *lhs, const T *rhs, int op) {
  typedef typename Scalar<T>::compute C;
  for (int64_t p = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; p < s.n_packs;
       p += (int64_t)gridDim.x * blockDim.x) {
    int64_t off[3];
    decompose<3, 1>(s, p, off);
    C a = Scalar<T>::load(lhs + off[1]);
    C b = Scalar<T>::load(rhs + off[2]);
    out[off[0]] = cmp_eval<C>(op, a, b);
  }
}

// where: operand order in IterSpace = out, on_true, on_false; cond has its own strides
struct CondSpace { int64_t stride[RAI_HIP_MAX_RANK]; };
template <typename T, typename CT>
__global__ void __launch_bounds__(256)
k_where(IterSpace s, CondSpace cs, T *out, const T *on_true, const T *on_false, const CT *cond) {
  for (int64_t p = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; p < s.n_packs;
       p += (int64_t)gridDim.x * blockDim.x) {
    int64_t off[3] = {0, 0, 0};
    int64_t coff = 0;
    int64_t rem = p;
    for (int d = s.rank - 1; d >= 0; --d) {
      int64_t q = rem / s.shape[d];
      int64_t i = rem - q * s.shape[d];
      rem = q;
      off[0] += i * s.stride[0][d];
      off[1] += i * s.stride[1][d];
      off[2] += i * s.stride[2][d];
      coff += i * cs.stride[d];
    }
    out[off[0]] = cond[coff] != 0 ? on_true[off[1]] : on_false[off[2]];
  }
}

template <typename T>
__global__ void __launch_bounds__(256) k_fill(T *out, int64_t n, double value) {
  typedef typename Scalar<T>::compute C;
  T v;
  Scalar<T>::store(&v, (C)value);
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    out[i] = v;
}

template <typename T>
__global__ void __launch_bounds__(256) k_arange(T *out, int64_t n, double start, double step) {
  typedef typename Scalar<T>::compute C;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    Scalar<T>::store(out + i, (C)(start + (double)i * step));
}

// ---- cast
template <typename D, typename CS> struct Convert {
  static __device__ __forceinline__ void run(D *dst, CS v) {
    Scalar<D>::store(dst, (typename Scalar<D>::compute)v);
  }
};
// float -> integer: Rust `as` (truncate toward zero, saturate, NaN -> 0)
template <typename I, typename F> __device__ __forceinline__ I sat_cast(F v, double lo, double hi) {
  if (v != v) return I(0);
  double d = (double)v;
  if (d <= lo) return (I)lo;
  if (d >= hi) return (I)hi;
  return (I)d;
}
template <> struct Convert<uint8_t, float> {
  static __device__ __forceinline__ void run(uint8_t *d, float v) { *d = sat_cast<uint8_t>(v, 0.0, 255.0); }
};
template <> struct Convert<uint8_t, double> {
  static __device__ __forceinline__ void run(uint8_t *d, double v) { *d = sat_cast<uint8_t>(v, 0.0, 255.0); }
};
template <> struct Convert<uint32_t, float> {
  static __device__ __forceinline__ void run(uint32_t *d, float v) { *d = sat_cast<uint32_t>(v, 0.0, 4294967295.0); }
};
template <> struct Convert<uint32_t, double> {
  static __device__ __forceinline__ void run(uint32_t *d, double v) { *d = sat_cast<uint32_t>(v, 0.0, 4294967295.0); }
};
template <> struct Convert<int64_t, float> {
  static __device__ __forceinline__ void run(int64_t *d, float v) {
    if (v != v) { *d = 0; return; }
    if (v >= 9223372036854775808.0f) { *d = INT64_MAX; return; }
    if (v <= -9223372036854775808.0f) { *d = INT64_MIN; return; }
    *d = (int64_t)v;
  }
};
template <> struct Convert<int64_t, double> {
  static __device__ __forceinline__ void run(int64_t *d, double v) {
    if (v != v) { *d = 0; return; }
    if (v >= 9223372036854775808.0) { *d = INT64_MAX; return; }
    if (v <= -9223372036854775808.0) { *d = INT64_MIN; return; }
    *d = (int64_t)v;
  }
};

template <typename D, typename S>
__global__ void __launch_bounds__(256) k_cast(IterSpace s, D *out, const S *in) {
  typedef typename Scalar<S>::compute CS;
  for (int64_t p = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; p < s.n_packs;
       p += (int64_t)gridDim.x * blockDim.x) {
    int64_t off[2];
    decompose<2, 1>(s, p, off);
    CS v = Scalar<S>::load(in + off[1]);
    Convert<D, CS>::run(out + off[0], v);
  }
}

// ------------------------------------------------------------------ fused elementwise regions
__device__ __forceinline__ float fused_round(float v, int dtype) {
  if (dtype == RAI_BF16) return bf16_bits_to_f32(f32_to_bf16_bits(v));
  if (dtype == RAI_F16) return __half2float(__float2half_rn(v));
  return v;
}
__device__ __forceinline__ float fused_load(const void *base, int dtype, int64_t off) {
  if (dtype == RAI_BF16) return bf16_bits_to_f32(((const uint16_t *)base)[off]);
  if (dtype == RAI_F16) return __half2float(__ushort_as_half(((const uint16_t *)base)[off]));
  return ((const float *)base)[off];
}
// One element per thread per step; the register file of the little machine
// lives in LDS (one column per thread) because its indices are only known at
// run time.  Each instruction is evaluated in f32 by the same routines as the
// single-op kernels and rounded to the dtype of its node.
__global__ void __launch_bounds__(256) k_fused_elementwise(FusedProgram p) {
  __shared__ float regs[kFusedMaxInstr][256];
  const int tid = threadIdx.x;
  for (int64_t e = blockIdx.x * (int64_t)blockDim.x + tid; e < p.numel; e += (int64_t)gridDim.x * blockDim.x) {
    int64_t loff[kFusedMaxLeaves];
#pragma unroll
    for (int l = 0; l < kFusedMaxLeaves; ++l) loff[l] = 0;
    int64_t rem = e;
    for (int d = p.rank - 1; d >= 0; --d) {
      const int64_t c = rem % p.shape[d];
      rem /= p.shape[d];
#pragma unroll
      for (int l = 0; l < kFusedMaxLeaves; ++l)
        if (l < p.n_leaves) loff[l] += c * p.lstride[l][d];
    }
    float v = 0.f;
    for (int i = 0; i < p.n_instr; ++i) {
      const FusedInstr in = p.instr[i];
      switch (in.kind) {
        case FUSED_LEAF: {
          int64_t off = 0;
#pragma unroll
          for (int l = 0; l < kFusedMaxLeaves; ++l)
            if (l == in.a) off = loff[l];
          v = fused_load(p.leaf[in.a], p.leaf_dtype[in.a], off);
          break;
        }
        case FUSED_CONST: v = in.param; break;
        case FUSED_UNARY: v = fused_round(unary_eval<float>(in.op, regs[in.a][tid], in.param), in.dtype); break;
        case FUSED_BINARY: v = fused_round(arith_eval<float>(in.op, regs[in.a][tid], regs[in.b][tid]), in.dtype); break;
        default: v = fused_round(regs[in.a][tid], in.dtype); break;  // FUSED_CAST
      }
      regs[i][tid] = v;
    }
    if (p.out_dtype == RAI_BF16) ((uint16_t *)p.out)[e] = f32_to_bf16_bits(v);
    else if (p.out_dtype == RAI_F16) ((uint16_t *)p.out)[e] = __half_as_ushort(__float2half_rn(v));
    else ((float *)p.out)[e] = v;
  }
}

// ------------------------------------------------------------------ host side
static int grid_for(int64_t work_items) {
  int64_t blocks = (work_items + 255) / 256;
  int64_t cap = (int64_t)kNumCU * 16;
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  return (int)blocks;
}

// Builds the shared iteration space; picks the pack width (elements) such that
// every operand's innermost stride is 0 or 1... (stride 1 -> vector access).
static int build_space(int nops, const rai_hip_tensor *const *ts, int max_v, IterSpace *s, int *v_out) {
  StridedArgs a;
  coalesce(nops, ts, &a);
  s->rank = a.rank;
  int64_t total = 1;
  for (int i = 0; i < RAI_HIP_MAX_RANK; ++i) {
    s->shape[i] = a.shape[i];
    for (int k = 0; k < 3; ++k) s->stride[k][i] = a.stride[k][i];
    if (i < a.rank) total *= a.shape[i];
  }
  int v = max_v;
  int last = a.rank - 1;
  while (v > 1) {
    bool ok = (a.shape[last] % v) == 0;
    for (int k = 0; k < nops && ok; ++k) {
      int64_t is = a.stride[k][last];
      if (is != 0 && is != 1) ok = false;
      if (is == 1) {
        size_t es = dtype_size(ts[k]->dtype);
        uintptr_t addr = (uintptr_t)base_ptr(ts[k]);
        if (addr % (es * v)) ok = false;
        for (int d = 0; d < last; ++d)
          if (a.stride[k][d] % v) ok = false;
      }
    }
    if (ok) break;
    v >>= 1;
  }
  *v_out = v;
  s->n_packs = total / v;
  return RAI_OK;
}

template <typename T> static int max_pack() { return (int)(16 / sizeof(T)); }

int launch_fused_elementwise(int dev, const FusedProgram &p) {
  hipStream_t st = stream_of(dev);
  if (!st) return RAI_ERR_HIP;
  if (p.numel == 0) return RAI_OK;
  RAI_REQUIRE(p.n_instr >= 1 && p.n_instr <= kFusedMaxInstr && p.n_leaves <= kFusedMaxLeaves, RAI_ERR_BAD_ARG,
              "fused region: %d instructions, %d leaves", p.n_instr, p.n_leaves);
  hipLaunchKernelGGL(k_fused_elementwise, dim3(grid_for(p.numel)), dim3(256), 0, st, p);
  return launch_check("fused_elementwise");
}

}  // namespace rai

using namespace rai;

#define LAUNCH_V(KERNEL, T, v, grid, stream, ...)                                             \
  do {                                                                                        \
    switch (v) {                                                                              \
      case 16: if constexpr (sizeof(T) == 1) { hipLaunchKernelGGL((KERNEL<T, 16>), dim3(grid), dim3(256), 0, stream, __VA_ARGS__); } break; \
      case 8: if constexpr (sizeof(T) <= 2) { hipLaunchKernelGGL((KERNEL<T, 8>), dim3(grid), dim3(256), 0, stream, __VA_ARGS__); } break; \
      case 4: if constexpr (sizeof(T) <= 4) { hipLaunchKernelGGL((KERNEL<T, 4>), dim3(grid), dim3(256), 0, stream, __VA_ARGS__); } break; \
      case 2: hipLaunchKernelGGL((KERNEL<T, 2>), dim3(grid), dim3(256), 0, stream, __VA_ARGS__); break; \
      default: hipLaunchKernelGGL((KERNEL<T, 1>), dim3(grid), dim3(256), 0, stream, __VA_ARGS__); break; \
    }                                                                                         \
  } while (0)

extern "C" {

int rai_hip_fill(int dev, const rai_hip_tensor *out, double value) {
  RAI_TRY(validate(out, "out"));
  RAI_REQUIRE(is_contiguous(out), RAI_ERR_BAD_STRIDE, "fill: out must be contiguous");
  hipStream_t st = stream_of(dev);
  if (!st) return RAI_ERR_HIP;
  int64_t n = numel(out);
  if (n == 0) return RAI_OK;
  RAI_DISPATCH_ALL(out->dtype, T,
                   hipLaunchKernelGGL((k_fill<T>), dim3(grid_for(n)), dim3(256), 0, st, (T *)base_ptr(out), n, value));
  return launch_check("fill");
}

int rai_hip_arange(int dev, const rai_hip_tensor *out, double start, double step) {
  RAI_TRY(validate(out, "out"));
  RAI_REQUIRE(is_contiguous(out), RAI_ERR_BAD_STRIDE, "arange: out must be contiguous");
  hipStream_t st = stream_of(dev);
  if (!st) return RAI_ERR_HIP;
  int64_t n = numel(out);
  if (n == 0) return RAI_OK;
  RAI_DISPATCH_ALL(out->dtype, T,
                   hipLaunchKernelGGL((k_arange<T>), dim3(grid_for(n)), dim3(256), 0, st, (T *)base_ptr(out), n, start,
                                      step));
  return launch_check("arange");
}

int rai_hip_copy(int dev, const rai_hip_tensor *in, const rai_hip_tensor *out) {
  RAI_TRY(validate(in, "in"));
  RAI_TRY(validate(out, "out"));
  RAI_REQUIRE(in->dtype == out->dtype, RAI_ERR_BAD_DTYPE, "copy: dtype mismatch %s vs %s", dtype_name(in->dtype),
              dtype_name(out->dtype));
  RAI_REQUIRE(same_shape(in, out), RAI_ERR_BAD_SHAPE, "copy: shape mismatch");
  hipStream_t st = stream_of(dev);
  if (!st) return RAI_ERR_HIP;
  if (numel(out) == 0) return RAI_OK;
  const rai_hip_tensor *ts[2] = {out, in};
  IterSpace s;
  int v;
  RAI_DISPATCH_ALL(out->dtype, T, {
    build_space(2, ts, max_pack<T>(), &s, &v);
    LAUNCH_V(k_copy, T, v, grid_for(s.n_packs), st, s, (T *)base_ptr(out), (const T *)base_ptr(in));
  });
  return launch_check("copy");
}

int rai_hip_unary(int dev, int op, const rai_hip_tensor *in, const rai_hip_tensor *out, double param) {
  RAI_TRY(validate(in, "in"));
  RAI_TRY(validate(out, "out"));
  RAI_REQUIRE(op >= 0 && op < RAI_UN_COUNT_, RAI_ERR_BAD_ARG, "unary: bad op %d", op);
  RAI_REQUIRE(in->dtype == out->dtype, RAI_ERR_BAD_DTYPE, "unary: dtype mismatch");
  RAI_REQUIRE(same_shape(in, out), RAI_ERR_BAD_SHAPE, "unary: shape mismatch");
  hipStream_t st = stream_of(dev);
  if (!st) return RAI_ERR_HIP;
  if (numel(out) == 0) return RAI_OK;
  const rai_hip_tensor *ts[2] = {out, in};
  IterSpace s;
  int v;
  RAI_DISPATCH_FLOAT(out->dtype, T, {
    build_space(2, ts, max_pack<T>(), &s, &v);
    LAUNCH_V(k_unary, T, v, grid_for(s.n_packs), st, s, (T *)base_ptr(out), (const T *)base_ptr(in), op, param);
  });
  return launch_check("unary");
}

int rai_hip_binary(int dev, int op, const rai_hip_tensor *lhs, const rai_hip_tensor *rhs, const rai_hip_tensor *out) {
  RAI_TRY(validate(lhs, "lhs"));
  RAI_TRY(validate(rhs, "rhs"));
  RAI_TRY(validate(out, "out"));
  RAI_REQUIRE(op >= 0 && op < RAI_BIN_COUNT_, RAI_ERR_BAD_ARG, "binary: bad op %d", op);
  RAI_REQUIRE(lhs->dtype == rhs->dtype, RAI_ERR_BAD_DTYPE, "binary: operand dtypes differ (%s, %s)",
              dtype_name(lhs->dtype), dtype_name(rhs->dtype));
  RAI_REQUIRE(same_shape(lhs, out) && same_shape(rhs, out), RAI_ERR_BAD_SHAPE,
              "binary: operands must be broadcast to the output shape");
  hipStream_t st = stream_of(dev);
  if (!st) return RAI_ERR_HIP;
  if (numel(out) == 0) return RAI_OK;
  const rai_hip_tensor *ts[3] = {out, lhs, rhs};
  IterSpace s;
  int v;
  if (op >= RAI_BIN_EQ) {
    RAI_REQUIRE(out->dtype == RAI_U8, RAI_ERR_BAD_DTYPE, "binary: comparison output must be u8");
    build_space(3, ts, 1, &s, &v);
    RAI_DISPATCH_ALL(lhs->dtype, T,
                     hipLaunchKernelGGL((k_compare<T>), dim3(grid_for(s.n_packs)), dim3(256), 0, st, s,
                                        (uint8_t *)base_ptr(out), (const T *)base_ptr(lhs), (const T *)base_ptr(rhs),
                                        op));
    return launch_check("compare");
  }
  RAI_REQUIRE(out->dtype == lhs->dtype, RAI_ERR_BAD_DTYPE, "binary: output dtype must equal operand dtype");
  RAI_DISPATCH_ALL(out->dtype, T, {
    build_space(3, ts, max_pack<T>(), &s, &v);
    LAUNCH_V(k_binary, T, v, grid_for(s.n_packs), st, s, (T *)base_ptr(out), (const T *)base_ptr(lhs),
             (const T *)base_ptr(rhs), op);
  });
  return launch_check("binary");
}

int rai_hip_where(int dev, const rai_hip_tensor *cond, const rai_hip_tensor *on_true, const rai_hip_tensor *on_false,
                  const rai_hip_tensor *out) {
  RAI_TRY(validate(cond, "cond"));
  RAI_TRY(validate(on_true, "on_true"));
  RAI_TRY(validate(on_false, "on_false"));
  RAI_TRY(validate(out, "out"));
  RAI_REQUIRE(on_true->dtype == out->dtype && on_false->dtype == out->dtype, RAI_ERR_BAD_DTYPE,
              "where: value dtypes must equal the output dtype");
  RAI_REQUIRE(cond->dtype == RAI_U8 || cond->dtype == RAI_U32 || cond->dtype == RAI_I64, RAI_ERR_BAD_DTYPE,
              "where: cond must be u8/u32/i64");
  RAI_REQUIRE(same_shape(cond, out) && same_shape(on_true, out) && same_shape(on_false, out), RAI_ERR_BAD_SHAPE,
              "where: operands must be broadcast to the output shape");
  hipStream_t st = stream_of(dev);
  if (!st) return RAI_ERR_HIP;
  if (numel(out) == 0) return RAI_OK;
  // No dim merging here: cond carries its own strides over the same (uncoalesced) space.
  IterSpace s;
  CondSpace cs;
  s.rank = out->rank > 0 ? out->rank : 1;
  int64_t total = 1;
  for (int i = 0; i < RAI_HIP_MAX_RANK; ++i) {
    bool in = i < out->rank;
    s.shape[i] = in ? out->shape[i] : 1;
    s.stride[0][i] = in ? out->stride[i] : 0;
    s.stride[1][i] = in ? on_true->stride[i] : 0;
    s.stride[2][i] = in ? on_false->stride[i] : 0;
    cs.stride[i] = in ? cond->stride[i] : 0;
    total *= s.shape[i];
  }
  s.n_packs = total;
  int grid = grid_for(total);
#define WHERE_LAUNCH(T, CT)                                                                                        \
  hipLaunchKernelGGL((k_where<T, CT>), dim3(grid), dim3(256), 0, st, s, cs, (T *)base_ptr(out),                    \
                     (const T *)base_ptr(on_true), (const T *)base_ptr(on_false), (const CT *)base_ptr(cond))
  RAI_DISPATCH_ALL(out->dtype, T, {
    if (cond->dtype == RAI_U8) WHERE_LAUNCH(T, uint8_t);
    else if (cond->dtype == RAI_U32) WHERE_LAUNCH(T, uint32_t);
    else WHERE_LAUNCH(T, int64_t);
  });
#undef WHERE_LAUNCH
  return launch_check("where");
}

int rai_hip_cast(int dev, const rai_hip_tensor *in, const rai_hip_tensor *out) {
  RAI_TRY(validate(in, "in"));
  RAI_TRY(validate(out, "out"));
  RAI_REQUIRE(same_shape(in, out), RAI_ERR_BAD_SHAPE, "cast: shape mismatch");
  if (in->dtype == out->dtype) return rai_hip_copy(dev, in, out);
  hipStream_t st = stream_of(dev);
  if (!st) return RAI_ERR_HIP;
  if (numel(out) == 0) return RAI_OK;
  const rai_hip_tensor *ts[2] = {out, in};
  IterSpace s;
  int v;
  build_space(2, ts, 1, &s, &v);
  int grid = grid_for(s.n_packs);
  RAI_DISPATCH_ALL(out->dtype, D, {
    RAI_DISPATCH_ALL(in->dtype, S,
                     hipLaunchKernelGGL((k_cast<D, S>), dim3(grid), dim3(256), 0, st, s, (D *)base_ptr(out),
                                        (const S *)base_ptr(in)));
  });
  return launch_check("cast");
}

}  // extern "C"
