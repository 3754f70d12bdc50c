// Internal helpers shared by the HIP translation units of librai_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>

#include "rai_hip.h"

namespace rai {

// ---------------------------------------------------------------- errors
void set_error(const char *fmt, ...);
int fail(int code, const char *fmt, ...);

#define RAI_HIP_TRY(expr)                                                                     \
  do {                                                                                        \
    hipError_t _e = (expr);                                                                   \
    if (_e != hipSuccess)                                                                     \
      return ::rai::fail(RAI_ERR_HIP, "%s:%d %s -> %s", __FILE__, __LINE__, #expr,            \
                         hipGetErrorString(_e));                                              \
  } while (0)

#define RAI_TRY(expr)        \
  do {                       \
    int _s = (expr);         \
    if (_s != RAI_OK) return _s; \
  } while (0)

#define RAI_REQUIRE(cond, code, ...)                  \
  do {                                                \
    if (!(cond)) return ::rai::fail(code, __VA_ARGS__); \
  } while (0)

// ---------------------------------------------------------------- device ctx
struct DeviceCtx;
// Returns nullptr (and sets the error) when dev is out of range or init fails.
DeviceCtx *ctx(int dev);
hipStream_t stream_of(int dev);
// The stream of an already initialised device; never creates a context (no allocation): nullptr + error otherwise.
hipStream_t stream_if_ready(int dev);
// Compute units of the device, asked of it once when its context is created (0 when the device cannot be set up).
int device_cu_count(int dev);
// Kernels that wait for other blocks bound their wait; one that gives up stores a RAI_FAULT_* code (system scope) to
// this word, which lives in pinned host memory, and every wave still exits normally.  The host looks at the word after
// each synchronisation of the device's stream (rai_hip_sync, rai_hip_d2h, the decoder's generate) and turns a
// non-zero code into RAI_ERR_HIP, clears it and resets the counters those kernels share.
int *kernel_fault_word(int dev);
int check_kernel_fault(int dev);
enum { RAI_FAULT_STREAMK = 1, RAI_FAULT_CHAIN = 2 };
// Zeroes the stream-K tile kernel's arrival counters on `st` (gemm_mfma.hip).
int streamk_counters_reset(int dev, hipStream_t st);
// Looks up this device's address of the fixed scratch array of the allocation-free argmax (reduce.hip); called once
// per device, with that device current, while its context is created.
int arg_static_scratch_init(int dev);
// First stage of an argmax over the last axis of contiguous [rows, n] (bf16, f16 or f32): the axis is cut into `splits`
// shares, and share s of row r leaves its best (value, index) under rai_hip_argmax's ordering in pval / pidx
// [r * splits + s] (a share of NaNs only leaves a NaN).  The caller merges the shares (reduce.hip).
int launch_argmax_partials(hipStream_t st, int dtype, const void *in, int64_t rows, int64_t n, int splits, float *pval,
                           uint32_t *pidx);
// Workspace that lives as long as the device context (grown on demand, never
// shrinks); used by kernels that need partial results.  Stream-ordered reuse.
int workspace(int dev, size_t bytes, void **out);
// Device counter bumped by gather kernels on an out-of-range index.
unsigned long long *index_error_counter(int dev);
int launch_check(const char *what);

// ---------------------------------------------------------------- dtypes
inline size_t dtype_size(int dt) {
  switch (dt) {
    case RAI_U8: return 1;
    case RAI_U32: return 4;
    case RAI_I64: return 8;
    case RAI_F16: return 2;
    case RAI_BF16: return 2;
    case RAI_F32: return 4;
    case RAI_F64: return 8;
    default: return 0;
  }
}
inline bool is_float(int dt) { return dt == RAI_F16 || dt == RAI_BF16 || dt == RAI_F32 || dt == RAI_F64; }
inline const char *dtype_name(int dt) {
  static const char *n[] = {"u8", "u32", "i64", "f16", "bf16", "f32", "f64"};
  return (dt >= 0 && dt <= 6) ? n[dt] : "?";
}

inline int64_t numel(const rai_hip_tensor *t) {
  int64_t n = 1;
  for (int i = 0; i < t->rank; ++i) n *= t->shape[i];
  return n;
}
inline bool is_contiguous(const rai_hip_tensor *t) {
  int64_t expect = 1;
  for (int i = t->rank - 1; i >= 0; --i) {
    if (t->shape[i] == 1) continue;
    if (t->stride[i] != expect) return false;
    expect *= t->shape[i];
  }
  return true;
}
inline bool same_shape(const rai_hip_tensor *a, const rai_hip_tensor *b) {
  if (a->rank != b->rank) return false;
  for (int i = 0; i < a->rank; ++i)
    if (a->shape[i] != b->shape[i]) return false;
  return true;
}
int validate(const rai_hip_tensor *t, const char *name);
inline char *base_ptr(const rai_hip_tensor *t) {
  return static_cast<char *>(t->data) + t->offset * (int64_t)dtype_size(t->dtype);
}

// A tensor view with dims merged where strides allow, for index decomposition on
// the device.  Up to three operands share one iteration space.
struct StridedArgs {
  int rank;
  int64_t shape[RAI_HIP_MAX_RANK];
  int64_t stride[3][RAI_HIP_MAX_RANK];
};
// Collapses the common iteration space of n (<=3) same-shape views.
void coalesce(int n, const rai_hip_tensor *const *ts, StridedArgs *out);

// ---------------------------------------------------------------- device-side scalar conversion
typedef __hip_bfloat16 bf16_t;
typedef __half f16_t;

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }
// round-to-nearest-even through the gfx950 conversion instruction (v_cvt_pk_bf16_f32)
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  return __builtin_bit_cast(uint16_t, (__bf16)f);
}
// two floats -> packed bf16 pair (lo in bits 0..15)
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  typedef __attribute__((ext_vector_type(2))) float f32x2_t;
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
  f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

template <typename T> struct Scalar;  // load/store through a compute type
template <> struct Scalar<float> {
  typedef float compute;
  static __device__ __forceinline__ float load(const float *p) { return *p; }
  static __device__ __forceinline__ void store(float *p, float v) { *p = v; }
};
template <> struct Scalar<double> {
  typedef double compute;
  static __device__ __forceinline__ double load(const double *p) { return *p; }
  static __device__ __forceinline__ void store(double *p, double v) { *p = v; }
};
struct bf16_raw { uint16_t bits; };
struct f16_raw { uint16_t bits; };
template <> struct Scalar<bf16_raw> {
  typedef float compute;
  static __device__ __forceinline__ float load(const bf16_raw *p) { return bf16_bits_to_f32(p->bits); }
  static __device__ __forceinline__ void store(bf16_raw *p, float v) { p->bits = f32_to_bf16_bits(v); }
};
template <> struct Scalar<f16_raw> {
  typedef float compute;
  static __device__ __forceinline__ float load(const f16_raw *p) {
    return __half2float(__ushort_as_half(p->bits));
  }
  static __device__ __forceinline__ void store(f16_raw *p, float v) {
    p->bits = __half_as_ushort(__float2half_rn(v));
  }
};
template <> struct Scalar<uint8_t> {
  typedef uint8_t compute;
  static __device__ __forceinline__ uint8_t load(const uint8_t *p) { return *p; }
  static __device__ __forceinline__ void store(uint8_t *p, uint8_t v) { *p = v; }
};
template <> struct Scalar<uint32_t> {
  typedef uint32_t compute;
  static __device__ __forceinline__ uint32_t load(const uint32_t *p) { return *p; }
  static __device__ __forceinline__ void store(uint32_t *p, uint32_t v) { *p = v; }
};
template <> struct Scalar<int64_t> {
  typedef int64_t compute;
  static __device__ __forceinline__ int64_t load(const int64_t *p) { return *p; }
  static __device__ __forceinline__ void store(int64_t *p, int64_t v) { *p = v; }
};

// Calls f(T{}) with the storage type matching a runtime dtype.
#define RAI_DISPATCH_ALL(dt, T, ...)                         \
  switch (dt) {                                              \
    case RAI_U8: { typedef uint8_t T; __VA_ARGS__; break; }   \
    case RAI_U32: { typedef uint32_t T; __VA_ARGS__; break; } \
    case RAI_I64: { typedef int64_t T; __VA_ARGS__; break; }  \
    case RAI_F16: { typedef ::rai::f16_raw T; __VA_ARGS__; break; }  \
    case RAI_BF16: { typedef ::rai::bf16_raw T; __VA_ARGS__; break; } \
    case RAI_F32: { typedef float T; __VA_ARGS__; break; }    \
    case RAI_F64: { typedef double T; __VA_ARGS__; break; }   \
    default: return ::rai::fail(RAI_ERR_BAD_DTYPE, "bad dtype %d", (int)(dt)); \
  }
#define RAI_DISPATCH_FLOAT(dt, T, ...)                       \
  switch (dt) {                                              \
    case RAI_F16: { typedef ::rai::f16_raw T; __VA_ARGS__; break; }  \
    case RAI_BF16: { typedef ::rai::bf16_raw T; __VA_ARGS__; break; } \
    case RAI_F32: { typedef float T; __VA_ARGS__; break; }    \
    case RAI_F64: { typedef double T; __VA_ARGS__; break; }   \
    default: return ::rai::fail(RAI_ERR_BAD_DTYPE, "float dtype required, got %s", ::rai::dtype_name(dt)); \
  }

// ---------------------------------------------------------------- wave helpers (wave64)
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

constexpr int kWave = 64;
constexpr int kNumCU = 256;

}  // namespace rai
