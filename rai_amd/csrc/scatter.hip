// gather / index_add / scatter_add along one dimension: the primitives the reference's vjp rules of
// index_select, gather and scatter_add evaluate (rai-core/src/ops/index_select.rs:40-48,
// ops/gather.rs:36-43, ops/scatter_add.rs:36-50).  Reference evaluation:
// rai-core/src/backend/candle.rs:838-849 (Gather), :851-865 (IndexAdd), :990-1004 (ScatterAdd).
//
// The two additions are written as "pull" kernels wherever that is affordable: every output element
// collects its own contributions in increasing source order and rounds to the storage dtype after
// each addition, so the result equals a sequential host loop bit for bit, duplicates included, and no
// floating-point atomics (whose order varies from run to run) are used.
#include <algorithm>

#include "common.h"

namespace rai {

template <typename T>
__device__ __forceinline__ typename Scalar<T>::compute add_rounded(typename Scalar<T>::compute a,
                                                                   typename Scalar<T>::compute b) {
  T t;
  Scalar<T>::store(&t, a + b);
  return Scalar<T>::load(&t);
}

// x [outer, D, inner], index / out [outer, J, inner], all contiguous: out[o, j, i] = x[o, index[o, j, i], i].
template <typename T, typename IT>
__global__ void __launch_bounds__(256)
k_gather(T *out, const T *x, const IT *index, int64_t outer, int64_t J, int64_t D, int64_t inner,
         unsigned long long *errors) {
  const int64_t total = outer * J * inner;
  for (int64_t e = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; e < total; e += (int64_t)gridDim.x * blockDim.x) {
    const int64_t row = e / inner, i = e - row * inner, o = row / J;
    const int64_t id = (int64_t)index[e];
    if (id < 0 || id >= D) {
      atomicAdd(errors, 1ull);
      memset(&out[e], 0, sizeof(T));
      continue;
    }
    out[e] = x[(o * D + id) * inner + i];
  }
}

// x / out [outer, D, inner], source [outer, L, inner], index [L]: out[o, r, :] = x[o, r, :] + the rows
// source[o, l, :] with index[l] == r, added in increasing l.  One wave per output row (grid-stride): it
// scans the index list 64 entries at a time (one per lane, from an LDS copy when the list fits) and
// walks the ballot mask of the matches in order.  A row is moved in units of U: 16-byte packs when the
// row length and the addresses allow, single elements otherwise; kIndexAddUnits of them per lane and pass.
constexpr int kIndexAddUnits = 8;
constexpr int kIndexAddLdsEntries = 32768;   // 128 KB of staged indices
template <typename T> struct alignas(16) Pack16 { T v[16 / sizeof(T)]; };
template <typename T> __device__ __forceinline__ void add_unit(T &acc, const T &s) {
  Scalar<T>::store(&acc, Scalar<T>::load(&acc) + Scalar<T>::load(&s));
}
template <typename T> __device__ __forceinline__ void add_unit(Pack16<T> &acc, const Pack16<T> &s) {
#pragma unroll
  for (int j = 0; j < (int)(16 / sizeof(T)); ++j) Scalar<T>::store(&acc.v[j], Scalar<T>::load(&acc.v[j]) + Scalar<T>::load(&s.v[j]));
}
template <typename U, typename IT>
__global__ void __launch_bounds__(256)
k_index_add(U *out, const U *x, const U *source, const IT *index, int64_t index_stride, int64_t outer, int64_t D,
            int64_t L, int64_t units, int staged, unsigned long long *errors) {
  extern __shared__ int32_t s_idx[];
  if (staged) {   // ids outside [0, D) can match no row: stored as -1
    for (int64_t l = threadIdx.x; l < L; l += blockDim.x) {
      const int64_t id = (int64_t)index[l * index_stride];
      const bool ok = id >= 0 && id < D;
      s_idx[l] = ok ? (int32_t)id : -1;
      if (!ok && blockIdx.x == 0) atomicAdd(errors, 1ull);
    }
    __syncthreads();
  } else if (blockIdx.x == 0) {
    for (int64_t l = threadIdx.x; l < L; l += blockDim.x) {
      const int64_t id = (int64_t)index[l * index_stride];
      if (id < 0 || id >= D) atomicAdd(errors, 1ull);
    }
  }
  const int lane = threadIdx.x & 63;
  const int64_t rows = outer * D, n_waves = (int64_t)gridDim.x * 4;
  for (int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); row < rows; row += n_waves) {
    const int64_t o = row / D, r = row - o * D;
    for (int64_t i0 = 0; i0 < units; i0 += 64 * kIndexAddUnits) {
      U acc[kIndexAddUnits];
#pragma unroll
      for (int u = 0; u < kIndexAddUnits; ++u) {
        const int64_t i = i0 + u * 64 + lane;
        if (i < units) acc[u] = x[row * units + i];
      }
      for (int64_t l0 = 0; l0 < L; l0 += 64) {
        const int64_t l = l0 + lane;
        int64_t id = -1;
        if (l < L) id = staged ? (int64_t)s_idx[l] : (int64_t)index[l * index_stride];
        unsigned long long m = __ballot(id == r);
        while (m) {
          const int b = __ffsll((long long)m) - 1;
          m &= m - 1;
          const U *srow = source + (o * L + l0 + b) * units;
#pragma unroll
          for (int u = 0; u < kIndexAddUnits; ++u) {
            const int64_t i = i0 + u * 64 + lane;
            if (i < units) add_unit(acc[u], srow[i]);
          }
        }
      }
#pragma unroll
      for (int u = 0; u < kIndexAddUnits; ++u) {
        const int64_t i = i0 + u * 64 + lane;
        if (i < units) out[row * units + i] = acc[u];
      }
    }
  }
}

// x / out [outer, D, inner], index / source [outer, J, inner]:
// out[o, r, i] = x[o, r, i] + the source[o, j, i] with index[o, j, i] == r, added in increasing j.
// Pull form (short J): one thread per output element scans its column of indices.
template <typename T, typename IT>
__global__ void __launch_bounds__(256)
k_scatter_add_pull(T *out, const T *x, const T *source, const IT *index, int64_t outer, int64_t D, int64_t J,
                   int64_t inner, unsigned long long *errors) {
  typedef typename Scalar<T>::compute CT;
  const int64_t total = outer * D * inner;
  for (int64_t e = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; e < total; e += (int64_t)gridDim.x * blockDim.x) {
    const int64_t row = e / inner, i = e - row * inner, o = row / D, r = row - o * D;
    CT acc = Scalar<T>::load(x + e);
    for (int64_t j = 0; j < J; ++j) {
      const int64_t s = (o * J + j) * inner + i;
      const int64_t id = (int64_t)index[s];
      if (r == 0 && (id < 0 || id >= D)) atomicAdd(errors, 1ull);
      if (id == r) acc = add_rounded<T>(acc, Scalar<T>::load(source + s));
    }
    Scalar<T>::store(out + e, acc);
  }
}
// Push form (long J): out already holds a copy of x; one thread per (o, i) column walks j in order, so
// no two threads touch the same output element.
template <typename T, typename IT>
__global__ void __launch_bounds__(256)
k_scatter_add_push(T *out, const T *source, const IT *index, int64_t outer, int64_t D, int64_t J, int64_t inner,
                   unsigned long long *errors) {
  const int64_t cols = outer * inner;
  for (int64_t c = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; c < cols; c += (int64_t)gridDim.x * blockDim.x) {
    const int64_t o = c / inner, i = c - o * inner;
    for (int64_t j = 0; j < J; ++j) {
      const int64_t s = (o * J + j) * inner + i;
      const int64_t id = (int64_t)index[s];
      if (id < 0 || id >= D) { atomicAdd(errors, 1ull); continue; }
      T *p = out + (o * D + id) * inner + i;
      Scalar<T>::store(p, add_rounded<T>(Scalar<T>::load(p), Scalar<T>::load(source + s)));
    }
  }
}

static int grid_for(int64_t work_items, int per_block) {
  int64_t blocks = (work_items + per_block - 1) / per_block;
  if (blocks < 1) blocks = 1;
  return (int)(blocks < (int64_t)kNumCU * 32 ? blocks : (int64_t)kNumCU * 32);
}

// Splits t's shape around `d` into [outer, t.shape[d], inner].
static void split_dims(const rai_hip_tensor *t, int d, int64_t *outer, int64_t *inner) {
  *outer = *inner = 1;
  for (int i = 0; i < d; ++i) *outer *= t->shape[i];
  for (int i = d + 1; i < t->rank; ++i) *inner *= t->shape[i];
}

static bool index_dtype_ok(int dt) { return dt == RAI_U8 || dt == RAI_U32 || dt == RAI_I64; }

#define RAI_DISPATCH_INDEX(dt, IT, ...)                       \
  switch (dt) {                                               \
    case RAI_U8: { typedef uint8_t IT; __VA_ARGS__; break; }   \
    case RAI_U32: { typedef uint32_t IT; __VA_ARGS__; break; } \
    default: { typedef int64_t IT; __VA_ARGS__; break; }       \
  }

}  // namespace rai

using namespace rai;

extern "C" {

int rai_hip_gather(int dev, const rai_hip_tensor *x, const rai_hip_tensor *index, int32_t dim, const rai_hip_tensor *out) {
  RAI_TRY(validate(x, "x"));
  RAI_TRY(validate(index, "index"));
  RAI_TRY(validate(out, "out"));
  RAI_REQUIRE(x->dtype == out->dtype, RAI_ERR_BAD_DTYPE, "gather: dtype mismatch");
  RAI_REQUIRE(index_dtype_ok(index->dtype), RAI_ERR_BAD_DTYPE, "gather: index must be u8/u32/i64, got %s", dtype_name(index->dtype));
  RAI_REQUIRE(x->rank >= 1 && index->rank == x->rank && same_shape(index, out), RAI_ERR_BAD_SHAPE,
              "gather: x and index need equal rank, out the shape of index");
  const int d = dim < 0 ? dim + x->rank : dim;
  RAI_REQUIRE(d >= 0 && d < x->rank, RAI_ERR_BAD_ARG, "gather: dim %d out of range for rank %d", dim, x->rank);
  for (int i = 0; i < x->rank; ++i)
    RAI_REQUIRE(i == d || index->shape[i] == x->shape[i], RAI_ERR_BAD_SHAPE, "gather: index.shape[%d]=%lld differs from x's %lld", i,
                (long long)index->shape[i], (long long)x->shape[i]);
  RAI_REQUIRE(is_contiguous(x) && is_contiguous(index) && is_contiguous(out), RAI_ERR_BAD_STRIDE, "gather: operands must be contiguous");
  hipStream_t st = stream_of(dev);
  if (!st) return RAI_ERR_HIP;
  if (numel(out) == 0) return RAI_OK;
  int64_t outer, inner;
  split_dims(x, d, &outer, &inner);
  const int64_t D = x->shape[d], J = index->shape[d];
  unsigned long long *errs = index_error_counter(dev);
  const int grid = grid_for(numel(out), 256);
  RAI_DISPATCH_ALL(x->dtype, T, {
    RAI_DISPATCH_INDEX(index->dtype, IT, {
      hipLaunchKernelGGL((k_gather<T, IT>), dim3(grid), dim3(256), 0, st, (T *)base_ptr(out), (const T *)base_ptr(x),
                         (const IT *)base_ptr(index), outer, J, D, inner, errs);
    });
  });
  return launch_check("gather");
}

int rai_hip_index_add(int dev, const rai_hip_tensor *x, const rai_hip_tensor *index, const rai_hip_tensor *source, int32_t dim,
                      const rai_hip_tensor *out) {
  RAI_TRY(validate(x, "x"));
  RAI_TRY(validate(index, "index"));
  RAI_TRY(validate(source, "source"));
  RAI_TRY(validate(out, "out"));
  RAI_REQUIRE(x->dtype == out->dtype && x->dtype == source->dtype, RAI_ERR_BAD_DTYPE, "index_add: dtype mismatch");
  RAI_REQUIRE(index_dtype_ok(index->dtype), RAI_ERR_BAD_DTYPE, "index_add: index must be u8/u32/i64, got %s", dtype_name(index->dtype));
  RAI_REQUIRE(index->rank == 1, RAI_ERR_BAD_SHAPE, "index_add: index must be rank 1");
  RAI_REQUIRE(x->rank >= 1 && source->rank == x->rank && same_shape(x, out), RAI_ERR_BAD_SHAPE,
              "index_add: x and source need equal rank, out the shape of x");
  const int d = dim < 0 ? dim + x->rank : dim;
  RAI_REQUIRE(d >= 0 && d < x->rank, RAI_ERR_BAD_ARG, "index_add: dim %d out of range for rank %d", dim, x->rank);
  const int64_t L = index->shape[0], D = x->shape[d];
  for (int i = 0; i < x->rank; ++i)
    RAI_REQUIRE(source->shape[i] == (i == d ? L : x->shape[i]), RAI_ERR_BAD_SHAPE, "index_add: source.shape[%d]=%lld unexpected", i,
                (long long)source->shape[i]);
  RAI_REQUIRE(is_contiguous(x) && is_contiguous(source) && is_contiguous(out), RAI_ERR_BAD_STRIDE,
              "index_add: x, source and out must be contiguous");
  hipStream_t st = stream_of(dev);
  if (!st) return RAI_ERR_HIP;
  if (numel(out) == 0) return RAI_OK;
  int64_t outer, inner;
  split_dims(x, d, &outer, &inner);
  unsigned long long *errs = index_error_counter(dev);
  const size_t es = dtype_size(x->dtype);
  const bool packs = (inner * es) % 16 == 0 && (uintptr_t)base_ptr(x) % 16 == 0 && (uintptr_t)base_ptr(source) % 16 == 0 &&
                     (uintptr_t)base_ptr(out) % 16 == 0;
  const int64_t units = packs ? inner * (int64_t)es / 16 : inner;
  const int staged = L <= kIndexAddLdsEntries && D <= 0x7fffffffLL ? 1 : 0;
  const size_t lds = staged ? (size_t)(L > 0 ? L : 1) * sizeof(int32_t) : 0;
  // one wave per row, four waves per block; few enough blocks that staging the index list stays cheap
  const int grid = std::min(grid_for(outer * D, 4), kNumCU * 8);
  RAI_DISPATCH_ALL(x->dtype, T, {
    RAI_DISPATCH_INDEX(index->dtype, IT, {
      if (packs) {
        if (lds > 48 * 1024)
          RAI_HIP_TRY(hipFuncSetAttribute((const void *)k_index_add<Pack16<T>, IT>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        hipLaunchKernelGGL((k_index_add<Pack16<T>, IT>), dim3(grid), dim3(256), lds, st, (Pack16<T> *)base_ptr(out),
                           (const Pack16<T> *)base_ptr(x), (const Pack16<T> *)base_ptr(source), (const IT *)base_ptr(index),
                           index->stride[0], outer, D, L, units, staged, errs);
      } else {
        if (lds > 48 * 1024)
          RAI_HIP_TRY(hipFuncSetAttribute((const void *)k_index_add<T, IT>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        hipLaunchKernelGGL((k_index_add<T, IT>), dim3(grid), dim3(256), lds, st, (T *)base_ptr(out), (const T *)base_ptr(x),
                           (const T *)base_ptr(source), (const IT *)base_ptr(index), index->stride[0], outer, D, L, units,
                           staged, errs);
      }
    });
  });
  return launch_check("index_add");
}

int rai_hip_scatter_add(int dev, const rai_hip_tensor *x, const rai_hip_tensor *index, const rai_hip_tensor *source, int32_t dim,
                        const rai_hip_tensor *out) {
  RAI_TRY(validate(x, "x"));
  RAI_TRY(validate(index, "index"));
  RAI_TRY(validate(source, "source"));
  RAI_TRY(validate(out, "out"));
  RAI_REQUIRE(x->dtype == out->dtype && x->dtype == source->dtype, RAI_ERR_BAD_DTYPE, "scatter_add: dtype mismatch");
  RAI_REQUIRE(index_dtype_ok(index->dtype), RAI_ERR_BAD_DTYPE, "scatter_add: index must be u8/u32/i64, got %s", dtype_name(index->dtype));
  RAI_REQUIRE(x->rank >= 1 && index->rank == x->rank && same_shape(index, source) && same_shape(x, out), RAI_ERR_BAD_SHAPE,
              "scatter_add: index and source need x's rank and one shape, out the shape of x");
  const int d = dim < 0 ? dim + x->rank : dim;
  RAI_REQUIRE(d >= 0 && d < x->rank, RAI_ERR_BAD_ARG, "scatter_add: dim %d out of range for rank %d", dim, x->rank);
  for (int i = 0; i < x->rank; ++i)
    RAI_REQUIRE(i == d || index->shape[i] == x->shape[i], RAI_ERR_BAD_SHAPE, "scatter_add: index.shape[%d]=%lld differs from x's %lld", i,
                (long long)index->shape[i], (long long)x->shape[i]);
  RAI_REQUIRE(is_contiguous(x) && is_contiguous(index) && is_contiguous(source) && is_contiguous(out), RAI_ERR_BAD_STRIDE,
              "scatter_add: operands must be contiguous");
  hipStream_t st = stream_of(dev);
  if (!st) return RAI_ERR_HIP;
  if (numel(out) == 0) return RAI_OK;
  int64_t outer, inner;
  split_dims(x, d, &outer, &inner);
  const int64_t D = x->shape[d], J = index->shape[d];
  unsigned long long *errs = index_error_counter(dev);
  const bool pull = J <= 32;
  if (!pull && base_ptr(out) != base_ptr(x))
    RAI_HIP_TRY(hipMemcpyAsync(base_ptr(out), base_ptr(x), (size_t)numel(x) * dtype_size(x->dtype), hipMemcpyDeviceToDevice, st));
  if (J == 0) {
    if (pull && base_ptr(out) != base_ptr(x))
      RAI_HIP_TRY(hipMemcpyAsync(base_ptr(out), base_ptr(x), (size_t)numel(x) * dtype_size(x->dtype), hipMemcpyDeviceToDevice, st));
    return RAI_OK;
  }
  RAI_DISPATCH_ALL(x->dtype, T, {
    RAI_DISPATCH_INDEX(index->dtype, IT, {
      if (pull)
        hipLaunchKernelGGL((k_scatter_add_pull<T, IT>), dim3(grid_for(numel(out), 256)), dim3(256), 0, st, (T *)base_ptr(out),
                           (const T *)base_ptr(x), (const T *)base_ptr(source), (const IT *)base_ptr(index), outer, D, J, inner, errs);
      else
        hipLaunchKernelGGL((k_scatter_add_push<T, IT>), dim3(grid_for(outer * inner, 256)), dim3(256), 0, st, (T *)base_ptr(out),
                           (const T *)base_ptr(source), (const IT *)base_ptr(index), outer, D, J, inner, errs);
    });
  });
  return launch_check("scatter_add");
}

}  // extern "C"
