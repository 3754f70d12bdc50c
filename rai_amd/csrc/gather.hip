// index_select (embedding gather).  Pure HBM copy: every lane moves 16 bytes.
// Reference: rai-core/src/backend/candle.rs:867-878, ops/index_select.rs:52-61,
// rai-nn/src/embedding.rs:25-30.
#include "common.h"

namespace rai {

struct alignas(16) Bytes16 { uint32_t w[4]; };

// in is contiguous [outer, D, inner]; rows of `inner` elements are copied as
// 16-byte packs (inner_packs per row).  One pack per thread, grid-stride.
template <typename IT>
__global__ void __launch_bounds__(256)
k_index_select_vec(Bytes16 *out, const Bytes16 *in, const IT *index, int64_t index_stride, int64_t outer, int64_t L,
                   int64_t D, int64_t inner_packs, unsigned long long *errors) {
  const int64_t total = outer * L * inner_packs;
  if (total < ((int64_t)1 << 31)) {
    // 32-bit index arithmetic, four packs per thread with their index and data loads batched
    const uint32_t tot = (uint32_t)total, ipk = (uint32_t)inner_packs, Lu = (uint32_t)L;
    const uint32_t stride = gridDim.x * blockDim.x;
    for (uint32_t p0 = blockIdx.x * blockDim.x + threadIdx.x; p0 < tot; p0 += stride * 4) {
      uint32_t ip[4], o[4];
      int64_t id[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const uint32_t p = p0 + u * stride;
        const uint32_t row = (p < tot ? p : p0) / ipk;
        ip[u] = (p < tot ? p : p0) - row * ipk;
        o[u] = row / Lu;
        id[u] = (int64_t)index[(int64_t)(row - o[u] * Lu) * index_stride];
      }
      Bytes16 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        v[u] = Bytes16{{0u, 0u, 0u, 0u}};
        if (id[u] >= 0 && id[u] < D) v[u] = in[((int64_t)o[u] * D + id[u]) * inner_packs + ip[u]];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const uint32_t p = p0 + u * stride;
        if (p < tot) {
          if (!(id[u] >= 0 && id[u] < D) && ip[u] == 0) atomicAdd(errors, 1ull);
          out[p] = v[u];
        }
      }
    }
    return;
  }
  for (int64_t p = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; p < total; p += (int64_t)gridDim.x * blockDim.x) {
    int64_t row = p / inner_packs;
    int64_t ip = p - row * inner_packs;
    int64_t o = row / L;
    int64_t l = row - o * L;
    int64_t id = (int64_t)index[l * index_stride];
    Bytes16 v = {{0u, 0u, 0u, 0u}};
    if (id >= 0 && id < D) {
      v = in[(o * D + id) * inner_packs + ip];
    } else if (ip == 0) {
      atomicAdd(errors, 1ull);
    }
    out[p] = v;
  }
}

struct GatherSpace {
  int outer_rank, inner_rank;
  int64_t outer_shape[RAI_HIP_MAX_RANK], outer_stride[RAI_HIP_MAX_RANK];
  int64_t inner_shape[RAI_HIP_MAX_RANK], inner_stride[RAI_HIP_MAX_RANK];
  int64_t n_outer, n_inner, dim_stride;
};

template <typename T, typename IT>
__global__ void __launch_bounds__(256)
k_index_select_generic(T *out, const T *in, const IT *index, int64_t index_stride, GatherSpace s, int64_t L, int64_t D,
                       unsigned long long *errors) {
  const int64_t total = s.n_outer * L * s.n_inner;
  for (int64_t e = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; e < total; e += (int64_t)gridDim.x * blockDim.x) {
    int64_t row = e / s.n_inner;
    int64_t i = e - row * s.n_inner;
    int64_t o = row / L;
    int64_t l = row - o * L;
    int64_t id = (int64_t)index[l * index_stride];
    if (id < 0 || id >= D) {
      if (i == 0) atomicAdd(errors, 1ull);
      memset(&out[e], 0, sizeof(T));
      continue;
    }
    int64_t off = id * s.dim_stride;
    int64_t rem = o;
    for (int d = s.outer_rank - 1; d >= 0; --d) {
      int64_t q = rem / s.outer_shape[d];
      off += (rem - q * s.outer_shape[d]) * s.outer_stride[d];
      rem = q;
    }
    rem = i;
    for (int d = s.inner_rank - 1; d >= 0; --d) {
      int64_t q = rem / s.inner_shape[d];
      off += (rem - q * s.inner_shape[d]) * s.inner_stride[d];
      rem = q;
    }
    out[e] = in[off];
  }
}

}  // namespace rai

using namespace rai;

extern "C" int rai_hip_index_select(int dev, const rai_hip_tensor *in, const rai_hip_tensor *index, int32_t dim,
                                    const rai_hip_tensor *out) {
  RAI_TRY(validate(in, "in"));
  RAI_TRY(validate(index, "index"));
  RAI_TRY(validate(out, "out"));
  RAI_REQUIRE(in->dtype == out->dtype, RAI_ERR_BAD_DTYPE, "index_select: dtype mismatch");
  RAI_REQUIRE(index->dtype == RAI_U8 || index->dtype == RAI_U32 || index->dtype == RAI_I64, RAI_ERR_BAD_DTYPE,
              "index_select: index must be u8/u32/i64, got %s", dtype_name(index->dtype));
  RAI_REQUIRE(index->rank == 1, RAI_ERR_BAD_SHAPE, "index_select: index must be rank 1");
  int d = dim < 0 ? dim + in->rank : dim;
  RAI_REQUIRE(d >= 0 && d < in->rank, RAI_ERR_BAD_ARG, "index_select: dim %d out of range for rank %d", dim, in->rank);
  RAI_REQUIRE(out->rank == in->rank, RAI_ERR_BAD_SHAPE, "index_select: rank mismatch");
  const int64_t L = index->shape[0], D = in->shape[d];
  for (int i = 0; i < in->rank; ++i)
    RAI_REQUIRE(out->shape[i] == (i == d ? L : in->shape[i]), RAI_ERR_BAD_SHAPE,
                "index_select: out.shape[%d]=%lld unexpected", i, (long long)out->shape[i]);
  RAI_REQUIRE(is_contiguous(out), RAI_ERR_BAD_STRIDE, "index_select: output must be contiguous");
  hipStream_t st = stream_of(dev);
  if (!st) return RAI_ERR_HIP;
  if (numel(out) == 0) return RAI_OK;
  unsigned long long *errs = index_error_counter(dev);
  int64_t outer = 1, inner = 1;
  for (int i = 0; i < d; ++i) outer *= in->shape[i];
  for (int i = d + 1; i < in->rank; ++i) inner *= in->shape[i];
  const size_t es = dtype_size(in->dtype);
  const int64_t total = numel(out);

  bool vec = is_contiguous(in) && (inner * es) % 16 == 0 && (uintptr_t)base_ptr(in) % 16 == 0 &&
             (uintptr_t)base_ptr(out) % 16 == 0;
  if (vec) {
    int64_t inner_packs = inner * es / 16;
    int64_t work = outer * L * inner_packs;
    int64_t blocks = (work / 4 + 255) / 256;   // four packs per thread
    int grid = (int)(blocks < kNumCU * 32 ? (blocks < 1 ? 1 : blocks) : kNumCU * 32);
#define ISV(IT)                                                                                                   \
  hipLaunchKernelGGL((k_index_select_vec<IT>), dim3(grid), dim3(256), 0, st, (Bytes16 *)base_ptr(out),            \
                     (const Bytes16 *)base_ptr(in), (const IT *)base_ptr(index), index->stride[0], outer, L, D,   \
                     inner_packs, errs)
    if (index->dtype == RAI_U8) ISV(uint8_t);
    else if (index->dtype == RAI_U32) ISV(uint32_t);
    else ISV(int64_t);
#undef ISV
    return launch_check("index_select_vec");
  }
  GatherSpace s;
  s.outer_rank = s.inner_rank = 0;
  s.n_outer = outer;
  s.n_inner = inner;
  s.dim_stride = in->stride[d];
  for (int i = 0; i < d; ++i) {
    s.outer_shape[s.outer_rank] = in->shape[i];
    s.outer_stride[s.outer_rank++] = in->stride[i];
  }
  for (int i = d + 1; i < in->rank; ++i) {
    s.inner_shape[s.inner_rank] = in->shape[i];
    s.inner_stride[s.inner_rank++] = in->stride[i];
  }
  int64_t blocks = (total + 255) / 256;
  int grid = (int)(blocks < kNumCU * 32 ? blocks : kNumCU * 32);
#define ISG(T, IT)                                                                                                 \
  hipLaunchKernelGGL((k_index_select_generic<T, IT>), dim3(grid), dim3(256), 0, st, (T *)base_ptr(out),            \
                     (const T *)base_ptr(in), (const IT *)base_ptr(index), index->stride[0], s, L, D, errs)
  RAI_DISPATCH_ALL(in->dtype, T, {
    if (index->dtype == RAI_U8) ISG(T, uint8_t);
    else if (index->dtype == RAI_U32) ISG(T, uint32_t);
    else ISG(T, int64_t);
  });
#undef ISG
  return launch_check("index_select");
}
