// Reductions: sum/max/min over arbitrary axes, softmax / log-softmax along one
// axis, argmax / argmin along one axis.  HBM-bound; contiguous rows are read
// once with 16-byte accesses and reduced with wave64 shuffles.
//
// Reference semantics: rai-core/src/backend/candle.rs:475-523 (reduce),
// :793-843 (softmax, log_softmax chains), :917-944 (argmax; argmin there calls
// argmax by mistake — not reproduced).
#include <cfloat>

#include "common.h"

namespace rai {

// ---------------------------------------------------------------- generic reduce
struct ReduceSpace {
  int out_rank, red_rank;
  int64_t out_shape[RAI_HIP_MAX_RANK], out_stride[RAI_HIP_MAX_RANK];  // strides into `in`
  int64_t red_shape[RAI_HIP_MAX_RANK], red_stride[RAI_HIP_MAX_RANK];
  int64_t n_out, n_red;
};

__device__ __forceinline__ int64_t space_offset(const int64_t *shape, const int64_t *stride, int rank, int64_t lin) {
  int64_t off = 0;
  for (int d = rank - 1; d >= 0; --d) {
    int64_t q = lin / shape[d];
    off += (lin - q * shape[d]) * stride[d];
    lin = q;
  }
  return off;
}

template <typename C> struct RedOp {
  static __device__ __forceinline__ C init(int op, C first) { return op == RAI_RED_SUM ? C(0) : first; }
  static __device__ __forceinline__ C apply(int op, C a, C b) {
    if (op == RAI_RED_SUM) return a + b;
    if (op == RAI_RED_MAX) return b > a ? b : a;
    return b < a ? b : a;
  }
};

template <typename C> __device__ __forceinline__ C shfl_xor_c(C v, int o) { return __shfl_xor(v, o, 64); }
template <> __device__ __forceinline__ uint8_t shfl_xor_c<uint8_t>(uint8_t v, int o) {
  return (uint8_t)__shfl_xor((int)v, o, 64);
}
template <> __device__ __forceinline__ int64_t shfl_xor_c<int64_t>(int64_t v, int o) {
  return (int64_t)__shfl_xor((long long)v, o, 64);
}
template <> __device__ __forceinline__ uint32_t shfl_xor_c<uint32_t>(uint32_t v, int o) {
  return (uint32_t)__shfl_xor((int)v, o, 64);
}

// One 256-thread block per output element; the reduce space is walked with a
// block-stride loop (coalesced when its innermost stride is 1).
template <typename T>
__global__ void __launch_bounds__(256) k_reduce_block(ReduceSpace s, T *out, const T *in, int op) {
  typedef typename Scalar<T>::compute C;
  __shared__ C part[4];
  for (int64_t o = blockIdx.x; o < s.n_out; o += gridDim.x) {
    const T *base = in + space_offset(s.out_shape, s.out_stride, s.out_rank, o);
    C first = Scalar<T>::load(base);
    C acc = RedOp<C>::init(op, first);
    for (int64_t r = threadIdx.x; r < s.n_red; r += blockDim.x) {
      int64_t off = s.red_rank == 1 ? r * s.red_stride[0] : space_offset(s.red_shape, s.red_stride, s.red_rank, r);
      acc = RedOp<C>::apply(op, acc, Scalar<T>::load(base + off));
    }
#pragma unroll
    for (int w = 32; w > 0; w >>= 1) acc = RedOp<C>::apply(op, acc, shfl_xor_c<C>(acc, w));
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
      C r = part[0];
      for (int w = 1; w < 4; ++w) r = RedOp<C>::apply(op, r, part[w]);
      Scalar<T>::store(out + o, r);
    }
    __syncthreads();
  }
}

// One thread per output element, sequential walk over the reduce space: used
// when the kept innermost axis is the contiguous one (e.g. sum over dim 0).
template <typename T>
__global__ void __launch_bounds__(256) k_reduce_thread(ReduceSpace s, T *out, const T *in, int op) {
  typedef typename Scalar<T>::compute C;
  for (int64_t o = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; o < s.n_out;
       o += (int64_t)gridDim.x * blockDim.x) {
    const T *base = in + space_offset(s.out_shape, s.out_stride, s.out_rank, o);
    C acc = RedOp<C>::init(op, Scalar<T>::load(base));
    for (int64_t r = 0; r < s.n_red; ++r) {
      int64_t off = s.red_rank == 1 ? r * s.red_stride[0] : space_offset(s.red_shape, s.red_stride, s.red_rank, r);
      acc = RedOp<C>::apply(op, acc, Scalar<T>::load(base + off));
    }
    Scalar<T>::store(out + o, acc);
  }
}

// ---------------------------------------------------------------- softmax
// Row-major rows of length n with unit stride.  Each thread keeps up to
// ITEMS*V values in registers, so the row is read exactly once.
template <typename T, int V> struct alignas(sizeof(T) * V) RowPack { T v[V]; };

__device__ __forceinline__ float block_reduce_max(float v, float *sh) {
  v = wave_max(v);
  int w = threadIdx.x >> 6, nw = blockDim.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) sh[w] = v;
  __syncthreads();
  float r = sh[0];
  for (int i = 1; i < nw; ++i) r = fmaxf(r, sh[i]);
  return r;
}
__device__ __forceinline__ float block_reduce_sum(float v, float *sh) {
  v = wave_sum(v);
  int w = threadIdx.x >> 6, nw = blockDim.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) sh[w] = v;
  __syncthreads();
  float r = 0.f;
  for (int i = 0; i < nw; ++i) r += sh[i];
  return r;
}

template <typename T, int V, int ITEMS, bool LOG>
__global__ void __launch_bounds__(256) k_softmax_row(T *out, const T *in, int64_t rows, int64_t n, int64_t in_row_stride) {
  __shared__ float sh[4];
  const int64_t packs = n / V;
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const T *x = in + row * in_row_stride;
    T *y = out + row * n;
    float vals[ITEMS][V];
    float m = -INFINITY;
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
      int64_t p = threadIdx.x + (int64_t)it * 256;
      if (p < packs) {
        RowPack<T, V> pk = *reinterpret_cast<const RowPack<T, V> *>(x + p * V);
#pragma unroll
        for (int j = 0; j < V; ++j) {
          vals[it][j] = (float)Scalar<T>::load(&pk.v[j]);
          m = fmaxf(m, vals[it][j]);
        }
      }
    }
    m = block_reduce_max(m, sh);
    float sum = 0.f;
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
      int64_t p = threadIdx.x + (int64_t)it * 256;
      if (p < packs) {
#pragma unroll
        for (int j = 0; j < V; ++j) {
          float d = vals[it][j] - m;
          float e = expf(d);
          sum += e;
          vals[it][j] = LOG ? d : e;
        }
      }
    }
    sum = block_reduce_sum(sum, sh);
    const float inv = 1.0f / sum, lse = logf(sum);
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
      int64_t p = threadIdx.x + (int64_t)it * 256;
      if (p < packs) {
        RowPack<T, V> pk;
#pragma unroll
        for (int j = 0; j < V; ++j) Scalar<T>::store(&pk.v[j], LOG ? vals[it][j] - lse : vals[it][j] * inv);
        *reinterpret_cast<RowPack<T, V> *>(y + p * V) = pk;
      }
    }
  }
}

// The same with one row per wave (a block is four rows): every lane has all its 16-byte loads in flight at once and
// the two reductions are wave shuffles, with no LDS and no block barrier between the row's three phases.
template <typename T, int V, int ITEMS, bool LOG>
__global__ void __launch_bounds__(256) k_softmax_wave(T *out, const T *in, int64_t rows, int64_t n, int64_t in_row_stride) {
  const int lane = threadIdx.x & 63;
  const int64_t packs = n / V;
  for (int64_t row = blockIdx.x * 4 + (threadIdx.x >> 6); row < rows; row += (int64_t)gridDim.x * 4) {
    const T *x = in + row * in_row_stride;
    T *y = out + row * n;
    RowPack<T, V> pk[ITEMS];
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
      const int64_t p = lane + it * 64;
      if (p < packs) pk[it] = *reinterpret_cast<const RowPack<T, V> *>(x + p * V);
    }
    float vals[ITEMS][V];
    float m = -INFINITY;
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
      if (lane + it * 64 < packs) {
#pragma unroll
        for (int j = 0; j < V; ++j) {
          vals[it][j] = (float)Scalar<T>::load(&pk[it].v[j]);
          m = fmaxf(m, vals[it][j]);
        }
      }
    }
    m = wave_max(m);
    float sum = 0.f;
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
      if (lane + it * 64 < packs) {
#pragma unroll
        for (int j = 0; j < V; ++j) {
          const float d = vals[it][j] - m;
          const float e = expf(d);
          sum += e;
          vals[it][j] = LOG ? d : e;
        }
      }
    }
    sum = wave_sum(sum);
    const float inv = 1.0f / sum, lse = logf(sum);
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
      const int64_t p = lane + it * 64;
      if (p < packs) {
        RowPack<T, V> o;
#pragma unroll
        for (int j = 0; j < V; ++j) Scalar<T>::store(&o.v[j], LOG ? vals[it][j] - lse : vals[it][j] * inv);
        *reinterpret_cast<RowPack<T, V> *>(y + p * V) = o;
      }
    }
  }
}

// Any stride along the softmax axis, any row length; three passes over the row.
// One block per row when the axis is long, else one thread per row.
template <typename T, bool LOG>
__global__ void __launch_bounds__(256)
k_softmax_strided_block(T *out, const T *in, ReduceSpace s, int64_t axis_stride_in, int64_t axis_stride_out,
                        ReduceSpace so) {
  typedef typename Scalar<T>::compute C;
  __shared__ float sh[4];
  for (int64_t row = blockIdx.x; row < s.n_out; row += gridDim.x) {
    const T *x = in + space_offset(s.out_shape, s.out_stride, s.out_rank, row);
    T *y = out + space_offset(so.out_shape, so.out_stride, so.out_rank, row);
    float m = -INFINITY;
    for (int64_t i = threadIdx.x; i < s.n_red; i += blockDim.x) m = fmaxf(m, (float)Scalar<T>::load(x + i * axis_stride_in));
    m = block_reduce_max(m, sh);
    float sum = 0.f;
    for (int64_t i = threadIdx.x; i < s.n_red; i += blockDim.x) sum += expf((float)Scalar<T>::load(x + i * axis_stride_in) - m);
    sum = block_reduce_sum(sum, sh);
    const float inv = 1.0f / sum, lse = logf(sum);
    for (int64_t i = threadIdx.x; i < s.n_red; i += blockDim.x) {
      float d = (float)Scalar<T>::load(x + i * axis_stride_in) - m;
      Scalar<T>::store(y + i * axis_stride_out, (C)(LOG ? d - lse : expf(d) * inv));
    }
  }
}
template <typename T, bool LOG>
__global__ void __launch_bounds__(256)
k_softmax_strided_thread(T *out, const T *in, ReduceSpace s, int64_t axis_stride_in, int64_t axis_stride_out,
                         ReduceSpace so) {
  typedef typename Scalar<T>::compute C;
  for (int64_t row = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; row < s.n_out;
       row += (int64_t)gridDim.x * blockDim.x) {
    const T *x = in + space_offset(s.out_shape, s.out_stride, s.out_rank, row);
    T *y = out + space_offset(so.out_shape, so.out_stride, so.out_rank, row);
    C m = Scalar<T>::load(x);
    for (int64_t i = 1; i < s.n_red; ++i) {
      C v = Scalar<T>::load(x + i * axis_stride_in);
      m = v > m ? v : m;
    }
    C sum = 0;
    for (int64_t i = 0; i < s.n_red; ++i) sum += exp(Scalar<T>::load(x + i * axis_stride_in) - m);
    C lse = log(sum);
    for (int64_t i = 0; i < s.n_red; ++i) {
      C d = Scalar<T>::load(x + i * axis_stride_in) - m;
      Scalar<T>::store(y + i * axis_stride_out, LOG ? d - lse : exp(d) / sum);
    }
  }
}

// ---------------------------------------------------------------- argmax / argmin
// Ordering used by every stage: candidate b replaces a when b is strictly
// better, or equally good with a smaller index.  NaN is never better than
// anything; a NaN at index 0 wins (the sequential scan of the reference starts
// from element 0 and replaces only on a strict comparison), which is patched in
// by the final stage.
template <typename C, bool IS_MAX> __device__ __forceinline__ bool better(C bv, uint32_t bi, C av, uint32_t ai) {
  bool b_nan = bv != bv, a_nan = av != av;
  if (b_nan) return a_nan && bi < ai;
  if (a_nan) return true;
  if (IS_MAX ? (bv > av) : (bv < av)) return true;
  return bv == av && bi < ai;
}

// blockDim.x = 256 or 1024: the wider block where a row's share is long enough to give every thread several 16-byte
// loads, all of them in flight at once (one memory round trip for the share).
template <typename T, bool IS_MAX>
__global__ void __launch_bounds__(1024)
k_arg_row_partial(const T *in, int64_t rows, int64_t n, int64_t row_stride, int64_t axis_stride, int splits,
                  float *pval_f, double *pval_d, uint32_t *pidx, uint32_t *counters, uint32_t *out) {
  typedef typename Scalar<T>::compute C;
  __shared__ C shv[16];
  __shared__ uint32_t shi[16];
  int64_t row = blockIdx.x / splits;
  int split = blockIdx.x % splits;
  if (row >= rows) return;
  int64_t chunk = (n + splits - 1) / splits;
  int64_t lo = split * chunk, hi = lo + chunk < n ? lo + chunk : n;
  const T *x = in + row * row_stride;
  C bv = C(0);
  uint32_t bi = 0xffffffffu;
  bool have = false;
  constexpr int VEC = 16 / sizeof(T);
  if (axis_stride == 1 && lo % VEC == 0 && ((uintptr_t)(x + lo) & 15) == 0) {
    // unit-stride axis: 16-byte loads, four per thread in flight, elements still visited in index order
    struct alignas(16) Pack { T v[VEC]; };
    const Pack *xp = reinterpret_cast<const Pack *>(x + lo);
    const int64_t chunks = (hi - lo) / VEC;
    for (int64_t c0 = threadIdx.x; c0 < chunks; c0 += (int64_t)blockDim.x * 4) {
      Pack pk[4];
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (c0 + (int64_t)u * blockDim.x < chunks) pk[u] = xp[c0 + (int64_t)u * blockDim.x];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t c = c0 + (int64_t)u * blockDim.x;
        if (c < chunks) {
#pragma unroll
          for (int j = 0; j < VEC; ++j) {
            const C v = Scalar<T>::load(&pk[u].v[j]);
            const uint32_t i = (uint32_t)(lo + c * VEC + j);
            if (!have || better<C, IS_MAX>(v, i, bv, bi)) { bv = v; bi = i; have = true; }
          }
        }
      }
    }
    for (int64_t i = lo + chunks * VEC + threadIdx.x; i < hi; i += blockDim.x) {  // tail shorter than one pack
      C v = Scalar<T>::load(x + i);
      if (!have || better<C, IS_MAX>(v, (uint32_t)i, bv, bi)) { bv = v; bi = (uint32_t)i; have = true; }
    }
  } else {
    for (int64_t i = lo + threadIdx.x; i < hi; i += blockDim.x) {
      C v = Scalar<T>::load(x + i * axis_stride);
      if (!have || better<C, IS_MAX>(v, (uint32_t)i, bv, bi)) {
        bv = v;
        bi = (uint32_t)i;
        have = true;
      }
    }
  }
  // Lanes that saw nothing carry index 0xffffffff and a NaN so they never win.
  if (!have) bv = C(NAN);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    C ov = shfl_xor_c<C>(bv, o);
    uint32_t oi = (uint32_t)__shfl_xor((int)bi, o, 64);
    if (better<C, IS_MAX>(ov, oi, bv, bi)) { bv = ov; bi = oi; }
  }
  if ((threadIdx.x & 63) == 0) { shv[threadIdx.x >> 6] = bv; shi[threadIdx.x >> 6] = bi; }
  __syncthreads();
  if (threadIdx.x >= 64) return;   // wave 0 finishes the block
  if (threadIdx.x == 0) {
    const int nw = (int)(blockDim.x >> 6);
    for (int w = 1; w < nw; ++w)
      if (better<C, IS_MAX>(shv[w], shi[w], bv, bi)) { bv = shv[w]; bi = shi[w]; }
  }
  if (!out) {   // two-launch form: k_arg_row_final merges
    if (threadIdx.x == 0) {
      if (sizeof(C) == 8) pval_d[blockIdx.x] = (double)bv; else pval_f[blockIdx.x] = (float)bv;
      pidx[blockIdx.x] = bi;
    }
    return;
  }
  // One-launch form: the block of a row that arrives last merges the row's partial results.  They cross blocks
  // (and XCDs, whose L2s are not coherent for ordinary accesses) as device-scope relaxed atomics, which write
  // through / read around the L2; the arrival counter is bumped only after this block's stores have completed,
  // and the last block sets it back to zero for the next call.  The merge is one memory round trip: every lane of
  // the wave fetches one split's result, then the lanes are reduced with the same ordering.
  if (splits > 1) {
    int last = 0;
    if (threadIdx.x == 0) {
      if (sizeof(C) == 8) __hip_atomic_store(&pval_d[blockIdx.x], (double)bv, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      else __hip_atomic_store(&pval_f[blockIdx.x], (float)bv, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(&pidx[blockIdx.x], bi, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      last = atomicAdd(&counters[row], 1u) == (uint32_t)splits - 1u;
    }
    if (!__shfl(last, 0, 64)) return;
    const int64_t base = row * splits;
    bool got = false;
    bv = C(NAN);
    bi = 0xffffffffu;
    for (int sp = threadIdx.x; sp < splits; sp += 64) {
      C v;
      if (sizeof(C) == 8) v = (C)__hip_atomic_load(&pval_d[base + sp], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      else v = (C)__hip_atomic_load(&pval_f[base + sp], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const uint32_t i = __hip_atomic_load(&pidx[base + sp], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (!got || better<C, IS_MAX>(v, i, bv, bi)) { bv = v; bi = i; got = true; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      C ov = shfl_xor_c<C>(bv, o);
      uint32_t oi = (uint32_t)__shfl_xor((int)bi, o, 64);
      if (better<C, IS_MAX>(ov, oi, bv, bi)) { bv = ov; bi = oi; }
    }
    if (threadIdx.x == 0) __hip_atomic_store(&counters[row], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  if (threadIdx.x == 0) {
    // all-NaN row: every candidate is NaN and index 0 wins already; a NaN at element 0 wins in the reference's
    // sequential scan even with finite values elsewhere
    const C first = Scalar<T>::load(x);
    out[row] = (bi == 0xffffffffu || first != first) ? 0u : bi;
  }
}

template <typename T, typename C, bool IS_MAX>
__global__ void __launch_bounds__(64)
k_arg_row_final(const C *pval, const uint32_t *pidx, int64_t rows, int splits, uint32_t *out, const T *in,
                int64_t row_stride) {
  int64_t row = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  if (row >= rows) return;
  C bv = pval[row * splits];
  uint32_t bi = pidx[row * splits];
  for (int s = 1; s < splits; ++s) {
    C v = pval[row * splits + s];
    uint32_t i = pidx[row * splits + s];
    if (better<C, IS_MAX>(v, i, bv, bi)) { bv = v; bi = i; }
  }
  // all-NaN row: every candidate is NaN and the smallest index (0) wins already;
  // NaN at element 0 wins in the reference's sequential scan even with finite values elsewhere
  const typename Scalar<T>::compute first = Scalar<T>::load(in + row * row_stride);
  out[row] = (bi == 0xffffffffu || first != first) ? 0u : bi;
}

// Generic strided variant: one thread per output, sequential scan like the reference.
template <typename T, bool IS_MAX>
__global__ void __launch_bounds__(256) k_arg_thread(const T *in, ReduceSpace s, int64_t axis_stride, uint32_t *out) {
  typedef typename Scalar<T>::compute C;
  for (int64_t o = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; o < s.n_out;
       o += (int64_t)gridDim.x * blockDim.x) {
    const T *x = in + space_offset(s.out_shape, s.out_stride, s.out_rank, o);
    C bv = Scalar<T>::load(x);
    uint32_t bi = 0;
    for (int64_t i = 1; i < s.n_red; ++i) {
      C v = Scalar<T>::load(x + i * axis_stride);
      if (IS_MAX ? (v > bv) : (v < bv)) { bv = v; bi = (uint32_t)i; }
    }
    out[o] = bi;
  }
}

// ---------------------------------------------------------------- host helpers
static int build_reduce_space(const rai_hip_tensor *in, const bool *reduced, ReduceSpace *s) {
  s->out_rank = s->red_rank = 0;
  s->n_out = s->n_red = 1;
  for (int i = 0; i < in->rank; ++i) {
    if (reduced[i]) {
      if (in->shape[i] == 1) continue;
      // merge with previous reduced dim when contiguous with it
      if (s->red_rank > 0 && s->red_stride[s->red_rank - 1] == in->stride[i] * in->shape[i] && i > 0 && reduced[i - 1]) {
        s->red_shape[s->red_rank - 1] *= in->shape[i];
        s->red_stride[s->red_rank - 1] = in->stride[i];
      } else {
        s->red_shape[s->red_rank] = in->shape[i];
        s->red_stride[s->red_rank] = in->stride[i];
        s->red_rank++;
      }
      s->n_red *= in->shape[i];
    } else {
      if (in->shape[i] == 1) continue;
      s->out_shape[s->out_rank] = in->shape[i];
      s->out_stride[s->out_rank] = in->stride[i];
      s->out_rank++;
      s->n_out *= in->shape[i];
    }
  }
  if (s->red_rank == 0) { s->red_rank = 1; s->red_shape[0] = 1; s->red_stride[0] = 1; }
  if (s->out_rank == 0) { s->out_rank = 1; s->out_shape[0] = 1; s->out_stride[0] = 0; }
  for (int i = s->red_rank; i < RAI_HIP_MAX_RANK; ++i) { s->red_shape[i] = 1; s->red_stride[i] = 0; }
  for (int i = s->out_rank; i < RAI_HIP_MAX_RANK; ++i) { s->out_shape[i] = 1; s->out_stride[i] = 0; }
  return RAI_OK;
}

static int check_reduced_shape(const rai_hip_tensor *in, const bool *reduced, int keep_dim, const rai_hip_tensor *out,
                               const char *what) {
  int64_t expect[RAI_HIP_MAX_RANK];
  int r = 0;
  for (int i = 0; i < in->rank; ++i) {
    if (reduced[i]) {
      if (keep_dim) expect[r++] = 1;
    } else {
      expect[r++] = in->shape[i];
    }
  }
  if (out->rank != r) return fail(RAI_ERR_BAD_SHAPE, "%s: output rank %d, expected %d", what, out->rank, r);
  for (int i = 0; i < r; ++i)
    if (out->shape[i] != expect[i])
      return fail(RAI_ERR_BAD_SHAPE, "%s: output shape[%d]=%lld, expected %lld", what, i, (long long)out->shape[i],
                  (long long)expect[i]);
  if (!is_contiguous(out)) return fail(RAI_ERR_BAD_STRIDE, "%s: output must be contiguous", what);
  return RAI_OK;
}

static int norm_dim(int dim, int rank) { return dim < 0 ? dim + rank : dim; }

template <bool LOG> static int softmax_impl(int dev, const rai_hip_tensor *in, int32_t dim, const rai_hip_tensor *out) {
  RAI_TRY(validate(in, "in"));
  RAI_TRY(validate(out, "out"));
  RAI_REQUIRE(in->dtype == out->dtype, RAI_ERR_BAD_DTYPE, "softmax: dtype mismatch");
  RAI_REQUIRE(is_float(in->dtype), RAI_ERR_BAD_DTYPE, "softmax: float dtype required");
  RAI_REQUIRE(same_shape(in, out), RAI_ERR_BAD_SHAPE, "softmax: shape mismatch");
  RAI_REQUIRE(is_contiguous(out), RAI_ERR_BAD_STRIDE, "softmax: output must be contiguous");
  int d = norm_dim(dim, in->rank);
  RAI_REQUIRE(d >= 0 && d < in->rank, RAI_ERR_BAD_ARG, "softmax: dim %d out of range for rank %d", dim, in->rank);
  hipStream_t st = stream_of(dev);
  if (!st) return RAI_ERR_HIP;
  if (numel(out) == 0) return RAI_OK;
  bool reduced[RAI_HIP_MAX_RANK] = {false};
  reduced[d] = true;
  ReduceSpace si, so;
  build_reduce_space(in, reduced, &si);
  build_reduce_space(out, reduced, &so);
  const int64_t n = in->shape[d];
  si.n_red = so.n_red = n;
  const int64_t ax_in = in->stride[d], ax_out = out->stride[d];
  // Fast path: softmax over a unit-stride axis whose rows are laid out with one
  // uniform row stride (the outer dims collapse to a single dim).
  bool last = (d == in->rank - 1) && (ax_in == 1 || n == 1);
  if (last && in->dtype != RAI_F64) {
    rai_hip_tensor rows_view = *in;
    rows_view.rank = in->rank - 1;
    const rai_hip_tensor *ts[1] = {&rows_view};
    StridedArgs ca;
    coalesce(1, ts, &ca);
    if (ca.rank == 1) {
      int64_t rows = si.n_out, row_stride = rows == 1 ? n : ca.stride[0][0];
      size_t es = dtype_size(in->dtype);
      int v = (int)(16 / es);
      bool aligned = (n % v == 0) && (row_stride % v == 0) && ((uintptr_t)base_ptr(in) % 16 == 0) &&
                     ((uintptr_t)base_ptr(out) % 16 == 0);
      int64_t packs = aligned ? n / v : n;
      int grid = (int)(rows < kNumCU * 32 ? rows : kNumCU * 32);
#define SM_LAUNCH(T, V, ITEMS)                                                                               \
  hipLaunchKernelGGL((k_softmax_row<T, V, ITEMS, LOG>), dim3(grid), dim3(256), 0, st, (T *)base_ptr(out),    \
                     (const T *)base_ptr(in), rows, n, row_stride)
#define SM_BY_ITEMS(T, V)                                   \
  do {                                                      \
    if (packs <= 256) SM_LAUNCH(T, V, 1);                   \
    else if (packs <= 512) SM_LAUNCH(T, V, 2);              \
    else if (packs <= 1024) SM_LAUNCH(T, V, 4);             \
    else SM_LAUNCH(T, V, 8);                                \
  } while (0)
      // rows of up to 512 packs (4096 bf16 / 2048 f32 elements), several of them: one wave per row
      if (aligned && packs <= 512 && rows >= 4) {
        const int64_t wblocks = (rows + 3) / 4;
        const int wgrid = (int)(wblocks < kNumCU * 32 ? wblocks : kNumCU * 32);
#define SMW_LAUNCH(T, V, ITEMS)                                                                                 \
  hipLaunchKernelGGL((k_softmax_wave<T, V, ITEMS, LOG>), dim3(wgrid), dim3(256), 0, st, (T *)base_ptr(out),       \
                     (const T *)base_ptr(in), rows, n, row_stride)
#define SMW_BY_ITEMS(T, V)                          \
  do {                                              \
    if (packs <= 64) SMW_LAUNCH(T, V, 1);           \
    else if (packs <= 128) SMW_LAUNCH(T, V, 2);     \
    else if (packs <= 256) SMW_LAUNCH(T, V, 4);     \
    else SMW_LAUNCH(T, V, 8);                       \
  } while (0)
        if (in->dtype == RAI_F32) SMW_BY_ITEMS(float, 4);
        else if (in->dtype == RAI_BF16) SMW_BY_ITEMS(bf16_raw, 8);
        else SMW_BY_ITEMS(f16_raw, 8);
#undef SMW_BY_ITEMS
#undef SMW_LAUNCH
        return launch_check("softmax_wave");
      }
      if (packs <= 2048) {
        if (in->dtype == RAI_F32) { if (aligned) SM_BY_ITEMS(float, 4); else SM_BY_ITEMS(float, 1); }
        else if (in->dtype == RAI_BF16) { if (aligned) SM_BY_ITEMS(bf16_raw, 8); else SM_BY_ITEMS(bf16_raw, 1); }
        else { if (aligned) SM_BY_ITEMS(f16_raw, 8); else SM_BY_ITEMS(f16_raw, 1); }
        return launch_check("softmax_row");
      }
#undef SM_BY_ITEMS
#undef SM_LAUNCH
    }
  }
  if (n >= 256 && in->dtype != RAI_F64) {
    int grid = (int)(si.n_out < kNumCU * 16 ? si.n_out : kNumCU * 16);
    RAI_DISPATCH_FLOAT(in->dtype, T,
                       hipLaunchKernelGGL((k_softmax_strided_block<T, LOG>), dim3(grid), dim3(256), 0, st,
                                          (T *)base_ptr(out), (const T *)base_ptr(in), si, ax_in, ax_out, so));
  } else {
    int64_t blocks = (si.n_out + 255) / 256;
    int grid = (int)(blocks < kNumCU * 16 ? blocks : kNumCU * 16);
    RAI_DISPATCH_FLOAT(in->dtype, T,
                       hipLaunchKernelGGL((k_softmax_strided_thread<T, LOG>), dim3(grid), dim3(256), 0, st,
                                          (T *)base_ptr(out), (const T *)base_ptr(in), si, ax_in, ax_out, so));
  }
  return launch_check("softmax");
}

// Partial results of the allocation-free argmax: a fixed array in device memory instead of the grown-on-demand
// workspace.  Every GPU holds its own copy at its own address; the address is looked up once per device when the
// device context is created (arg_static_scratch_init) and only that pointer is ever handed to kernels.
static constexpr size_t kArgStaticParts = 65536;   // (row, split) partial results one call may produce
// values (8 bytes, f64 rows), indices and one arrival counter per row; the counters start at zero (the array is
// zero-initialised when the code object is loaded) and every call leaves them at zero
static constexpr size_t kArgStaticBytes = kArgStaticParts * (sizeof(double) + 2 * sizeof(uint32_t));
static __device__ __align__(256) unsigned char scratch[kArgStaticBytes];
static void *g_scratch_ptr[16] = {nullptr};

int arg_static_scratch_init(int dev) {
  if (dev < 0 || dev >= 16) return fail(RAI_ERR_BAD_ARG, "device index %d out of range", dev);
  void *p = nullptr;
  RAI_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
  g_scratch_ptr[dev] = p;
  return RAI_OK;
}

template <bool IS_MAX>
static int arg_impl(int dev, const rai_hip_tensor *in, int32_t dim, int32_t keep_dim, const rai_hip_tensor *out,
                    bool no_alloc = false) {
  RAI_TRY(validate(in, "in"));
  RAI_TRY(validate(out, "out"));
  RAI_REQUIRE(out->dtype == RAI_U32, RAI_ERR_BAD_DTYPE, "argmax: output must be u32");
  int d = norm_dim(dim, in->rank);
  RAI_REQUIRE(d >= 0 && d < in->rank, RAI_ERR_BAD_ARG, "argmax: dim %d out of range for rank %d", dim, in->rank);
  RAI_REQUIRE(in->shape[d] > 0, RAI_ERR_BAD_SHAPE, "argmax: empty axis");
  RAI_REQUIRE(in->shape[d] < 0xffffffffLL, RAI_ERR_BAD_SHAPE, "argmax: axis too long for u32");
  bool reduced[RAI_HIP_MAX_RANK] = {false};
  reduced[d] = true;
  RAI_TRY(check_reduced_shape(in, reduced, keep_dim, out, "argmax"));
  // the allocation-free form must not create a device context either (that allocates): rai_hip_init comes first
  hipStream_t st = no_alloc ? stream_if_ready(dev) : stream_of(dev);
  if (!st) return RAI_ERR_HIP;
  if (numel(out) == 0) return RAI_OK;
  ReduceSpace s;
  build_reduce_space(in, reduced, &s);
  const int64_t n = in->shape[d];
  s.n_red = n;
  const int64_t ax = in->stride[d];
  uint32_t *o = (uint32_t *)base_ptr(out);
  // Row path: rows addressable by one uniform stride and a long axis.
  if (s.out_rank == 1 && n >= 1024 && in->dtype != RAI_U8 && in->dtype != RAI_U32 && in->dtype != RAI_I64) {
    int64_t rows = s.n_out, row_stride = s.out_stride[0];
    // A row is cut over blocks until there are two blocks per CU: one CU alone draws a long row too slowly ([64, 51200]
    // uncut, one block of 1024 threads per row: 10.2 us against 9.2 us for eight shares per row and the merge).
    int splits = 1;
    while (rows * splits < 2 * kNumCU && n / (splits * 2) >= 2048) splits *= 2;
    const int threads = 256;
    void *ws = nullptr;
    size_t nparts = (size_t)rows * splits;
    if (no_alloc)
      RAI_REQUIRE(nparts <= kArgStaticParts, RAI_ERR_UNSUPPORTED,
                  "argmax_static: %lld rows x %d splits = %zu partial results, the static scratch holds %zu",
                  (long long)rows, splits, nparts, kArgStaticParts);
    if (nparts <= kArgStaticParts && dev >= 0 && dev < 16 && g_scratch_ptr[dev]) {
      // one launch: partial results and arrival counters in the fixed device array, the last block of a row merges
      ws = g_scratch_ptr[dev];
      double *pd = (double *)ws;
      uint32_t *pi = (uint32_t *)((char *)ws + kArgStaticParts * sizeof(double));
      uint32_t *cnt = pi + kArgStaticParts;
      RAI_DISPATCH_FLOAT(in->dtype, T,
                         hipLaunchKernelGGL((k_arg_row_partial<T, IS_MAX>), dim3((unsigned)nparts), dim3(threads), 0, st,
                                            (const T *)base_ptr(in), rows, n, row_stride, ax, splits, (float *)ws, pd, pi,
                                            cnt, o));
      return launch_check("arg_row");
    }
    RAI_REQUIRE(!no_alloc, RAI_ERR_HIP, "argmax_static: scratch address of device %d unknown (rai_hip_init failed?)", dev);
    RAI_TRY(workspace(dev, nparts * (sizeof(double) + sizeof(uint32_t)) + 64, &ws));
    double *pd = (double *)ws;
    float *pf = (float *)ws;
    uint32_t *pi = (uint32_t *)((char *)ws + nparts * sizeof(double));
    RAI_DISPATCH_FLOAT(in->dtype, T,
                       hipLaunchKernelGGL((k_arg_row_partial<T, IS_MAX>), dim3((unsigned)nparts), dim3(threads), 0, st,
                                          (const T *)base_ptr(in), rows, n, row_stride, ax, splits, pf, pd, pi,
                                          (uint32_t *)nullptr, (uint32_t *)nullptr));
    RAI_TRY(launch_check("arg_partial"));
    int fgrid = (int)((rows + 63) / 64);
    if (in->dtype == RAI_F64)
      hipLaunchKernelGGL((k_arg_row_final<double, double, IS_MAX>), dim3(fgrid), dim3(64), 0, st, pd, pi, rows, splits, o,
                         (const double *)base_ptr(in), row_stride);
    else
      RAI_DISPATCH_FLOAT(in->dtype, T,
                         hipLaunchKernelGGL((k_arg_row_final<T, float, IS_MAX>), dim3(fgrid), dim3(64), 0, st, pf, pi,
                                            rows, splits, o, (const T *)base_ptr(in), row_stride));
    return launch_check("arg_final");
  }
  int64_t blocks = (s.n_out + 255) / 256;
  int grid = (int)(blocks < kNumCU * 16 ? blocks : kNumCU * 16);
  RAI_DISPATCH_ALL(in->dtype, T,
                   hipLaunchKernelGGL((k_arg_thread<T, IS_MAX>), dim3(grid), dim3(256), 0, st,
                                      (const T *)base_ptr(in), s, ax, o));
  return launch_check("arg_thread");
}

int launch_argmax_partials(hipStream_t st, int dtype, const void *in, int64_t rows, int64_t n, int splits, float *pval,
                           uint32_t *pidx) {
  RAI_REQUIRE(rows > 0 && n > 0 && splits >= 1 && in && pval && pidx, RAI_ERR_BAD_ARG, "argmax partials: bad arguments");
  RAI_REQUIRE(dtype == RAI_BF16 || dtype == RAI_F16 || dtype == RAI_F32, RAI_ERR_BAD_DTYPE, "argmax partials: dtype %s",
              dtype_name(dtype));
  const int threads = n / splits >= 8192 ? 1024 : 256;
  RAI_DISPATCH_FLOAT(dtype, T, {
    if constexpr (sizeof(T) <= 4)
      hipLaunchKernelGGL((k_arg_row_partial<T, true>), dim3((unsigned)(rows * splits)), dim3(threads), 0, st, (const T *)in,
                         rows, n, n, (int64_t)1, splits, pval, (double *)nullptr, pidx, (uint32_t *)nullptr,
                         (uint32_t *)nullptr);
  });
  return launch_check("argmax_partials");
}

}  // namespace rai

using namespace rai;

extern "C" {

int rai_hip_reduce(int dev, int op, const rai_hip_tensor *in, const int32_t *dims, int32_t ndims, int32_t keep_dim,
                   const rai_hip_tensor *out) {
  RAI_TRY(validate(in, "in"));
  RAI_TRY(validate(out, "out"));
  RAI_REQUIRE(op >= RAI_RED_SUM && op <= RAI_RED_MIN, RAI_ERR_BAD_ARG, "reduce: bad op %d", op);
  RAI_REQUIRE(in->dtype == out->dtype, RAI_ERR_BAD_DTYPE, "reduce: dtype mismatch");
  RAI_REQUIRE(ndims >= 0 && ndims <= in->rank && (ndims == 0 || dims), RAI_ERR_BAD_ARG, "reduce: bad dims");
  bool reduced[RAI_HIP_MAX_RANK] = {false};
  for (int i = 0; i < ndims; ++i) {
    int d = norm_dim(dims[i], in->rank);
    RAI_REQUIRE(d >= 0 && d < in->rank, RAI_ERR_BAD_ARG, "reduce: dim %d out of range", dims[i]);
    RAI_REQUIRE(!reduced[d], RAI_ERR_BAD_ARG, "reduce: dim %d listed twice", dims[i]);
    reduced[d] = true;
  }
  RAI_TRY(check_reduced_shape(in, reduced, keep_dim, out, "reduce"));
  hipStream_t st = stream_of(dev);
  if (!st) return RAI_ERR_HIP;
  if (numel(out) == 0) return RAI_OK;
  ReduceSpace s;
  build_reduce_space(in, reduced, &s);
  if (s.n_red == 0 || numel(in) == 0) {
    RAI_REQUIRE(op == RAI_RED_SUM, RAI_ERR_BAD_SHAPE, "reduce: max/min over an empty axis");
    return rai_hip_fill(dev, out, 0.0);
  }
  // A block per output when the reduce space is long or its innermost stride is
  // the unit one; otherwise a thread per output keeps loads coalesced.
  bool red_inner_unit = s.red_stride[s.red_rank - 1] == 1;
  bool use_block = s.n_red >= 64 && (red_inner_unit || s.n_out < 4096);
  if (use_block) {
    int grid = (int)(s.n_out < kNumCU * 32 ? s.n_out : kNumCU * 32);
    RAI_DISPATCH_ALL(in->dtype, T,
                     hipLaunchKernelGGL((k_reduce_block<T>), dim3(grid), dim3(256), 0, st, s, (T *)base_ptr(out),
                                        (const T *)base_ptr(in), op));
  } else {
    int64_t blocks = (s.n_out + 255) / 256;
    int grid = (int)(blocks < kNumCU * 16 ? blocks : kNumCU * 16);
    RAI_DISPATCH_ALL(in->dtype, T,
                     hipLaunchKernelGGL((k_reduce_thread<T>), dim3(grid), dim3(256), 0, st, s, (T *)base_ptr(out),
                                        (const T *)base_ptr(in), op));
  }
  return launch_check("reduce");
}

int rai_hip_softmax(int dev, const rai_hip_tensor *in, int32_t dim, const rai_hip_tensor *out) {
  return softmax_impl<false>(dev, in, dim, out);
}
int rai_hip_log_softmax(int dev, const rai_hip_tensor *in, int32_t dim, const rai_hip_tensor *out) {
  return softmax_impl<true>(dev, in, dim, out);
}
int rai_hip_argmax(int dev, const rai_hip_tensor *in, int32_t dim, int32_t keep_dim, const rai_hip_tensor *out) {
  return arg_impl<true>(dev, in, dim, keep_dim, out);
}
int rai_hip_argmin(int dev, const rai_hip_tensor *in, int32_t dim, int32_t keep_dim, const rai_hip_tensor *out) {
  return arg_impl<false>(dev, in, dim, keep_dim, out);
}
int rai_hip_argmax_static(int dev, const rai_hip_tensor *in, int32_t dim, int32_t keep_dim, const rai_hip_tensor *out) {
  return arg_impl<true>(dev, in, dim, keep_dim, out, true);
}

}  // extern "C"
