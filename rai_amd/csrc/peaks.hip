// Measured ceilings of this GPU, as loops without a workload around them: what the matrix pipes sustain with nothing
// to wait for, what LDS fragment reads cost beside them, how fast global memory streams into registers and into LDS.
// The kernels behind rai_hip_measure_peak (include/rai_hip_peaks.h); bench.py --workload peaks prints them.  The
// library's product kernels do not use anything in this file.
#include <cstdlib>

#include "common.h"
#include "rai_hip_peaks.h"

namespace rai {
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 pk_bf16x8;
typedef __attribute__((ext_vector_type(16))) float pk_f32x16;
typedef __attribute__((ext_vector_type(4))) uint32_t pk_u32x4;

constexpr int kPeakThreads = 512;   // eight waves per CU, two per SIMD
constexpr int kMfmaPerIter = 16;

// Eight independent 32 x 32 accumulators per wave, two v_mfma_f32_32x32x16_bf16 on each per iteration (the instruction
// and the accumulator count of the library's tile GEMM): issue never waits for a result.  LDS_READS > 0: that many
// 1 KB fragment reads (ds_read_b128 per lane) are issued per iteration beside the multiplies -- twelve per sixteen
// multiplies is what a wave of the 256 x 256 tile kernel reads -- and their values become operands of the next
// iteration.
template <int LDS_READS>
__global__ void __launch_bounds__(kPeakThreads) k_peak_mfma(float *out, int iters) {
  __shared__ __attribute__((aligned(16))) pk_u32x4 frag[2048];   // 32 KB
  const int tid = threadIdx.x, lane = tid & 63;
  for (int i = tid; i < 2048; i += kPeakThreads) frag[i] = pk_u32x4{0x3c003c00u + i, 0x3c003c00u, 0x3c003c00u, 0x3c003c00u};
  __syncthreads();
  pk_bf16x8 a, b;
  for (int j = 0; j < 8; ++j) { a[j] = (__bf16)(0.001f * (float)(lane + j)); b[j] = (__bf16)(1.0f / (float)(1 + j)); }
  pk_f32x16 acc[kMfmaPerIter / 2];
  for (int j = 0; j < kMfmaPerIter / 2; ++j)
    for (int r = 0; r < 16; ++r) acc[j][r] = 0.f;
  pk_u32x4 got[LDS_READS > 0 ? LDS_READS : 1];
  const int base = lane + (tid >> 6) * 37;
  for (int it = 0; it < iters; ++it) {
    if constexpr (LDS_READS > 0) {
#pragma unroll
      for (int r = 0; r < LDS_READS; ++r) got[r] = frag[((it + r) * 64 + base) & 2047];
    }
#pragma unroll
    for (int j = 0; j < kMfmaPerIter; ++j)
      acc[j % (kMfmaPerIter / 2)] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[j % (kMfmaPerIter / 2)], 0, 0, 0);
    if constexpr (LDS_READS > 0) {
      pk_u32x4 x = got[0];
#pragma unroll
      for (int r = 1; r < LDS_READS; ++r) { x.x ^= got[r].x; x.y ^= got[r].y; x.z ^= got[r].z; x.w ^= got[r].w; }
      // the fragments feed the next iteration's operand: one low mantissa bit of each element
      pk_u32x4 av;
      __builtin_memcpy(&av, &a, 16);
      av.x ^= x.x & 0x00010001u; av.y ^= x.y & 0x00010001u; av.z ^= x.z & 0x00010001u; av.w ^= x.w & 0x00010001u;
      __builtin_memcpy(&a, &av, 16);
    }
  }
  float s = 0.f;
  for (int j = 0; j < kMfmaPerIter / 2; ++j)
    for (int r = 0; r < 16; ++r) s += acc[j][r];
  out[blockIdx.x * kPeakThreads + tid] = s;
}

// LDS fragment reads alone: 16 reads of 1 KB per wave and iteration.
__global__ void __launch_bounds__(kPeakThreads) k_peak_lds_read(float *out, int iters) {
  __shared__ __attribute__((aligned(16))) pk_u32x4 frag[2048];
  const int tid = threadIdx.x, lane = tid & 63;
  for (int i = tid; i < 2048; i += kPeakThreads) frag[i] = pk_u32x4{(uint32_t)i, 1u, 2u, 3u};
  __syncthreads();
  pk_u32x4 x = {0u, 0u, 0u, 0u};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const pk_u32x4 v = frag[((it * 16 + r) * 64 + lane + (tid >> 6) * 37) & 2047];
      x.x ^= v.x; x.y += v.y; x.z ^= v.z; x.w += v.w;
    }
  }
  out[blockIdx.x * kPeakThreads + tid] = (float)(x.x ^ x.y ^ x.z ^ x.w);
}

// Plain streaming read (COPY: and write) of n 16-byte words, eight loads in flight per lane.
template <bool COPY>
__global__ void __launch_bounds__(256) k_peak_stream(const pk_u32x4 *src, pk_u32x4 *dst, int64_t n, uint32_t *sink) {
  const int64_t stride = (int64_t)gridDim.x * 256 * 8;
  pk_u32x4 x = {0u, 0u, 0u, 0u};
  for (int64_t base = (int64_t)blockIdx.x * 256 * 8 + threadIdx.x; base < n; base += stride) {
    pk_u32x4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int64_t i = base + u * 256;
      v[u] = i < n ? __builtin_nontemporal_load(src + i) : pk_u32x4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int64_t i = base + u * 256;
      if constexpr (COPY) {
        if (i < n) __builtin_nontemporal_store(v[u], dst + i);
      } else {
        x.x ^= v[u].x; x.y ^= v[u].y; x.z ^= v[u].z; x.w ^= v[u].w;
      }
    }
  }
  if (!COPY && (x.x ^ x.y ^ x.z ^ x.w) == 0x9e3779b9u) *sink = 1u;   // keeps the loads; practically never taken
}

// Every CU stages 64 KB tiles (what one K tile of a 256 x 256 x 64 GEMM block needs) out of a buffer of `tiles` tiles
// (small: resident in the XCDs' L2s; tens of MB: in the memory-side cache), one tile in flight while the block waits
// for the one before, as the tile kernel's two LDS stages do.  DMA: global_load_lds_dwordx4, 16 bytes per lane straight
// into LDS; otherwise global -> VGPR -> ds_write_b128.
template <bool DMA>
__global__ void __launch_bounds__(kPeakThreads) k_peak_stage(const pk_u32x4 *src, int64_t tiles, int iters, uint32_t *sink) {
  extern __shared__ __attribute__((aligned(16))) pk_u32x4 stage_lds[];   // two stages of 64 KB
  pk_u32x4(*stage)[4096] = reinterpret_cast<pk_u32x4(*)[4096]>(stage_lds);
  typedef __attribute__((address_space(3))) void *lds_ptr;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  auto tile_of = [&](int it) { return src + ((int64_t)(blockIdx.x * 7 + it) % tiles) * 4096 + wave * 512 + lane; };
  if constexpr (DMA) {
    auto issue = [&](int it) {
      const pk_u32x4 *t = tile_of(it);
      pk_u32x4 *dst = stage[it & 1] + wave * 512;
#pragma unroll
      for (int j = 0; j < 8; ++j)   // one instruction: 64 lanes x 16 bytes into 1 KB of consecutive LDS
        __builtin_amdgcn_global_load_lds((const void *)(t + j * 64), (lds_ptr)(dst + j * 64), 16, 0, 0);
    };
    issue(0);
    for (int it = 0; it < iters; ++it) {
      issue(it + 1);
      asm volatile("s_waitcnt vmcnt(8)" ::: "memory");   // tile `it` has landed; tile it + 1 is on its way
      __builtin_amdgcn_s_barrier();
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  } else {
    pk_u32x4 v[8];
    {
      const pk_u32x4 *t = tile_of(0);
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = t[j * 64];
    }
    for (int it = 0; it < iters; ++it) {
      pk_u32x4 *dst = stage[it & 1] + wave * 512 + lane;
      pk_u32x4 nx[8];
      const pk_u32x4 *t = tile_of(it + 1);
#pragma unroll
      for (int j = 0; j < 8; ++j) nx[j] = t[j * 64];
#pragma unroll
      for (int j = 0; j < 8; ++j) dst[j * 64] = v[j];
      __syncthreads();
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = nx[j];
    }
  }
  __syncthreads();
  const pk_u32x4 v0 = stage[0][tid];
  if ((v0.x ^ v0.y ^ v0.z ^ v0.w) == 0x9e3779b9u && stage[1][tid].x == 0x7f4a7c15u) *sink = 1u;
}

// The tile GEMM's main loop without the GEMM: per iteration (one K tile of 64 of a 256 x 256 block) every wave
// issues its eight global_load_lds of the next 64 KB stage, reads 24 fragments of 1 KB from the current stage, issues
// 32 v_mfma_f32_32x32x16_bf16, waits for its loads and meets the block at a barrier.  The stages come out of a buffer
// of `tiles` tiles as in k_peak_stage, so the same loop can be fed from the L2, from the memory-side cache or from HBM.
__global__ void __launch_bounds__(kPeakThreads) k_peak_gemm_loop(const pk_u32x4 *src, int64_t tiles, int iters, float *out) {
  extern __shared__ __attribute__((aligned(16))) pk_u32x4 stage_lds[];   // two stages of 64 KB
  pk_u32x4(*stage)[4096] = reinterpret_cast<pk_u32x4(*)[4096]>(stage_lds);
  typedef __attribute__((address_space(3))) void *lds_ptr;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  auto issue = [&](int it) {
    const pk_u32x4 *t = src + ((int64_t)(blockIdx.x * 7 + it) % tiles) * 4096 + wave * 512 + lane;
    pk_u32x4 *dst = stage[it & 1] + wave * 512;
#pragma unroll
    for (int j = 0; j < 8; ++j) __builtin_amdgcn_global_load_lds((const void *)(t + j * 64), (lds_ptr)(dst + j * 64), 16, 0, 0);
  };
  pk_f32x16 acc[8];
  for (int j = 0; j < 8; ++j)
    for (int r = 0; r < 16; ++r) acc[j][r] = 0.f;
  issue(0);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  for (int it = 0; it < iters; ++it) {
    issue(it + 1);
    const pk_u32x4 *cur = stage[it & 1];
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      pk_u32x4 f[12];
#pragma unroll
      for (int r = 0; r < 12; ++r) f[r] = cur[((half * 12 + r) * 64 + lane + wave * 37) & 4095];
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        pk_bf16x8 a, b;
        __builtin_memcpy(&a, &f[j % 12], 16);
        __builtin_memcpy(&b, &f[(j + 5) % 12], 16);
        acc[j % 8] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[j % 8], 0, 0, 0);
      }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the next stage has landed
    __builtin_amdgcn_s_barrier();                       // ... for every wave, and this stage is free again
  }
  float sum = 0.f;
  for (int j = 0; j < 8; ++j)
    for (int r = 0; r < 16; ++r) sum += acc[j][r];
  out[blockIdx.x * kPeakThreads + tid] = sum;
}

struct Timed {
  hipEvent_t e0 = nullptr, e1 = nullptr;
  ~Timed() {
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
  }
};

}  // namespace
}  // namespace rai

using namespace rai;

extern "C" int rai_hip_measure_peak(int dev, int32_t kind, int64_t bytes, int32_t launches, double *seconds_per_launch, double *work_per_launch) {
  RAI_REQUIRE(seconds_per_launch && work_per_launch && launches >= 1 && launches <= 1000, RAI_ERR_BAD_ARG, "measure_peak: bad arguments");
  hipStream_t st = stream_of(dev);
  if (!st) return RAI_ERR_HIP;
  const int cus = device_cu_count(dev);
  RAI_REQUIRE(cus > 0, RAI_ERR_HIP, "measure_peak: device %d reports no CUs", dev);
  RAI_REQUIRE(kind >= RAI_PEAK_MFMA_BF16 && kind <= RAI_PEAK_GEMM_LOOP, RAI_ERR_BAD_ARG, "measure_peak: unknown kind %d", kind);
  if (kind == RAI_PEAK_HBM_READ || kind == RAI_PEAK_HBM_COPY)
    RAI_REQUIRE(bytes >= (1 << 20) && bytes <= ((int64_t)8 << 30) && bytes % 16 == 0, RAI_ERR_BAD_ARG, "measure_peak: 1 MiB .. 8 GiB, a multiple of 16");
  if (kind == RAI_PEAK_STAGE_DMA || kind == RAI_PEAK_STAGE_VGPR || kind == RAI_PEAK_GEMM_LOOP)
    RAI_REQUIRE(bytes >= 65536 && bytes <= ((int64_t)1 << 30) && bytes % 65536 == 0, RAI_ERR_BAD_ARG, "measure_peak: 64 KiB .. 1 GiB of 64 KiB tiles");
  void *buf = nullptr, *out = nullptr;
  uint32_t *sink = nullptr;
  RAI_TRY(rai_hip_alloc(dev, (size_t)cus * kPeakThreads * sizeof(float) + 256, &out));
  sink = (uint32_t *)((char *)out + (size_t)cus * kPeakThreads * sizeof(float));
  const int iters = 4096;
  double work = 0.0;
  int64_t words = 0;
  const bool streams = kind == RAI_PEAK_HBM_READ || kind == RAI_PEAK_HBM_COPY;
  const bool stages = kind == RAI_PEAK_STAGE_DMA || kind == RAI_PEAK_STAGE_VGPR || kind == RAI_PEAK_GEMM_LOOP;
  if (streams) {
    words = bytes / 16;
    const size_t total = (size_t)bytes * (kind == RAI_PEAK_HBM_COPY ? 2 : 1);
    int rc = rai_hip_alloc(dev, total, &buf);
    if (rc != RAI_OK) { (void)rai_hip_release(out); return rc; }
    (void)hipMemsetAsync(buf, 0x5a, total, st);
    work = (double)bytes;   // bytes read (a copy writes as many again)
  } else if (stages) {
    const size_t total = (size_t)bytes;   // a whole number of 64 KB tiles
    int rc = rai_hip_alloc(dev, total, &buf);
    if (rc != RAI_OK) { (void)rai_hip_release(out); return rc; }
    (void)hipMemsetAsync(buf, 0x11, total, st);
    work = kind == RAI_PEAK_GEMM_LOOP ? (double)cus * (kPeakThreads / 64) * (double)iters * 32.0 * (2.0 * 32 * 32 * 16)   // flops
                                      : (double)cus * iters * 65536.0;
  } else if (kind == RAI_PEAK_LDS_READ) {
    work = (double)cus * (kPeakThreads / 64) * (double)iters * 16.0 * 1024.0;
  } else {
    work = (double)cus * (kPeakThreads / 64) * (double)iters * kMfmaPerIter * (2.0 * 32 * 32 * 16);
  }
  constexpr size_t kStageLds = 2 * 65536;
  if (stages) {
    const void *fn = kind == RAI_PEAK_STAGE_DMA ? (const void *)k_peak_stage<true>
                     : kind == RAI_PEAK_STAGE_VGPR ? (const void *)k_peak_stage<false> : (const void *)k_peak_gemm_loop;
    hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kStageLds);
    if (e != hipSuccess) {
      (void)rai_hip_release(buf);
      (void)rai_hip_release(out);
      return fail(RAI_ERR_HIP, "measure_peak: %s", hipGetErrorString(e));
    }
  }
  auto launch = [&]() {
    switch (kind) {
      case RAI_PEAK_MFMA_BF16: hipLaunchKernelGGL(k_peak_mfma<0>, dim3(cus), dim3(kPeakThreads), 0, st, (float *)out, iters); break;
      case RAI_PEAK_MFMA_BF16_LDS: hipLaunchKernelGGL(k_peak_mfma<12>, dim3(cus), dim3(kPeakThreads), 0, st, (float *)out, iters); break;
      case RAI_PEAK_LDS_READ: hipLaunchKernelGGL(k_peak_lds_read, dim3(cus), dim3(kPeakThreads), 0, st, (float *)out, iters); break;
      case RAI_PEAK_HBM_READ:
        hipLaunchKernelGGL(k_peak_stream<false>, dim3(cus * 8), dim3(256), 0, st, (const pk_u32x4 *)buf, (pk_u32x4 *)nullptr, words, sink);
        break;
      case RAI_PEAK_HBM_COPY:
        hipLaunchKernelGGL(k_peak_stream<true>, dim3(cus * 8), dim3(256), 0, st, (const pk_u32x4 *)buf, (pk_u32x4 *)buf + words, words, sink);
        break;
      case RAI_PEAK_STAGE_DMA: hipLaunchKernelGGL(k_peak_stage<true>, dim3(cus), dim3(kPeakThreads), kStageLds, st, (const pk_u32x4 *)buf, (int64_t)(bytes / 65536), iters, sink); break;
      case RAI_PEAK_GEMM_LOOP:
        hipLaunchKernelGGL(k_peak_gemm_loop, dim3(cus), dim3(kPeakThreads), kStageLds, st, (const pk_u32x4 *)buf, (int64_t)(bytes / 65536), iters, (float *)out);
        break;
      default: hipLaunchKernelGGL(k_peak_stage<false>, dim3(cus), dim3(kPeakThreads), kStageLds, st, (const pk_u32x4 *)buf, (int64_t)(bytes / 65536), iters, sink); break;
    }
  };
  Timed t;
  int rc = RAI_OK;
  float ms = 0.f;
  launch();   // warm-up
  if (hipEventCreate(&t.e0) != hipSuccess || hipEventCreate(&t.e1) != hipSuccess) rc = fail(RAI_ERR_HIP, "measure_peak: event");
  if (rc == RAI_OK) rc = launch_check("measure_peak");
  if (rc == RAI_OK) {
    (void)hipEventRecord(t.e0, st);
    for (int i = 0; i < launches; ++i) launch();
    (void)hipEventRecord(t.e1, st);
    if (hipEventSynchronize(t.e1) != hipSuccess || hipEventElapsedTime(&ms, t.e0, t.e1) != hipSuccess) rc = fail(RAI_ERR_HIP, "measure_peak: timing failed");
  }
  if (buf) (void)rai_hip_release(buf);
  (void)rai_hip_release(out);
  RAI_TRY(rc);
  *seconds_per_launch = (double)ms * 1e-3 / launches;
  *work_per_launch = work;
  return check_kernel_fault(dev);
}
