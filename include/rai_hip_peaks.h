/* Measurement aid of librai_hip.so: the ceilings of the GPU it runs on, measured with loops that have no workload
 * around them.  No counterpart in the reference (cksac/rai measures nothing of the kind); not used by any product
 * path.  `python bench.py --workload peaks` prints every figure. */
#ifndef RAI_HIP_PEAKS_H
#define RAI_HIP_PEAKS_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum rai_hip_peak_kind {
  RAI_PEAK_MFMA_BF16 = 0,     /* v_mfma_f32_32x32x16_bf16 on register operands, eight waves per CU; work = flops */
  RAI_PEAK_MFMA_BF16_LDS = 1, /* the same with twelve 1 KB LDS fragment reads per sixteen multiplies; work = flops */
  RAI_PEAK_LDS_READ = 2,      /* ds_read_b128 alone, eight waves per CU; work = bytes read from LDS */
  RAI_PEAK_HBM_READ = 3,      /* plain read of `bytes` of device memory; work = bytes */
  RAI_PEAK_HBM_COPY = 4,      /* plain copy of `bytes` (reads `bytes`, writes `bytes`); work = bytes read */
  RAI_PEAK_STAGE_DMA = 5,     /* every CU stages 64 KB tiles out of a buffer of `bytes` into LDS with global_load_lds,
                                 one tile in flight behind the one waited for; work = bytes staged */
  RAI_PEAK_STAGE_VGPR = 6,    /* the same through registers (global load, ds_write_b128); work = bytes staged */
  RAI_PEAK_GEMM_LOOP = 7      /* the tile GEMM's main loop without the GEMM: per K tile of 64 a block stages 64 KB out of
                                 a buffer of `bytes` with global_load_lds, reads 24 KB of fragments per wave, issues 32
                                 multiplies per wave, waits for its loads and meets at a barrier; work = flops */
} rai_hip_peak_kind;

/* Runs one warm-up launch and `launches` timed launches (HIP events on the library's stream of `dev`) of the loop
 * `kind`; `bytes` sizes the HBM kinds (1 MiB .. 8 GiB, a multiple of 16) and the source buffer of the staging kinds and of the GEMM loop
 * (64 KiB .. 1 GiB, a multiple of 64 KiB: 2 MiB stays in the L2s, 32 MiB in the memory-side cache); the others ignore it.  Returns the mean
 * time of a launch and the work one launch does (flops or bytes, see above).  Allocates and frees its own buffers. */
int rai_hip_measure_peak(int dev, int32_t kind, int64_t bytes, int32_t launches, double *seconds_per_launch,
                         double *work_per_launch);

#ifdef __cplusplus
}
#endif
#endif
