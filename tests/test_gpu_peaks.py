"""The ceiling loops behind `bench.py --workload peaks` (include/rai_hip_peaks.h): every kind runs, and what it
reports lies below the published peak it is compared with and above a floor that a broken loop (work optimised away,
wrong work count) would miss."""
import pytest

from rai_amd import _lib
from rai_amd.hip import measure_peak

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("kind,nbytes,low,high", [
    ("mfma_bf16", 0, 1.0e15, 2.52e15),          # flop/s: at least 40 % of the published 2.5 PFLOP/s, never above it
    ("mfma_bf16_lds", 0, 0.6e15, 2.52e15),
    ("lds_read", 0, 20e12, 256 * 256 * 2.5e9),  # bytes/s over the chip: below 256 B/clk/CU at 2.5 GHz
    ("hbm_read", 1 << 30, 3.0e12, 8.05e12),
    ("hbm_copy", 1 << 28, 1.0e12, 4.05e12),     # bytes read per second (as many written)
    ("stage_dma", 2 << 20, 2.0e12, 256 * 128 * 2.5e9),
    ("stage_vgpr", 32 << 20, 2.0e12, 256 * 128 * 2.5e9),
    ("gemm_loop", 2 << 20, 0.5e15, 2.52e15),    # flop/s of the GEMM main loop fed from the L2
])
def test_ceiling_loops_report_plausible_rates(hip, kind, nbytes, low, high):
    measure_peak(kind, nbytes, 1)
    sec, work = measure_peak(kind, nbytes, 5)
    assert sec > 0 and work > 0
    assert low < work / sec < high, (kind, work / sec)


def test_ceiling_loop_arguments_are_checked(hip):
    with pytest.raises(_lib.RaiHipError):
        measure_peak("hbm_read", 100, 1)
    with pytest.raises(_lib.RaiHipError):
        measure_peak("stage_dma", 1000, 1)
