"""Error measures shared by the parity tests.

Matvec outputs are zero-mean sums, so a per-element relative error needs a floor
on the denominator: an output that happens to land near zero must not turn an
absolute error of a few ulps of the typical magnitude into a large ratio.

  * fp32-accumulate results are held to TOL_F32_ACC with a floor of 1% of the RMS
    of the reference vector (FLOOR_F32).
  * Comparisons against fp16-accumulate arithmetic (the reference's "faster" 3-bit
    kernel, its LUT-GEMM and AQLM kernels, and the oracle's restatements of them)
    are held to TOL_F16_ACC with the RMS itself as the floor (FLOOR_F16): the
    rounding error of an fp16 running sum scales with the size of the partial
    sums, i.e. with the typical output magnitude, not with the output it lands on.
    The reference's own fp16 kernels sit at ~1e-3 of the RMS from the exact result.
"""
import numpy as np

TOL_F32_ACC = 1e-3   # relative error bound for fp32-accumulate matvec outputs
TOL_F16_ACC = 2e-2   # relative error bound against fp16-accumulate arithmetic
FLOOR_F32 = 0.01
FLOOR_F16 = 1.0


def rel_err(got, ref, floor_frac=FLOOR_F32):
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    if ref.size == 0:
        return 0.0
    floor = floor_frac * float(np.sqrt(np.mean(ref ** 2)))
    denom = np.maximum(np.abs(ref), max(floor, 1e-30))
    return float(np.max(np.abs(got - ref) / denom))
