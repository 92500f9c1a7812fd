"""Error measures shared by the parity tests.

Matvec outputs are zero-mean sums, so a per-element relative error needs a floor
on the denominator: an output that happens to land near zero must not turn an
absolute error of a few fp32 ulps of the typical magnitude into a large ratio.
The floor is 1% of the RMS of the reference vector."""
import numpy as np

TOL_F32_ACC = 1e-3   # relative error bound for fp32-accumulate matvec outputs
TOL_F16_ACC = 2e-2   # relative error bound for fp16-accumulate matvec outputs


def rel_err(got, ref):
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    floor = 0.01 * float(np.sqrt(np.mean(ref ** 2))) if ref.size else 0.0
    denom = np.maximum(np.abs(ref), max(floor, 1e-30))
    return float(np.max(np.abs(got - ref) / denom)) if ref.size else 0.0
