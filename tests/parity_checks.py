"""Result checks shared by the GPU parity suites.

fp16 results (fp16 inputs, fp32 accumulate, one rounding to fp16) must be within REL_TOL of the fp32 host reference,
measured per tensor as max|err| / max|ref|, and element by element within an fp16-rounding allowance.
"""
import numpy as np

REL_TOL = 1e-2          # tolerance stated for fp16 inputs / fp32 accumulate


def check_f16(got, ref):
    got = np.asarray(got).astype(np.float32)
    scale = float(np.abs(ref).max()) + 1e-30
    err = float(np.abs(got - ref).max())
    assert err / scale <= REL_TOL, (err, scale)
    # element-wise: fp16 rounding of the result (2^-11 relative) + accumulation noise
    assert np.all(np.abs(got - ref) <= 2e-3 * np.abs(ref) + 2e-3 * scale)
