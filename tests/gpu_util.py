"""Shared helpers of the GPU parity tests (the HIP path is always reached through the C ABI)."""
import numpy as np

from lumen_amd.autograd import Tensor


def f32(a):
    return np.ascontiguousarray(a, np.float32)


def dev(a):
    return Tensor.from_array_no_grad(np.ascontiguousarray(a))


def max_rel(got, ref):
    """max|got - ref| / max|ref|: the norm the tolerances are stated in (summation order differs
    from the reference's strict sequential sum, so elementwise relative error is unbounded near 0)."""
    ref = np.asarray(ref, np.float64)
    return float(np.abs(np.asarray(got, np.float64) - ref).max() / max(np.abs(ref).max(), 1e-30))
