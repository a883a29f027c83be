"""Helpers of the GPU tests: moving column-major windows between numpy and
device memory, and the parity criterion."""
import numpy as np

# Parity bound of every GPU test, elementwise:
#     |C_gpu - C_oracle| <= TOL_C * max(k, 1) * eps * (|alpha| |A||B| + |beta| |C|)
# The oracle (sequential sums, separate multiply and add) and the GPU (FMA, a
# different summation order) each stay within k*eps*gauge of the exact value.
TOL_C = 2.0


def to_device(X):
    """A Fortran-ordered (ld x cols) window as a device tensor with the same
    memory image (shape (cols, ld), contiguous)."""
    import torch
    assert X.flags.f_contiguous
    return torch.from_numpy(X.T).cuda()


def to_host(dX):
    """Inverse of to_device."""
    return np.asfortranarray(dX.cpu().numpy().T)


def parity_ratio(got, want, gauge, k, dtype):
    """max over elements of |got - want| / (max(k,1) * eps * gauge); elements
    whose gauge is zero must agree exactly (ratio inf otherwise)."""
    eps = np.finfo(dtype).eps
    diff = np.abs(got.astype(np.float64) - want.astype(np.float64))
    scale = max(k, 1) * eps * gauge
    with np.errstate(divide="ignore", invalid="ignore"):
        r = np.where(diff == 0, 0.0, diff / scale)
    return float(r.max()) if r.size else 0.0
