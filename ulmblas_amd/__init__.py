"""MI355X-native GEMM behind ulmBLAS's BLAS / CBLAS entry points.

The product is ``libulmblas_gpu.so`` (HIP kernels + a C ABI, sources under
``csrc/``, declarations in ``include/ulmblas_gpu.h``).  This package is the
thin Python access to it used by the tests and the benchmark:

* ``ulmblas_amd.blas``  -- ``dgemm_`` / ``sgemm_`` / ``cblas_dgemm`` / ... on
  numpy arrays in host memory, and the device-resident ``gpu_dgemm`` /
  ``gpu_sgemm`` on torch tensors;
* ``ulmblas_amd.synth`` -- seeded synthetic operands.

There is no CPU fallback: if the shared library has not been built, loading
fails with an error that says how to build it.
"""
from .lib import build, load, library_path  # noqa: F401
