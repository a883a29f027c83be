import ctypes
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

HELPERS = os.path.join(ROOT, "tests", "helpers")
CAPTURE_SO = os.path.join(HELPERS, "libxerbla_capture.so")


def _build_capture():
    src = os.path.join(HELPERS, "xerbla_capture.c")
    if (not os.path.exists(CAPTURE_SO)) or os.path.getmtime(CAPTURE_SO) < os.path.getmtime(src):
        subprocess.run(["gcc", "-O1", "-shared", "-fPIC", "-o", CAPTURE_SO, src], check=True)


# The netlib testers replace the library's xerbla at link time
# (test/F77/dblat3.f:2768-2823, test/C/c_xerbla.c:8-85).  The dynamic-loading
# equivalent: put our recording definitions into the global symbol scope
# before libulmblas_gpu.so (or the compiled reference) resolves its calls.
_build_capture()
XERBLA = ctypes.CDLL(CAPTURE_SO, mode=ctypes.RTLD_GLOBAL)
XERBLA.capture_count.restype = ctypes.c_int
XERBLA.capture_last_info.restype = ctypes.c_int
XERBLA.capture_last_name.restype = ctypes.c_char_p
XERBLA.hook_count.restype = ctypes.c_int
XERBLA.hook_last_status.restype = ctypes.c_int
XERBLA.hook_last_routine.restype = ctypes.c_char_p


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X; run with -m gpu on the GPU box")


def _have_gpu():
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _have_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as O
    O.lib()
    return O


@pytest.fixture()
def xerbla():
    """Recorder of xerbla_ / cblas_xerbla calls: reset before each test."""
    XERBLA.capture_reset()
    XERBLA.hook_reset()
    return XERBLA
