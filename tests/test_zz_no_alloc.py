"""ulmblas_gpu_dgetrf_static: the LU factorisation for callers that cannot
allocate device memory.  Its exchange area is a device array inside the
library instead of the caller's workspace; everything else is
ulmblas_gpu_dgetrf.  Called through the C ABI, two factorisations in a row
(the second smaller, so that whatever the first left in the array lies beyond
what the second one clears), each compared with ulmblas_gpu_dgetrf on the same
input: pivots, info and every bit of the factors must agree, and both must
agree with the oracle's pivots."""
import ctypes as C

import numpy as np
import pytest

from gpu_util import to_device, to_host
from ulmblas_amd import lib, synth

pytestmark = pytest.mark.gpu


def _p(x):
    return C.c_void_p(x.data_ptr())


def _factor(L, entry, m, n, dA, ld, work=None):
    import torch
    piv = torch.full((min(m, n),), -1, dtype=torch.int32, device="cuda")
    info = torch.full((1,), -7, dtype=torch.int32, device="cuda")
    s = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    if work is None:
        rc = entry(m, n, _p(dA), ld, _p(piv), _p(info), s)
    else:
        rc = entry(m, n, _p(dA), ld, _p(piv), _p(info), _p(work), s)
    assert rc == 0, L.ulmblas_gpu_last_error()
    torch.cuda.synchronize()
    return to_host(dA), piv.cpu().numpy(), int(info.cpu()[0])


def test_static_scratch_matches_workspace_entry(oracle):
    import torch
    L = lib.load()
    work = torch.zeros((L.ulmblas_gpu_dgetrf_worksize() + 7) // 8, dtype=torch.float64, device="cuda")
    # several workgroups per panel, ragged updates (strips), then a smaller, non-square one
    for seed, (m, n) in [(401, (1300, 1100)), (402, (515, 700))]:
        ld = m + 3
        A0 = synth.matrix(seed, m, n, ld)
        dA1, dA2 = to_device(A0), to_device(A0)
        want, wpiv, winfo = _factor(L, L.ulmblas_gpu_dgetrf, m, n, dA1, ld, work)
        free0 = torch.cuda.mem_get_info()[0]
        got, piv, info = _factor(L, L.ulmblas_gpu_dgetrf_static, m, n, dA2, ld)
        free1 = torch.cuda.mem_get_info()[0]
        assert info == winfo == 0, (m, n, info, winfo)
        assert np.array_equal(piv, wpiv), (m, n)
        assert got.tobytes() == want.tobytes(), (m, n)
        ref = A0.copy(order="F")
        oinfo, opiv = oracle.getrf_strided(m, n, ref, (1, ld))
        assert oinfo == 0 and np.array_equal(piv, opiv), (m, n)
        assert np.abs(got[:m] - ref[:m]).max() <= 1e-9 * np.abs(ref[:m]).max(), (m, n)
        assert np.array_equal(got[m:], A0[m:]), "padding rows were written"
        assert free1 >= free0, "device memory was taken"


def test_static_entry_under_graph_capture():
    """What the entry point is for: recorded into a HIP graph (a capture fails
    on any allocation, stream or event creation inside it) and replayed, with
    the library's allocation count unchanged, every replay bit-identical to the
    eager call.  (Launches under capture never share tiles between workgroups,
    so the eager call it is compared with is made with sharing switched off.)"""
    import torch
    from ulmblas_amd import blas
    L = lib.load()
    m, n = 1100, 900
    ld = m + 1
    A0 = to_device(synth.matrix(403, m, n, ld))
    dA = A0.clone()
    piv = torch.full((min(m, n),), -1, dtype=torch.int32, device="cuda")
    info = torch.full((1,), -7, dtype=torch.int32, device="cuda")
    side = torch.cuda.Stream()

    def enqueue(stream):
        assert L.ulmblas_gpu_dgetrf_static(m, n, _p(dA), ld, _p(piv), _p(info), C.c_void_p(stream)) == 0, \
            L.ulmblas_gpu_last_error()

    blas.test_control(blas.TEST_SHARED_PIECES, 0)
    try:
        enqueue(side.cuda_stream)           # warm: kernel attributes, the array's address
        torch.cuda.synchronize()
    finally:
        blas.test_control(blas.TEST_SHARED_PIECES, blas.SHARED_PIECES_DEFAULT)
    want = (to_host(dA).copy(), piv.cpu().numpy().copy(), int(info.cpu()[0]))
    assert want[2] == 0
    allocs = L.ulmblas_gpu_alloc_count()
    dA.copy_(A0)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        enqueue(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    for rep in range(3):
        dA.copy_(A0)
        piv.fill_(-1)
        info.fill_(-7)
        _ = (A0 @ torch.ones(A0.shape[1], dtype=torch.float64, device="cuda")).sum().item()     # eager work in between
        g.replay()
        torch.cuda.synchronize()
        assert int(info.cpu()[0]) == 0, rep
        assert np.array_equal(piv.cpu().numpy(), want[1]), rep
        assert to_host(dA).tobytes() == want[0].tobytes(), rep
    assert L.ulmblas_gpu_alloc_count() == allocs


def test_static_rejects_sizes_beyond_its_limit():
    L = lib.load()
    rc = L.ulmblas_gpu_dgetrf_static(65537, 8, None, 65537, None, None, None)
    assert rc == 1 and b"65536" in L.ulmblas_gpu_last_error()
