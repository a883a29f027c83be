"""The device entry points under HIP graph capture: they allocate nothing,
wait for nothing and clear nothing with memset nodes, so a caller can record
a sequence of them (here a ragged dgemm whose strips run on the library's
side streams, a triangular solve and an LU factorisation with its hundreds of
launches) into one graph and replay it.  Every replay is compared bit for bit
with what the same calls produce when run eagerly, with eager work and
synchronisations between the replays.  Launches that are being captured never
share tiles between workgroups along k (a replay would reuse the flags of the
capture), so the eager run the replays are held against bit for bit is made
with sharing switched off; the eager run as the planner launches it is held
against it within the parity bound."""
import ctypes as C

import numpy as np
import pytest

from gpu_util import to_device, to_host
from ulmblas_amd import blas, lib, synth

pytestmark = pytest.mark.gpu


def _p(x):
    return C.c_void_p(x.data_ptr())


def test_capture_and_replay():
    import torch
    L = lib.load()
    m, n, k = 1000, 777, 515                       # whole tiles plus strips
    A = to_device(synth.matrix(301, m, k, m + 3))
    B = to_device(synth.matrix(302, k, n, k + 1))
    C0 = to_device(synth.matrix(303, m, n, m + 2))
    nt = 900                                       # trsm: blocks, a ragged tail, GEMM updates
    T0 = synth.matrix(304, nt, nt, nt)
    T0[np.arange(nt), np.arange(nt)] += 4.0
    Tm = to_device(T0)
    R0 = to_device(synth.matrix(305, nt, 130, nt))
    nl = 1100                                      # LU: 18 panels, several groups per panel
    F0 = to_device(synth.matrix(306, nl, nl, nl))
    piv = torch.zeros(nl, dtype=torch.int32, device="cuda")
    info = torch.zeros(1, dtype=torch.int32, device="cuda")
    work = torch.zeros((L.ulmblas_gpu_dgetrf_worksize() + 7) // 8, dtype=torch.float64, device="cuda")
    Cc, Rr, Ff = C0.clone(), R0.clone(), F0.clone()

    def enqueue(stream):
        s = C.c_void_p(stream)
        assert L.ulmblas_gpu_dgemm(0, 0, m, n, k, 0.75, _p(A), m + 3, _p(B), k + 1, -0.5, _p(Cc), m + 2, s) == 0
        assert L.ulmblas_gpu_dtrsm(0, 1, 0, 0, nt, 130, 1.0, _p(Tm), nt, _p(Rr), nt, s) == 0
        assert L.ulmblas_gpu_dgetrf(nl, nl, _p(Ff), nl, _p(piv), _p(info), _p(work), s) == 0

    def restore():
        Cc.copy_(C0)
        Rr.copy_(R0)
        Ff.copy_(F0)
        piv.fill_(-1)
        info.fill_(-7)
        torch.cuda.synchronize()

    # eager: also the warm-up that creates the library's side streams and sets kernel attributes
    side = torch.cuda.Stream()
    restore()
    enqueue(side.cuda_stream)
    torch.cuda.synchronize()
    planned = [to_host(Cc).copy(), to_host(Rr).copy(), to_host(Ff).copy(), piv.cpu().numpy().copy(), int(info.cpu()[0])]
    restore()
    blas.test_control(blas.TEST_SHARED_PIECES, 0)
    try:
        enqueue(side.cuda_stream)
        torch.cuda.synchronize()
    finally:
        blas.test_control(blas.TEST_SHARED_PIECES, blas.SHARED_PIECES_DEFAULT)
    want = [to_host(Cc).copy(), to_host(Rr).copy(), to_host(Ff).copy(), piv.cpu().numpy().copy(), int(info.cpu()[0])]
    assert want[4] == 0 and planned[4] == 0 and np.array_equal(planned[3], want[3])
    for a, b in zip(planned[:3], want[:3]):
        assert np.abs(a - b).max() <= 1e-10 * max(1.0, np.abs(b).max())

    restore()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        enqueue(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    for rep in range(4):
        restore()
        # eager work of the program's own between the replays
        _ = (C0 @ torch.ones(C0.shape[1], dtype=torch.float64, device="cuda")).sum().item()
        g.replay()
        torch.cuda.synchronize()
        got = [to_host(Cc), to_host(Rr), to_host(Ff), piv.cpu().numpy(), int(info.cpu()[0])]
        assert got[4] == 0, rep
        assert np.array_equal(got[3], want[3]), rep
        for a, b, name in zip(got[:3], want[:3], ("gemm", "trsm", "getrf")):
            assert a.tobytes() == b.tobytes(), (rep, name)
