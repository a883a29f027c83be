#!/usr/bin/env python3
"""Headline benchmark: device-resident dgemm on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

A step is one call of ulmblas_gpu_dgemm / ulmblas_gpu_sgemm (the device entry
point behind dgemm_ / cblas_dgemm) on seeded synthetic operands that already
sit in HBM.  The default workload is the one the metric is quoted on:
column-major dgemm N,N, m = n = k = 8192, alpha = 1, beta = 0, C pre-filled
with NaN.  One JSON line is printed.

  value         whole-job GFLOP/s over the timed steps (2 m n k per step)
  roofline      the gemm kernel against the MI355X matrix-core peak, from HIP
                events around every launch on the launch stream
  cpu_baseline  the reference's CPU GEMM (built from its own sources where that
                library travelled with the tree, else this repository's
                restatement of it), one thread, on a column panel of the same
                product
  end_to_end    the same product through dgemm_ on host memory (H2D + kernel +
                D2H), one call
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"d": 78.6, "s": 157.3, "z": 78.6, "c": 157.3}          # MI355X dense matrix peak, FP64 / FP32
HBM_PEAK_GBS = 8000.0

# name -> (precision, transA, transB, m, n, k, alpha, beta, distribution)
WORKLOADS = {
    "dgemm_nn_8192": ("d", "N", "N", 8192, 8192, 8192, 1.0, 0.0, "uniform"),
    "dgemm_tn_8192": ("d", "T", "N", 8192, 8192, 8192, 1.0, 0.0, "uniform"),
    "dgemm_nt_8192": ("d", "N", "T", 8192, 8192, 8192, 1.0, 0.0, "uniform"),
    "dgemm_tt_8192": ("d", "T", "T", 8192, 8192, 8192, 1.0, 0.0, "uniform"),
    "dgemm_nn_4096": ("d", "N", "N", 4096, 4096, 4096, 1.0, 0.0, "uniform"),
    "dgemm_nn_2048": ("d", "N", "N", 2048, 2048, 2048, 1.0, 0.0, "uniform"),
    "dgemm_nn_512": ("d", "N", "N", 512, 512, 512, 1.0, 0.0, "uniform"),
    "sgemm_nt_4096": ("s", "N", "T", 4096, 4096, 4096, 1.0, 1.0, "normal"),
    "sgemm_nt_1024": ("s", "N", "T", 1024, 1024, 1024, 1.0, 1.0, "normal"),
    "dgemm_nn_16384": ("d", "N", "N", 16384, 16384, 16384, 1.0, 0.0, "uniform"),
    "dgemm_nn_1024": ("d", "N", "N", 1024, 1024, 1024, 1.5, 0.5, "uniform"),
    "sgemm_nt_8192": ("s", "N", "T", 8192, 8192, 8192, 1.0, 1.0, "normal"),
    "sgemm_nt_16384": ("s", "N", "T", 16384, 16384, 16384, 1.0, 1.0, "normal"),
    "dgemm_rankk_16384x256": ("d", "N", "N", 16384, 16384, 256, -1.0, 1.0, "uniform"),
    "dgemm_tall_65536x64x1024": ("d", "N", "N", 65536, 64, 1024, -1.0, 1.0, "uniform"),
    "dgemm_wide_64x65536x1024": ("d", "N", "N", 64, 65536, 1024, -1.0, 1.0, "uniform"),
    "dgemm_tn_strided_5000x3000x7000": ("d", "T", "N", 5000, 3000, 7000, 0.75, -0.25, "uniform"),
    # shapes outside the published sweep: no multiple of any tile, and few tiles with a long k
    "dgemm_nn_1000": ("d", "N", "N", 1000, 1000, 1000, 1.0, 0.0, "uniform"),
    "dgemm_nn_3000": ("d", "N", "N", 3000, 3000, 3000, 1.0, 0.0, "uniform"),
    "sgemm_nn_3000": ("s", "N", "N", 3000, 3000, 3000, 1.0, 0.0, "uniform"),
    "dgemm_nn_256x256x65536": ("d", "N", "N", 256, 256, 65536, 1.0, 0.0, "uniform"),
    "dgemm_tn_200x200x20000": ("d", "T", "N", 200, 200, 20000, 1.0, 0.0, "uniform"),
}

def measured_traffic(workload):
    """HBM bytes per launch of the gemm kernel from the rocprofv3 --pmc FETCH_SIZE /
    WRITE_SIZE runs of this script, each scaled by what the same counter reads
    for a device-to-device copy of known size: profiles/traffic.json, written
    together with the summaries under profiles/.  None = not measured."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            return json.load(f).get(workload, {}).get("bytes_per_launch")
    except (OSError, ValueError):
        return None


def algorithmic_bytes(prec, m, n, k, beta):
    s = 8 if prec == "d" else 4
    return s * (m * k + k * n + m * n * (2 if beta != 0 else 1))


def make_operands(prec, ta, tb, m, n, k, beta, dist, pads=(0, 0, 0)):
    from ulmblas_amd import synth
    dt = np.float64 if prec == "d" else np.float32
    ra, ca = (k, m) if ta == "T" else (m, k)
    rb, cb = (n, k) if tb == "T" else (k, n)
    lda, ldb, ldc = ra + pads[0], rb + pads[1], m + pads[2]
    A = synth.matrix(1001, ra, ca, lda, dist=dist, dtype=dt)
    B = synth.matrix(1002, rb, cb, ldb, dist=dist, dtype=dt)
    C = synth.matrix(1003, m, n, ldc, dist=dist, dtype=dt)
    if beta == 0.0:
        C[:m, :] = np.nan
    return A, B, C, (lda, ldb, ldc)


def cpu_baseline(prec, ta, tb, m, n, k, alpha, beta, A, lda, B, ldb, C, ldc, target_seconds=10.0):
    """Reference CPU GEMM, one thread, on the leading columns of the same
    product (a column panel of C and of op(B)), each build timed for about
    target_seconds: the reference as its own make.inc builds it (SSE3 assembly
    micro-kernel; `value`) and with its portable micro-kernel (`portable`),
    which is the build the parity tests use.  The panel's C is finite (the SSE
    kernel turns beta == 0 on NaN into NaN, ukernel/sse/ugemm.tcc:302-306).
    Where the compiled reference did not travel with the tree, this
    repository's restatement of it is timed instead (kind "port")."""
    from oracle import oracle as O
    variant = "d" if prec == "d" else "s"
    Cfin = np.nan_to_num(C, nan=0.5)

    def timed(f, what):
        def run(ns):
            if tb == "T":
                Bp = B                                           # stored B is n x k: rows 0..ns-1, same ld
            else:
                Bp = np.asfortranarray(B[:, :ns])
            Cp = np.asfortranarray(Cfin[:, :ns]).copy(order="F")
            t0 = time.perf_counter()
            f(variant, ta, tb, m, ns, k, alpha, A, lda, Bp, ldb, beta, Cp, ldc)
            return time.perf_counter() - t0

        # a panel of about one second first, at least 256 columns wide (narrower ones under-read the rate: the
        # packing of A is spread over fewer columns), to size the timed one for this core; its first pass also
        # touches the operands and the library's pool for the first time, the second one gives the rate
        ns0 = int(min(n, max(256, 3.0e10 // (2.0 * m * k))))
        run(ns0)
        rate = 2.0 * m * ns0 * k / run(ns0)
        ns = int(min(n, max(64, (target_seconds * rate) // (2.0 * m * k))))
        dt = run(ns)
        return {"value": round(2.0 * m * ns * k / dt / 1e9, 3), "seconds": round(dt, 1),
                "sample": f"columns 0..{ns - 1} of C (m={m}, n={ns}, k={k}) of the same product, {dt:.1f} s, {what}"}

    if O.have_ref("libulmref_sse.so") and O.have_ref():
        sse = timed(lambda *a: O.ref_gemm(*a, libname="libulmref_sse.so"),
                    "ulmBLAS::gemm compiled from the reference headers with its own flags (make.inc:12-13: -msse3 "
                    "-mfpmath=sse -O3 -fomit-frame-pointer; SSE3 assembly micro-kernel)")
        portable = timed(O.ref_gemm, "ulmBLAS::gemm compiled from the reference headers without -msse3 (portable "
                                     "micro-kernel, -O3)")
        return {"value": sse["value"], "unit": "GFLOP/s", "cores": 1, "host_cores": os.cpu_count(), "kind": "reference",
                "sample": sse["sample"], "portable": {"value": portable["value"], "unit": "GFLOP/s",
                                                      "sample": portable["sample"]}}
    use_ref = O.have_ref()
    one = timed(O.ref_gemm if use_ref else O.gemm,
                "ulmBLAS::gemm compiled from the reference headers (portable micro-kernel, -O3)" if use_ref
                else "this repository's C restatement of ulmBLAS gemm (-O3)")
    return {"value": one["value"], "unit": "GFLOP/s", "cores": 1, "host_cores": os.cpu_count(),
            "kind": "reference" if use_ref else "port", "sample": one["sample"]}


# name -> (precision, side, uplo, transA, diag, m, n, alpha)
TRSM_WORKLOADS = {
    "dtrsm_llnn_8192": ("d", "L", "L", "N", "N", 8192, 8192, 1.0),
    "dtrsm_lunn_8192": ("d", "L", "U", "N", "N", 8192, 8192, 1.0),
    "dtrsm_rutn_8192": ("d", "R", "U", "T", "N", 8192, 8192, 1.0),
    "dtrsm_llnu_256x16384": ("d", "L", "L", "N", "U", 256, 16384, 1.0),     # the solve of one LU step
    "dtrsm_llnn_2048": ("d", "L", "L", "N", "N", 2048, 2048, 1.0),
    "dtrsm_llnn_3000": ("d", "L", "L", "N", "N", 3000, 3000, 1.0),
    "strsm_llnn_8192": ("s", "L", "L", "N", "N", 8192, 8192, 1.0),
}


def run_trsm(args):
    """Device-resident triangular solve: a step is one ulmblas_gpu_?trsm call
    (B is restored from a copy before every step, outside the timed events)."""
    import torch
    from ulmblas_amd import blas, synth
    prec, side, uplo, trans, diag, m, n, alpha = TRSM_WORKLOADS[args.workload]
    dt = np.float64 if prec == "d" else np.float32
    na = m if side == "L" else n
    A = synth.matrix(2001, na, na, na, dtype=dt)
    A *= dt(min(1.0, 8.0 / na))                       # keep the triangle well conditioned
    idx = np.arange(na)
    A[idx, idx] += np.where(A[idx, idx] < 0, -2.0, 2.0).astype(dt)
    B0 = synth.matrix(2002, m, n, m, dtype=dt)
    torch.cuda.set_device(0)
    dA = torch.from_numpy(A.T).cuda()
    dB0 = torch.from_numpy(B0.T).cuda()
    dB = dB0.clone()
    f = blas.gpu_dtrsm if prec == "d" else blas.gpu_strsm
    stream = torch.cuda.current_stream()

    def step():
        f(side == "R", uplo == "L", trans == "T", diag == "U", m, n, alpha, dA, na, dB, m, stream=stream.cuda_stream)

    for _ in range(args.warmup):
        dB.copy_(dB0)
        step()
    torch.cuda.synchronize()
    ms = []
    t_all = 0.0
    for _ in range(args.steps):
        dB.copy_(dB0)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0.record(stream)
        step()
        e1.record(stream)
        torch.cuda.synchronize()
        t_all += time.perf_counter() - t0
        ms.append(e0.elapsed_time(e1))
    flops = float(na) * na * (n if side == "L" else m)
    avg_s = sum(ms) / len(ms) / 1e3
    s = 8 if prec == "d" else 4
    abytes = s * (na * (na + 1) // 2 + 2 * m * n)
    result = {
        "metric": f"{prec}trsm GFLOP/s ({args.workload})", "value": round(flops * args.steps / t_all / 1e9, 1),
        "unit": "GFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(t_all / args.steps * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f64" if prec == "d" else "f32",
        "data": "synthetic (seeded splitmix64 uniform, scaled triangle), operands resident in HBM",
        "config": {"workload": args.workload, "side": side, "uplo": uplo, "transA": trans, "diag": diag, "m": m,
                   "n": n, "alpha": alpha},
        "pct_of_peak": round(100.0 * flops / avg_s / 1e12 / PEAK_TFLOPS[prec], 2),
        "roofline": {"bound": "mfma", "achieved": round(flops / avg_s / 1e12, 3), "peak": PEAK_TFLOPS[prec],
                     "unit": "TFLOP/s", "frac": round(flops / avg_s / 1e12 / PEAK_TFLOPS[prec], 4), "traffic": None,
                     "kernel_ms_avg": round(avg_s * 1e3, 4), "kernel_ms_min": round(min(ms), 4),
                     "algorithmic_bytes": abytes, "algorithmic_GBps": round(abytes / avg_s / 1e9, 1),
                     "hbm_frac": round(abytes / avg_s / 1e9 / HBM_PEAK_GBS, 4)},
    }
    return result


# name -> (m, n)
LU_WORKLOADS = {
    "dgetrf_8192": (8192, 8192),
    "dgetrf_16384": (16384, 16384),
    "dgetrf_4096": (4096, 4096),
    "dgetrf_2048": (2048, 2048),
    "dgetrf_1024": (1024, 1024),
    "dgetrf_tall_16384x4096": (16384, 4096),
}


def run_lu(args):
    """Device-resident LU: a step is one ulmblas_gpu_dgetrf call (A restored
    from a copy before every step, outside the timed events)."""
    import torch
    from ulmblas_amd import blas, synth
    m, n = LU_WORKLOADS[args.workload]
    A0 = synth.matrix(3001, m, n, m)
    torch.cuda.set_device(0)
    dA0 = torch.from_numpy(A0.T).cuda()
    dA = dA0.clone()
    stream = torch.cuda.current_stream()
    for _ in range(args.warmup):
        dA.copy_(dA0)
        blas.gpu_dgetrf(m, n, dA, m, stream=stream.cuda_stream)
    torch.cuda.synchronize()
    ms, t_all = [], 0.0
    for _ in range(args.steps):
        dA.copy_(dA0)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0.record(stream)
        dPiv, dInfo = blas.gpu_dgetrf(m, n, dA, m, stream=stream.cuda_stream)
        e1.record(stream)
        torch.cuda.synchronize()
        t_all += time.perf_counter() - t0
        ms.append(e0.elapsed_time(e1))
    assert int(dInfo.cpu()[0]) == 0
    mn = min(m, n)
    flops = float(m) * n * mn - (m + n) * mn * mn / 2.0 + mn ** 3 / 3.0        # LAPACK's count for getrf
    avg_s = sum(ms) / len(ms) / 1e3
    abytes = 8 * 2 * m * n
    result = {
        "metric": f"dgetrf GFLOP/s ({args.workload})", "value": round(flops * args.steps / t_all / 1e9, 1),
        "unit": "GFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(t_all / args.steps * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f64",
        "data": "synthetic (seeded splitmix64 uniform[-1,1)), matrix resident in HBM",
        "config": {"workload": args.workload, "m": m, "n": n, "lda": m},
        "pct_of_peak": round(100.0 * flops / avg_s / 1e12 / PEAK_TFLOPS["d"], 2),
        "roofline": {"bound": "mfma", "achieved": round(flops / avg_s / 1e12, 3), "peak": PEAK_TFLOPS["d"],
                     "unit": "TFLOP/s", "frac": round(flops / avg_s / 1e12 / PEAK_TFLOPS["d"], 4), "traffic": None,
                     "kernel_ms_avg": round(avg_s * 1e3, 4), "kernel_ms_min": round(min(ms), 4),
                     "algorithmic_bytes": abytes, "algorithmic_GBps": round(abytes / avg_s / 1e9, 1),
                     "hbm_frac": round(abytes / avg_s / 1e9 / HBM_PEAK_GBS, 4)},
    }
    return result


# name -> (routine, prec, flags..., sizes)
L3_WORKLOADS = {
    "dsyrk_ln_8192": ("syrk", "d", "L", "N", 8192, 8192),
    "dsyrk_ut_8192": ("syrk", "d", "U", "T", 8192, 8192),
    "dsyrk_ln_8192x512": ("syrk", "d", "L", "N", 8192, 512),       # the trailing update of a blocked Cholesky
    "dsyrk_ln_5000": ("syrk", "d", "L", "N", 5000, 5000),           # 19 blocks of 256 and 136 rows beyond them
    "dsyrk_ln_1000": ("syrk", "d", "L", "N", 1000, 1000),
    "ssyrk_ln_8192": ("syrk", "s", "L", "N", 8192, 8192),
    "dsyr2k_ln_8192": ("syr2k", "d", "L", "N", 8192, 8192),
    "dsyr2k_ut_8192x512": ("syr2k", "d", "U", "T", 8192, 512),
    "zgemm_nn_8192": ("cgemm", "z", "N", "N", 8192, 8192, 8192),
    "zgemm_ct_8192": ("cgemm", "z", "C", "T", 8192, 8192, 8192),
    "zgemm_nn_4096": ("cgemm", "z", "N", "N", 4096, 4096, 4096),
    "cgemm_nn_8192": ("cgemm", "c", "N", "N", 8192, 8192, 8192),
    "dsymm_ll_8192": ("symm", "d", "L", "L", 8192, 8192),
    "dsymm_ru_8192": ("symm", "d", "R", "U", 8192, 8192),
    "ssymm_ll_8192": ("symm", "s", "L", "L", 8192, 8192),
    "dtrmm_llnn_8192": ("trmm", "d", "L", "L", "N", "N", 8192, 8192),
    "dtrmm_rutn_8192": ("trmm", "d", "R", "U", "T", "N", 8192, 8192),
    "strmm_llnn_8192": ("trmm", "s", "L", "L", "N", "N", 8192, 8192),
}


def run_l3(args):
    """Device-resident symmetric rank-k update, symmetric product or
    triangular product: a step is one ulmblas_gpu_? call.  Flops are the
    algorithm's (the triangle only): n(n+1)k for syrk (twice that for syr2k), 2 ka m n for symm,
    ka m n for trmm."""
    import torch
    from ulmblas_amd import blas, synth
    w = L3_WORKLOADS[args.workload]
    routine, prec = w[0], w[1]
    dt = np.float64 if prec in "dz" else np.float32
    tdt = torch.float64 if prec in "dz" else torch.float32
    s = 8 if prec in "dz" else 4
    torch.cuda.set_device(0)
    stream = torch.cuda.current_stream()
    restore = None
    if routine == "cgemm":
        ta, tb, m, n, k = w[2:]
        cdt = np.complex128 if prec == "z" else np.complex64

        def cm(seed, rows, cols):
            z = synth.matrix(seed, rows, cols, rows, dtype=dt) + 1j * synth.matrix(seed + 50, rows, cols, rows, dtype=dt)
            return torch.from_numpy(np.ascontiguousarray(z.astype(cdt).T)).cuda()

        dA = cm(3010, *((k, m) if ta in "TC" else (m, k)))
        dB = cm(3011, *((n, k) if tb in "TC" else (k, n)))
        dC = cm(3012, m, n)
        size = getattr(blas.load(), f"ulmblas_gpu_{prec}gemm_worksize")(blas.TRANS_OF_CHAR[tb], m, n, k)
        work = torch.empty(max(size, 16), dtype=torch.uint8, device="cuda")
        flops = 8.0 * m * n * k
        abytes = 2 * s * (m * k + k * n + 2 * m * n)
        cfg = {"transA": ta, "transB": tb, "m": m, "n": n, "k": k, "alpha": "0.7-0.9i", "beta": "0.5"}

        def step():
            blas.gpu_cgemm(prec, ta, tb, m, n, k, 0.7 - 0.9j, dA, dA.shape[1], dB, dB.shape[1], 0.5, dC, m,
                           stream=stream.cuda_stream, work=work)
    elif routine in ("syrk", "syr2k"):
        uplo, trans, n, k = w[2:]
        ra, ca = (k, n) if trans == "T" else (n, k)
        two = routine == "syr2k"
        dA = torch.from_numpy(synth.matrix(3001, ra, ca, ra, dtype=dt).T).cuda()
        dB = torch.from_numpy(synth.matrix(3008, ra, ca, ra, dtype=dt).T).cuda() if two else None
        dC = torch.from_numpy(synth.matrix(3002, n, n, n, dtype=dt).T).cuda()
        flops = float(n) * (n + 1) * k * (2 if two else 1)
        abytes = s * (n * k * (2 if two else 1) + n * (n + 1))
        cfg = {"uplo": uplo, "trans": trans, "n": n, "k": k, "alpha": 1.0 / (2 if two else 1), "beta": 0.5}

        def step():
            if two:
                blas.gpu_syr2k(prec, uplo == "L", trans == "T", n, k, 0.5, dA, ra, dB, ra, 0.5, dC, n,
                               stream=stream.cuda_stream)
            else:
                blas.gpu_syrk(prec, uplo == "L", trans == "T", n, k, 1.0, dA, ra, 0.5, dC, n,
                              stream=stream.cuda_stream)
    elif routine == "symm":
        side, uplo, m, n = w[2:]
        ka = m if side == "L" else n
        dA = torch.from_numpy(synth.matrix(3003, ka, ka, ka, dtype=dt).T).cuda()
        dB = torch.from_numpy(synth.matrix(3004, m, n, m, dtype=dt).T).cuda()
        dC = torch.from_numpy(synth.matrix(3005, m, n, m, dtype=dt).T).cuda()
        work = torch.empty(min(ka, 2048) ** 2, dtype=tdt, device="cuda")
        flops = 2.0 * ka * m * n
        abytes = s * (ka * (ka + 1) // 2 + 3 * m * n)
        cfg = {"side": side, "uplo": uplo, "m": m, "n": n, "alpha": 1.0, "beta": 0.5}

        def step():
            blas.gpu_symm(prec, side == "R", uplo == "L", m, n, 1.0, dA, ka, dB, m, 0.5, dC, m, work,
                          stream=stream.cuda_stream)
    else:
        side, uplo, trans, diag, m, n = w[2:]
        ka = m if side == "L" else n
        A = synth.matrix(3006, ka, ka, ka, dtype=dt)
        A *= dt(min(1.0, 8.0 / ka))                   # keeps repeated products in range
        dA = torch.from_numpy(A.T).cuda()
        dB0 = torch.from_numpy(synth.matrix(3007, m, n, m, dtype=dt).T).cuda()
        dB = dB0.clone()
        flops = float(ka) * m * n
        abytes = s * (ka * (ka + 1) // 2 + 2 * m * n)
        cfg = {"side": side, "uplo": uplo, "transA": trans, "diag": diag, "m": m, "n": n, "alpha": 1.0}

        def restore():
            dB.copy_(dB0)

        def step():
            blas.gpu_trmm(prec, side == "R", uplo == "L", trans == "T", diag == "U", m, n, 1.0, dA, ka, dB, m,
                          stream=stream.cuda_stream)

    for _ in range(args.warmup):
        if restore:
            restore()
        step()
    torch.cuda.synchronize()
    ms = []
    t_all = 0.0
    for _ in range(args.steps):
        if restore:
            restore()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0.record(stream)
        step()
        e1.record(stream)
        torch.cuda.synchronize()
        t_all += time.perf_counter() - t0
        ms.append(e0.elapsed_time(e1))
    avg_s = sum(ms) / len(ms) / 1e3
    cfg["workload"] = args.workload
    result = {
        "metric": f"{prec}{'gemm' if routine == 'cgemm' else routine} GFLOP/s ({args.workload})", "value": round(flops * args.steps / t_all / 1e9, 1),
        "unit": "GFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(t_all / args.steps * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": {"d": "f64", "s": "f32", "z": "c128 (f64 arithmetic)", "c": "c64 (f32 arithmetic)"}[prec],
        "data": "synthetic (seeded splitmix64 uniform), operands resident in HBM", "config": cfg,
        "pct_of_peak": round(100.0 * flops / avg_s / 1e12 / PEAK_TFLOPS[prec], 2),
        "roofline": {"bound": "mfma", "achieved": round(flops / avg_s / 1e12, 3), "peak": PEAK_TFLOPS[prec],
                     "unit": "TFLOP/s", "frac": round(flops / avg_s / 1e12 / PEAK_TFLOPS[prec], 4), "traffic": None,
                     "kernel_ms_avg": round(avg_s * 1e3, 4), "kernel_ms_min": round(min(ms), 4),
                     "algorithmic_bytes": abytes, "algorithmic_GBps": round(abytes / avg_s / 1e9, 1),
                     "hbm_frac": round(abytes / avg_s / 1e9 / HBM_PEAK_GBS, 4)},
    }
    return result


# The routines built on the GEMM (triangular solve, LU, rank-k update, complex
# product), timed after the BASELINE workloads in the default run and reported
# as the `next_rows` array of the same JSON line.
NEXT_ROWS = ["dtrsm_llnn_8192", "dtrsm_llnn_3000", "dgetrf_8192", "dsyrk_ln_8192", "dsyrk_ln_8192x512", "zgemm_nn_4096"]


def next_row_entry(name):
    import argparse as _ap
    import torch
    a = _ap.Namespace(workload=name, steps=10, warmup=3)
    if name in LU_WORKLOADS:
        a.steps, a.warmup = 5, 2
    r = (run_trsm if name in TRSM_WORKLOADS else run_lu if name in LU_WORKLOADS else run_l3)(a)
    torch.cuda.empty_cache()
    return {"workload": name, "ms": r["roofline"]["kernel_ms_avg"], "ms_min": r["roofline"]["kernel_ms_min"],
            "steps": a.steps, "warmup": a.warmup, "gflops": round(r["roofline"]["achieved"] * 1e3, 1),
            "frac": r["roofline"]["frac"], "hbm_frac": r["roofline"]["hbm_frac"]}


# The other BASELINE workloads, timed after the headline loop of the default
# run and reported as the `configs` array of the same JSON line.
SWEEP = ["dgemm_tn_8192", "dgemm_nt_8192", "dgemm_tt_8192", "dgemm_nn_512", "dgemm_nn_1024", "dgemm_nn_2048",
         "dgemm_nn_4096", "dgemm_nn_16384", "sgemm_nt_1024", "sgemm_nt_4096", "sgemm_nt_8192", "sgemm_nt_16384",
         "dgemm_rankk_16384x256", "dgemm_tall_65536x64x1024", "dgemm_wide_64x65536x1024",
         "dgemm_tn_strided_5000x3000x7000"]


_timer = None


def timer_lib():
    """libulmblas_timer.so: the timing loop in C (ulmblas_amd/csrc/timer.hip)."""
    global _timer
    if _timer is None:
        import ctypes as C
        from ulmblas_amd import lib
        lib.load()
        path = os.path.join(ROOT, "ulmblas_amd", "libulmblas_timer.so")
        if not os.path.exists(path):
            raise RuntimeError(f"{path} is missing: build it with `make -C ulmblas_amd/csrc`")
        _timer = C.CDLL(path)
        _timer.ulmblas_timer_gemm.argtypes = [C.c_int] * 6 + [C.c_double, C.c_double, C.c_void_p, C.c_int, C.c_void_p,
                                                                C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int,
                                                                C.c_void_p, C.POINTER(C.c_float)]
        _timer.ulmblas_timer_gemm.restype = C.c_int
    return _timer


def operand_set(dA, dB, dC, offset=0):
    """An operand set for time_gemm from three device tensors: for each the
    address `offset` bytes into it and the bytes of its storage from there on."""
    from ulmblas_amd import blas
    return tuple((x.data_ptr() + offset, blas.room(x) - offset) for x in (dA, dB, dC))


def time_gemm(prec, ta, tb, m, n, k, alpha, beta, sets, lda, ldb, ldc, warm, reps, stream):
    """Milliseconds per call of `reps` device-resident calls after `warm`
    untimed ones, call i on operand set i % len(sets); sets: per operand A, B,
    C a pair (device address, bytes of memory from there on), see operand_set.
    HIP events on `stream` around the timed calls.  The kernels trust the
    shapes they are given, and a window that does not fit its memory is a
    memory fault on the GPU: refused here."""
    import ctypes as C
    size = 8 if prec == "d" else 4
    windows = (((k, m) if ta == "T" else (m, k)) + (lda,), ((n, k) if tb == "T" else (k, n)) + (ldb,), (m, n, ldc))
    for q in sets:
        for (addr, room), (rows, cols, ld), what in zip(q, windows, "ABC"):
            need = ((cols - 1) * ld + rows) * size if rows > 0 and cols > 0 else 0
            if ld < max(rows, 1) or room < need:
                raise ValueError(f"time_gemm: {what} is a {rows} x {cols} window with leading dimension {ld} "
                                 f"({need} bytes) in {room} bytes of memory")
    sets = [tuple(addr for addr, _ in q) for q in sets]
    arr = [(C.c_void_p * len(sets))(*[q[j] for q in sets]) for j in range(3)]
    ms = C.c_float(0.0)
    rc = timer_lib().ulmblas_timer_gemm(ord(prec), int(ta == "T"), int(tb == "T"), m, n, k, alpha, beta, arr[0], lda,
                                        arr[1], ldb, arr[2], ldc, len(sets), warm, reps, C.c_void_p(stream), C.byref(ms))
    if rc != 0:
        from ulmblas_amd import lib
        raise RuntimeError(f"ulmblas_timer_gemm: status {rc}: {lib.load().ulmblas_gpu_last_error().decode()}")
    return ms.value / reps


# Above this many bytes of operands a call finds nothing of them in a cache
# when it comes round again (the GPU's last-level cache holds 256 MB).
COLD_ABOVE = 512 << 20
COLD_CYCLE = 5 << 28          # a cold rotation walks through at least 1.25 GB of operands


def sweep_entry(name):
    """One BASELINE workload, device resident, on seeded operands generated on
    the device (the splitmix64 streams of ulmblas_amd.synth): HIP events on
    the launch stream around the timed launches, which the timing loop in C
    issues.  Launches shorter than a few milliseconds are timed after 300
    warm-up launches, because the shader clock needs tens of milliseconds of
    load to reach its steady value.  `ms` / `frac`: every launch on the same
    three matrices, which for the smaller workloads stay in the caches.  Those
    workloads also get `cold_ms` / `cold_frac`: the launches rotate through as
    many operand sets as it takes to walk 1.25 GB, as the reference's timer
    rotates through more than a cache's worth (bench/l3blastst.c:1553-1603)."""
    import torch
    from ulmblas_amd import synth
    prec, ta, tb, m, n, k, alpha, beta, dist = WORKLOADS[name]
    dt = np.float64 if prec == "d" else np.float32
    pads = (37, 11, 5) if "strided" in name else (0, 0, 0)
    ra, ca = (k, m) if ta == "T" else (m, k)
    rb, cb = (n, k) if tb == "T" else (k, n)
    lda, ldb, ldc = ra + pads[0], rb + pads[1], m + pads[2]
    dA = synth.device_matrix(1001, ra, ca, lda, dist=dist, dtype=dt)
    dB = synth.device_matrix(1002, rb, cb, ldb, dist=dist, dtype=dt)
    dC = synth.device_matrix(1003, m, n, ldc, dist=dist, dtype=dt)
    if beta == 0.0:
        dC[:, :m] = float("nan")
    stream = torch.cuda.current_stream()
    flops = 2.0 * m * n * k
    short = flops < 4e11                      # under ~5 ms
    warmup, steps = (300, 100) if short else (3, 10 if flops < 5e12 else 5)
    torch.cuda.synchronize()
    avg = time_gemm(prec, ta, tb, m, n, k, alpha, beta, [operand_set(dA, dB, dC)], lda, ldb, ldc, warmup, steps, stream.cuda_stream)
    assert not torch.isnan(dC[:, :m]).any(), name
    abytes = algorithmic_bytes(prec, m, n, k, beta)
    out = {"workload": name, "ms": round(avg, 5), "steps": steps, "warmup": warmup,
           "gflops": round(flops / avg / 1e6, 1), "frac": round(flops / avg / 1e9 / PEAK_TFLOPS[prec], 4),
           "hbm_frac": round(abytes / avg / 1e6 / HBM_PEAK_GBS, 4)}
    set_bytes = sum(x.numel() * x.element_size() for x in (dA, dB, dC))
    if set_bytes < COLD_ABOVE:
        nsets = -(-COLD_CYCLE // set_bytes)
        sets = [(dA, dB, dC)] + [(dA.clone(), dB.clone(), dC.clone()) for _ in range(nsets - 1)]
        reps = max(2 * nsets, 20)
        torch.cuda.synchronize()
        cold = time_gemm(prec, ta, tb, m, n, k, alpha, beta, [operand_set(*q) for q in sets], lda, ldb, ldc,
                         max(nsets, warmup), reps, stream.cuda_stream)
        out.update({"cold_ms": round(cold, 5), "cold_frac": round(flops / cold / 1e9 / PEAK_TFLOPS[prec], 4),
                    "cold_sets": nsets, "cold_steps": reps})
        del sets
    else:
        out["cache"] = "operands exceed the caches: every launch is cold"
    del dA, dB, dC
    torch.cuda.empty_cache()
    return out


# The reference's own benchmark definition (bench/cases/make.gemm.inc:1-2: xdl3blastst -N 100 4000 100;
# make.gemm_tn.inc, make.gemm_nt.inc, make.gemm_tt.inc: -A 1 t / -B 1 t -N 100 1000 100).  Its timer's
# defaults (bench/l3blastst.c:3510-3860): alpha = beta = 1, leading dimensions = the largest N of the
# sweep, cold caches for every timed call.
REF_SWEEP = {"nn": ("N", "N", 100, 4000, 100), "tn": ("T", "N", 100, 1000, 100), "nt": ("N", "T", 100, 1000, 100),
             "tt": ("T", "T", 100, 1000, 100)}


def ref_sweep():
    """dgemm over the reference's benchmark sweep, device resident: per size
    [n, ms, fraction of the FP64 matrix peak].  Operands: windows of three
    seeded (nmax x columns) matrices, leading dimension nmax; successive calls
    rotate through disjoint windows that together span at least 1.25 GB, so no
    call finds its operands in a cache."""
    import torch
    from ulmblas_amd import synth
    stream = torch.cuda.current_stream()
    out = {"what": "dgemm, m = n = k = N, alpha = beta = 1, ld = largest N of the sweep, cold caches (calls rotate "
                   "through operand windows spanning >= 1.25 GB); entries [N, ms, frac of FP64 matrix peak]"}
    bufs = {}
    for key, (ta, tb, n0, n1, step) in REF_SWEEP.items():
        ld = n1
        if ld not in bufs:
            bufs.clear()
            torch.cuda.empty_cache()
            reps_cols = -(-(3 << 28) // (ld * ld * 8))              # 768 MB per operand
            bufs[ld] = [synth.device_matrix(1001 + j, ld, ld, ld).repeat(reps_cols, 1) for j in range(3)]
        mats = bufs[ld]
        cols = mats[0].shape[0]
        rows_out = []
        for n in range(n0, n1 + 1, step):
            per_col, per_row = cols // n, ld // n
            want = max(2, -(-COLD_CYCLE // (3 * n * n * 8)))
            nsets = min(want, per_col * per_row)
            sets = []
            for q in range(nsets):
                off = ((q // per_row) * n * ld + (q % per_row) * n) * 8
                sets.append(operand_set(*mats, offset=off))
            reps = max(nsets, 10)
            warm = max(nsets, int(3e10 // (2.0 * n ** 3)) if n < 2000 else 3)
            warm = min(warm, 20000)
            ms = time_gemm("d", ta, tb, n, n, n, 1.0, 1.0, sets, ld, ld, ld, warm, reps, stream.cuda_stream)
            rows_out.append([n, round(ms, 5), round(2.0 * n ** 3 / ms / 1e9 / PEAK_TFLOPS["d"], 4)])
            # beta = 1 on the same windows over and over: keep C from growing without bound
            mats[2].mul_(1e-3)
        out[key] = rows_out
    bufs.clear()
    torch.cuda.empty_cache()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="dgemm_nn_8192", choices=sorted(WORKLOADS) + sorted(TRSM_WORKLOADS) + sorted(LU_WORKLOADS) +
                    sorted(L3_WORKLOADS))
    ap.add_argument("--variant", type=int, default=0, help="force a tile variant id (0 = automatic)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-e2e", action="store_true", help="skip the host-memory (H2D+D2H) call")
    ap.add_argument("--no-sweep", action="store_true",
                    help="skip the `configs` array (the other BASELINE workloads), the reference's own benchmark sweep "
                         "(`ref_sweep`) and the routines built on the GEMM (`next_rows`)")
    ap.add_argument("--ref-sweep-only", action="store_true", help="print only the reference's benchmark sweep")
    ap.add_argument("--host-only", action="store_true",
                    help="only the host-memory call of the workload, three times, in a process that loads nothing else "
                         "(for timelines of its transfers and kernels)")
    ap.add_argument("--sweep-only", default=None,
                    help="print only the `configs` entries of these workloads (comma separated, or 'all')")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build drives one GPU; --gpus must be 1 (a multi-GPU run would split C by column "
                 "panels with no exchange step, which is not implemented)")

    if args.sweep_only:
        import torch
        torch.cuda.set_device(0)
        names = SWEEP if args.sweep_only == "all" else args.sweep_only.split(",")
        for nm in names:
            print(json.dumps(sweep_entry(nm)), flush=True)
        return
    if args.ref_sweep_only:
        import torch
        torch.cuda.set_device(0)
        print(json.dumps(ref_sweep()), flush=True)
        return
    if args.workload in TRSM_WORKLOADS:
        return print(json.dumps(run_trsm(args)))
    if args.workload in LU_WORKLOADS:
        return print(json.dumps(run_lu(args)))
    if args.workload in L3_WORKLOADS:
        return print(json.dumps(run_l3(args)))

    from ulmblas_amd import blas

    prec, ta, tb, m, n, k, alpha, beta, dist = WORKLOADS[args.workload]
    pads = (37, 11, 5) if "strided" in args.workload else (0, 0, 0)
    A, B, C0, (lda, ldb, ldc) = make_operands(prec, ta, tb, m, n, k, beta, dist, pads)

    if args.host_only:
        f = blas.dgemm_ if prec == "d" else blas.sgemm_
        times = []
        for _ in range(3):
            host_C = C0.copy(order="F")
            t0 = time.perf_counter()
            f(ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, host_C, ldc)
            times.append(time.perf_counter() - t0)
        print(json.dumps({"workload": args.workload, "host_call_ms": [round(t * 1e3, 2) for t in times],
                          "GFLOP/s": round(2.0 * m * n * k / min(times[1:]) / 1e9, 1)}))
        return
    import torch

    torch.cuda.set_device(0)
    dA = torch.from_numpy(A.T).cuda()
    dB = torch.from_numpy(B.T).cuda()
    dC0 = torch.from_numpy(C0.T).cuda()
    dC = dC0.clone()
    gemm = blas.gpu_dgemm if prec == "d" else blas.gpu_sgemm
    blas.set_variant(prec, args.variant)
    stream = torch.cuda.current_stream()

    def step():
        gemm(ta == "T", tb == "T", m, n, k, alpha, dA, lda, dB, ldb, beta, dC, ldc, stream=stream.cuda_stream)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()

    starts = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps)]
    stops = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        starts[i].record(stream)
        step()
        stops[i].record(stream)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0

    flops = 2.0 * m * n * k
    kernel_ms = [s.elapsed_time(e) for s, e in zip(starts, stops)]
    avg_kernel_s = sum(kernel_ms) / len(kernel_ms) / 1e3
    value = flops * args.steps / wall / 1e9
    achieved_tflops = flops / avg_kernel_s / 1e12
    abytes = algorithmic_bytes(prec, m, n, k, beta)

    # quick sanity of the timed output (full parity lives in tests/)
    out = dC[:, :m]
    assert not torch.isnan(out).any(), "NaN in the result: C was read although beta == 0?"

    result = {
        "metric": "dgemm GFLOP/s at m=n=k=8192 col-major; % of MI355X FP64 MFMA peak"
                  if args.workload == "dgemm_nn_8192" else f"{prec}gemm GFLOP/s ({args.workload})",
        "value": round(value, 1),
        "unit": "GFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall / args.steps * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f64" if prec == "d" else "f32",
        "data": "synthetic (seeded splitmix64 streams of ulmblas_amd/synth.py: uniform[-1,1) / N(0,1) by Box-Muller; "
                "generated on the host for the headline, on the device for the other entries), operands resident in HBM",
        "config": {"workload": args.workload, "transA": ta, "transB": tb, "m": m, "n": n, "k": k, "lda": lda,
                   "ldb": ldb, "ldc": ldc, "alpha": alpha, "beta": beta,
                   "variant": blas.variant_names(prec)[args.variant - 1] if args.variant else "auto"},
        "pct_of_peak": round(100.0 * value / 1e3 / PEAK_TFLOPS[prec], 2),
        "roofline": {
            "bound": "mfma",
            "achieved": round(achieved_tflops, 3),
            "peak": PEAK_TFLOPS[prec],
            "unit": "TFLOP/s",
            "frac": round(achieved_tflops / PEAK_TFLOPS[prec], 4),
            "traffic": measured_traffic(args.workload),
            "kernel_ms_avg": round(avg_kernel_s * 1e3, 4),
            "kernel_ms_min": round(min(kernel_ms), 4),
            "algorithmic_bytes": abytes,
            "algorithmic_GBps": round(abytes / avg_kernel_s / 1e9, 1),
            "hbm_frac": round(abytes / avg_kernel_s / 1e9 / HBM_PEAK_GBS, 4),
        },
    }

    if args.workload == "dgemm_nn_8192" and not args.no_sweep:
        del dA, dB, dC, dC0
        torch.cuda.empty_cache()
        result["configs"] = [sweep_entry(nm) for nm in SWEEP]
        result["ref_sweep"] = ref_sweep()
        result["next_rows"] = [next_row_entry(nm) for nm in NEXT_ROWS]

    if not args.no_e2e:
        host_C = C0.copy(order="F")
        f = blas.dgemm_ if prec == "d" else blas.sgemm_
        f(ta, tb, 64, 64, 64, alpha, A, lda, B, ldb, beta, host_C, ldc)        # create stream / warm the path
        times = []
        for _ in range(3):       # the first call also allocates device buffers and the pinned staging rings
            host_C = C0.copy(order="F")
            t0 = time.perf_counter()
            f(ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, host_C, ldc)
            times.append(time.perf_counter() - t0)
        e2e = min(times[1:])
        result["end_to_end"] = {"value": round(flops / e2e / 1e9, 1), "unit": "GFLOP/s", "ms": round(e2e * 1e3, 2),
                                "first_call_ms": round(times[0] * 1e3, 2),
                                "what": "one %s call on pageable host memory: H2D of A, B (and C if beta != 0), "
                                        "kernel, D2H of C; best of two calls after the first" % f.__name__}

        # the same call on page-locked host memory (hipHostMalloc through torch): the library copies
        # such operands where they lie instead of staging them
        def page_locked(arr):
            t = torch.empty(arr.shape[::-1], dtype=torch.float64 if prec == "d" else torch.float32, pin_memory=True)
            v = t.numpy().T
            v[...] = arr
            return v, t
        (pA, kA), (pB, kB), (pC0, kC0), (pC, kC) = page_locked(A), page_locked(B), page_locked(C0), page_locked(C0)
        times = []
        for _ in range(3):
            pC[...] = pC0
            t0 = time.perf_counter()
            f(ta, tb, m, n, k, alpha, pA, lda, pB, ldb, beta, pC, ldc)
            times.append(time.perf_counter() - t0)
        e2p = min(times[1:])
        result["end_to_end"]["page_locked"] = {"value": round(flops / e2p / 1e9, 1), "unit": "GFLOP/s",
                                               "ms": round(e2p * 1e3, 2),
                                               "same_result": bool(np.array_equal(pC, host_C))}
        # what the bus gives: one 512 MiB copy each way between page-locked host memory and the device
        # (the floor of any end-to-end figure is the larger of upload time and kernel time, plus what
        # cannot overlap: the first panel up and the last panel down)
        probe = torch.empty(64 << 20, dtype=torch.float64, pin_memory=True)
        dprobe = torch.empty(64 << 20, dtype=torch.float64, device="cuda")
        rates = {}
        for name, (dst, src) in (("h2d", (dprobe, probe)), ("d2h", (probe, dprobe))):
            best = 0.0
            for _ in range(3):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(stream)
                dst.copy_(src, non_blocking=True)
                e1.record(stream)
                torch.cuda.synchronize()
                best = max(best, probe.numel() * 8 / e0.elapsed_time(e1) / 1e6)
            rates[name] = best
        s_el = 8 if prec == "d" else 4
        up = s_el * (m * k + k * n + (m * n if beta != 0 else 0))
        down = s_el * m * n
        result["end_to_end"]["bus"] = {"h2d_GBps": round(rates["h2d"], 1), "d2h_GBps": round(rates["d2h"], 1),
                                       "upload_ms": round(up / rates["h2d"] / 1e6, 2),
                                       "download_ms": round(down / rates["d2h"] / 1e6, 2),
                                       "kernel_ms": round(avg_kernel_s * 1e3, 2)}
        del pA, pB, pC0, pC, kA, kB, kC0, kC, probe, dprobe

    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(prec, ta, tb, m, n, k, alpha, beta, A, lda, B, ldb, C0, ldc)

    print(json.dumps(result))


if __name__ == "__main__":
    main()
