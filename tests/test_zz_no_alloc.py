"""homGemmF16NoAlloc: the GEMM entry point that never allocates.

Its split-K partial tiles live in a fixed device array inside the library
instead of the grow-only buffer cutlassGemmF16 allocates.  Same kernels, so the
bar is bit equality with cutlassGemmF16 on the same inputs -- on two calls in a
row, the second with a smaller problem (the array still holds the first call's
partial tiles) -- plus parity with the oracle (rtol 1e-3 / atol 1e-2) and a
clean rejection of a problem whose partial tiles exceed the array.
"""
import importlib

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

GEMM_TOL = dict(rtol=1e-3, atol=1e-2)


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _knum(rt, tag):
    hits = [i for i, n, act, _ in rt.manifest() if tag in n and n.endswith("_linear")]
    assert hits, tag
    return hits[0] + 1


def _run(fn, rt, A, B, C, beta, num, sk):
    M = rt.MemRef.from_tensor
    ta, tb = _dev(A), _dev(B)
    td = torch.zeros((A.shape[0], A.shape[1], B.shape[2]), dtype=torch.float16, device="cuda")
    tc = _dev(C) if C is not None else td
    fn(*M(ta).args(), False, *M(tb).args(), False, *M(tc).args(), *M(td).args(), 0, 1.0, beta, num, sk)
    torch.cuda.synchronize()
    return td.cpu().numpy()


def test_no_alloc_gemm_matches_allocating_entry_point(gpu, rt, oracle):
    g = np.random.default_rng(77)
    num = _knum(rt, "64x64_64x2r2_w2x2")
    # (M, N, K, splitK): first the larger problem, then smaller ones that reuse
    # the array's leading bytes; ragged shapes and a residual source included
    cases = [(192, 1024, 4096, 8, False), (64, 512, 1024, 4, False), (72, 40, 392, 3, True),
             (64, 64, 256, 1, False)]
    for (M_, N_, K_, sk, with_c) in cases:
        A = g.standard_normal((1, M_, K_)).astype(np.float16)
        B = (g.standard_normal((1, K_, N_)) * 0.05).astype(np.float16)
        C = g.standard_normal((1, M_, N_)).astype(np.float16) if with_c else None
        beta = 1.0 if with_c else 0.0
        want = _run(gpu.cutlassGemmF16, rt, A, B, C, beta, num, sk)
        generation = gpu.homScratchGeneration()
        got = _run(gpu.homGemmF16NoAlloc, rt, A, B, C, beta, num, sk)
        assert gpu.homScratchGeneration() == generation, "the no-alloc entry point grew the library's scratch"
        assert np.array_equal(got, want), f"no-alloc GEMM differs from cutlassGemmF16 at {(M_, N_, K_, sk)}"
        ref = oracle.gemm(A[0], B[0], C[0] if with_c else None, beta=beta)
        err = np.abs(got[0].astype(np.float64) - ref)
        assert (err <= GEMM_TOL["atol"] + GEMM_TOL["rtol"] * np.abs(ref)).all(), (M_, N_, K_, sk, err.max())
    # library-selected kernel (gemmNum 0) on a shape whose tuned entry slices K
    A = g.standard_normal((1, 64, 4096)).astype(np.float16)
    B = (g.standard_normal((1, 4096, 1024)) * 0.02).astype(np.float16)
    assert np.array_equal(_run(gpu.homGemmF16NoAlloc, rt, A, B, None, 0.0, 0, 1),
                          _run(gpu.cutlassGemmF16, rt, A, B, None, 0.0, 0, 1))


def test_no_alloc_gemm_shrinks_a_split_k_it_chose_itself(gpu, rt, oracle):
    """gemmNum 0 leaves kernel and split-K to the library.  Whatever it picks, the call must neither
    allocate nor fail for a problem whose sliced partial tiles could exceed the array: 4096 x 4096
    outputs are 64 MiB per slice, so any factor above 1 is shrunk to 1."""
    g = np.random.default_rng(78)
    A = g.standard_normal((1, 4096, 256)).astype(np.float16)
    B = (g.standard_normal((1, 256, 4096)) * 0.05).astype(np.float16)
    generation = gpu.homScratchGeneration()
    got = _run(gpu.homGemmF16NoAlloc, rt, A, B, None, 0.0, 0, 1)
    assert gpu.homScratchGeneration() == generation
    rows = np.arange(0, 4096, 97)
    ref = oracle.gemm(np.ascontiguousarray(A[0][rows]), B[0])
    err = np.abs(got[0][rows].astype(np.float64) - ref)
    assert (err <= GEMM_TOL["atol"] + GEMM_TOL["rtol"] * np.abs(ref)).all(), err.max()


def test_no_alloc_gemm_rejects_oversized_split_k(gpu, rt):
    # 2048 x 2048 outputs x 4 slices x 4 bytes = 64 MiB of partial tiles > 32 MiB
    M = rt.MemRef.from_tensor
    ta = torch.zeros((1, 2048, 512), dtype=torch.float16, device="cuda")
    tb = torch.zeros((1, 512, 2048), dtype=torch.float16, device="cuda")
    td = torch.full((1, 2048, 2048), 3.0, dtype=torch.float16, device="cuda")
    gpu.homSetErrorMode(1)
    try:
        gpu.homGetLastError()
        gpu.homGemmF16NoAlloc(*M(ta).args(), False, *M(tb).args(), False, *M(td).args(), *M(td).args(),
                              0, 1.0, 0.0, _knum(rt, "64x64_64x2r2_w2x2"), 4)
        msg = gpu.homGetLastError().decode()
    finally:
        gpu.homSetErrorMode(0)
    assert "workspace" in msg and "bytes" in msg, msg
    torch.cuda.synchronize()
    assert (td.cpu().numpy() == 3.0).all(), "a rejected call must not launch anything"
