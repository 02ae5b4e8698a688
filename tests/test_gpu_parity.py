"""Parity of the HIP kernels with the CPU oracle, called through the C-ABI.

Tolerances (written where they are used):
  GEMM, GEMM+GELU, attention: rtol 1e-3 / atol 1e-2 against the fp32 oracle;
  layer norm: rtol 2e-3 (atol 1e-3 for outputs near zero);
  elementwise, gather, cu_seqlens: bit exact.
"""
import ctypes
import importlib

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

GEMM_TOL = dict(rtol=1e-3, atol=1e-2)
LN_TOL = dict(rtol=2e-3, atol=1e-3)


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def assert_close(got, want, rtol, atol, what=""):
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    err = np.abs(got - want)
    bad = err > atol + rtol * np.abs(want)
    assert not bad.any(), (f"{what}: {bad.sum()} of {bad.size} outside rtol={rtol} atol={atol}; "
                           f"max abs err {err.max():.3e} at {np.unravel_index(err.argmax(), err.shape)}")


# --------------------------------------------------------------- LayerNorm --
@pytest.mark.parametrize("shape", [(8, 128, 768), (1024, 768), (3, 5, 1024), (2, 7, 2048), (4, 4096),
                                   (5, 3, 100), (6, 10), (2, 3, 8200), (1, 1, 8)])
def test_layernorm_f16_in_place(gpu, rt, oracle, shape):
    g = np.random.default_rng(sum(shape))
    x = (g.standard_normal(shape) * 1.5 + 0.3).astype(np.float16)
    t = dev(x)
    gpu.nvteLayernormF16(*rt.MemRef.from_tensor(t).args(), 1e-12)
    assert_close(host(t), oracle.layernorm_f16(x, 1e-12), **LN_TOL, what=f"layernorm {shape}")


def test_layernorm_config2_and_large(gpu, rt, oracle, synth):
    c = synth.add_layernorm()
    t = dev(c["x"].reshape(8, 128, 768))
    gpu.nvteLayernormF16(*rt.MemRef.from_tensor(t).args(), c["eps"])
    assert_close(host(t).reshape(1024, 768), oracle.layernorm_f16(c["x"], c["eps"]), **LN_TOL)
    # fused residual add + affine (superset), out of place and in place
    x, r = dev(c["x"]), dev(c["res"])
    ga, be, out = dev(c["gamma"]), dev(c["beta"]), torch.empty_like(x)
    M = rt.MemRef.from_tensor
    gpu.homAddLayernormF16(*M(x).args(), *M(r).args(), *M(ga).args(), *M(be).args(), *M(out).args(), c["eps"])
    want = oracle.layernorm_f16(c["x"], c["eps"], res=c["res"], gamma=c["gamma"], beta=c["beta"])
    assert_close(host(out), want, **LN_TOL, what="add+layernorm")
    gpu.homAddLayernormF16(*M(x).args(), *M(r).args(), *M(ga).args(), *M(be).args(), *M(x).args(), c["eps"])
    assert np.array_equal(host(x), host(out))
    # with no residual / affine it is exactly the reference form
    y = dev(c["x"])
    gpu.homAddLayernormF16(*M(y).args(), 0, None, 0, None, 0, None, *M(y).args(), c["eps"])
    assert np.array_equal(host(y).reshape(1024, 768), host(t).reshape(1024, 768))
    # BERT-large activation size: oracle on the full tensor + invariants
    g = np.random.default_rng(11)
    big = (g.standard_normal((32, 512, 1024)) * 2).astype(np.float16)
    tb = dev(big)
    gpu.nvteLayernormF16(*M(tb).args(), 1e-12)
    got = host(tb).astype(np.float64)
    assert_close(got, oracle.layernorm_f16(big, 1e-12), **LN_TOL)
    assert np.abs(got.mean(-1)).max() < 2e-3 and np.abs(got.var(-1) - 1).max() < 5e-3


def test_layernorm_f32_reference_literal(gpu, rt, oracle, literals):
    x = np.array(literals["layernorm_2x10"], np.float32).reshape(2, 10)
    t = dev(x)
    gpu.nvteLayernormF32(*rt.MemRef.from_tensor(t).args(), 1e-5)
    assert_close(host(t), oracle.layernorm_f32(x, 1e-5), rtol=1e-5, atol=1e-6)
    g = np.random.default_rng(5)
    x = g.standard_normal((2, 33, 768)).astype(np.float32)
    t = dev(x)
    gpu.nvteLayernormF32(*rt.MemRef.from_tensor(t).args(), 1e-6)
    assert_close(host(t), oracle.layernorm_f32(x, 1e-6), rtol=1e-4, atol=1e-5)


# ------------------------------------------------------------- elementwise --
OPS = ["Add", "Sub", "Mul", "Div"]


@pytest.mark.parametrize("sfx,dtype", [("F16", np.float16), ("F32", np.float32)])
def test_elementwise_bit_exact(gpu, rt, oracle, literals, sfx, dtype):
    g = np.random.default_rng(21)
    cases = [((3, 3, 3), (3, 1, 3)), ((8, 128, 768), (1, 128, 768)), ((8, 128, 768), (8, 128, 768)),
             ((4, 6, 40), (1, 1, 40)), ((4, 6, 40), (4, 1, 1)), ((4, 6, 40), (1, 6, 1)),
             ((5, 7), (5, 7)), ((5, 7), (1, 7)), ((2, 3, 4, 8), (2, 1, 4, 1)), ((1000,), (1000,)),
             ((3, 5, 17), (1, 1, 1))]
    for ashape, bshape in cases:
        a = (g.standard_normal(ashape) + 2.5).astype(dtype)
        b = (g.standard_normal(bshape) + 2.5).astype(dtype)
        if ashape == (3, 3, 3) and dtype == np.float32:
            a = np.array(literals["add_a_3x3x3"], np.float32).reshape(3, 3, 3)
            b = np.array(literals["add_b_3x1x3"], np.float32).reshape(3, 1, 3)
        ta, tb = dev(a), dev(b)
        for op in OPS:
            out = torch.empty_like(ta)
            M = rt.MemRef.from_tensor
            getattr(gpu, f"thrustElementwise{op}{sfx}")(*M(ta).args(), *M(tb).args(), *M(out).args())
            want = oracle.elementwise(op.lower(), a, b)
            got = host(out)
            if op == "Div" and dtype == np.float32:
                assert_close(got, want, rtol=2e-7, atol=0, what=f"div {ashape}")
            else:
                assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (op, ashape, bshape)


def test_gather_and_cu_seqlens_exact(gpu, rt, oracle, literals):
    g = np.random.default_rng(22)
    M = rt.MemRef.from_tensor
    for dtype, sfx, H in [(np.float16, "F16", 768), (np.float32, "F32", 20), (np.float16, "F16", 7)]:
        table = g.standard_normal((1, 500, H)).astype(dtype)
        idx = g.integers(0, 500, size=(8, 128)).astype(np.int64)
        tt, ti = dev(table), dev(idx)
        out = torch.empty((8, 128, H), dtype=tt.dtype, device="cuda")
        getattr(gpu, f"thrustGather{sfx}")(*M(ti).args(), *M(tt).args(), *M(out).args())
        assert np.array_equal(host(out), oracle.gather(idx, table[0]))
    bs, seq, lens = literals["cuseqlen_bs"], literals["cuseqlen_seq"], literals["cuseqlen_lengths"]
    mask = np.array([[1 if j < lens[i % 8] else 0 for j in range(seq)] for i in range(bs)], np.int64)
    for m, fn in [(mask, gpu.thrustCuSeqLenI64), (mask.astype(np.int32), gpu.thrustCuSeqLenI32)]:
        tm, out = dev(m), torch.full((bs + 1,), -7, dtype=torch.int32, device="cuda")
        fn(*M(tm).args(), *M(out).args())
        assert host(out).tolist() == [0, 64, 76, 107, 139, 172, 206, 241, 277, 341, 353, 384, 416,
                                      449, 483, 518, 554]
    for bs, seq in [(1, 1), (3, 200), (33, 128), (300, 17)]:
        m = (g.random((bs, seq)) < 0.6).astype(np.int64)
        m[0] = 0
        tm, out = dev(m), torch.empty((bs + 1,), dtype=torch.int32, device="cuda")
        gpu.thrustCuSeqLenI64(*M(tm).args(), *M(out).args())
        assert np.array_equal(host(out), oracle.cu_seqlens(m))


def test_gelu_kernel(gpu, rt, oracle):
    x = np.linspace(-9, 9, 4096).astype(np.float16)
    M = rt.MemRef.from_tensor
    for form, name in [(0, "erf"), (1, "tanh")]:
        t, out = dev(x), torch.empty(4096, dtype=torch.float16, device="cuda")
        gpu.homGeluF16(*M(t).args(), *M(out).args(), form)
        assert_close(host(out), oracle.gelu(x.astype(np.float64), name), rtol=1e-3, atol=1e-4)


# -------------------------------------------------------------------- GEMM --
def knum(rt, tile, epi="linear"):
    """1-based manifest number of the kernel whose name holds `_<tile>_` and ends in `_<epi>`."""
    for idx, name, _, _ in rt.manifest():
        if f"_{tile}_" in name and name.endswith("_" + epi):
            return idx + 1
    raise KeyError((tile, epi))


def run_gemm(gpu, rt, A, B, C, D_init, num, splitk, alpha=1.0, beta=0.0, act=0, in_place=False):
    M = rt.MemRef.from_tensor
    ta, tb = dev(A), dev(B)
    td = dev(D_init)
    tc = td if in_place else (dev(C) if C is not None else td)
    gpu.cutlassGemmF16(*M(ta).args(), False, *M(tb).args(), False, *M(tc).args(), *M(td).args(),
                       act, alpha, beta, num, splitk)
    return host(td)


def test_gemm_every_manifest_kernel(gpu, rt, oracle):
    """Every kernel x {tile-aligned, ragged} shapes x {1, 3} K slices."""
    g = np.random.default_rng(31)
    shapes8 = [(256, 256, 128), (200, 264, 136), (72, 40, 392)]
    shapes1 = [(67, 45, 77), (130, 129, 33)]
    for idx, name, act, align in rt.manifest():
        epi = "gelu_tanh" if "gelutanh" in name else ("gelu_erf" if act else "linear")
        for (M_, N_, K_) in (shapes8 if align == 8 else shapes8[:1] + shapes1):
            A = g.standard_normal((1, M_, K_)).astype(np.float16)
            B = (g.standard_normal((1, K_, N_)) * 0.1).astype(np.float16)
            want = oracle.gemm(A[0], B[0], act=epi)
            for sk in (1, 3):
                got = run_gemm(gpu, rt, A, B, None, np.zeros((1, M_, N_), np.float16), idx + 1, sk)
                assert_close(got[0], want, **GEMM_TOL, what=f"{name} {M_}x{N_}x{K_} splitK={sk}")


FINE_TILES = ("128x96_64x2r2_w4x2", "64x48_64x2r2_w4x1", "64x48_64x2r4_w4x1", "64x144_64x2r2_w4x1")


# the register-staged pipeline with slabs staged by buffer_load ... lds (ring of LDS buffers, fragment reads issued
# by hand when B is row-major)
DMA_STAGED_TILES = ("128x128_64q2_w2x4", "128x128_64q3_w2x4", "64x64_64q3_w2x2", "256x256_64q1_w2x4")


def _gemm_family_cases(gpu, rt, oracle, monkeypatch, tiles, seed):
    """Every epilogue source form (none, bias row, in-place residual, a [M', N] source shared by the batch entries
    = the general epilogue), GELU, split-K, ragged M / N / K (a partial last slab, K smaller than the pipeline is
    deep), more tiles than CUs, and the [N, K] layout of B through nvteGemmF16."""
    g = np.random.default_rng(seed)
    M = rt.MemRef.from_tensor
    for tile in tiles:
        for (M_, N_, K_) in [(256, 288, 128), (200, 264, 136), (72, 40, 392), (1100, 2000, 72)]:
            A = g.standard_normal((1, M_, K_)).astype(np.float16)
            B = (g.standard_normal((1, K_, N_)) * 0.1).astype(np.float16)
            bias = g.standard_normal((1, 1, N_)).astype(np.float16)
            R = g.standard_normal((1, M_, N_)).astype(np.float16)
            want_bias = oracle.gemm(A[0], B[0], bias[0], beta=1.0, act="gelu_erf")
            want_res = oracle.gemm(A[0], B[0], R[0], beta=0.5, alpha=2.0)
            for sk in (1, 2):
                got = run_gemm(gpu, rt, A, B, bias, np.zeros((1, M_, N_), np.float16), knum(rt, tile, "gelu"), sk,
                               beta=1.0)
                assert_close(got[0], want_bias, **GEMM_TOL, what=f"{tile} splitK={sk} {M_}x{N_}x{K_} bias+gelu")
                got = run_gemm(gpu, rt, A, B, None, R, knum(rt, tile), sk, alpha=2.0, beta=0.5, in_place=True)
                assert_close(got[0], want_res, **GEMM_TOL, what=f"{tile} splitK={sk} {M_}x{N_}x{K_} residual")
        # batch of 3 with one [M', N] source shared by the entries (the source-row period form)
        b, Mp, N_, K_ = 3, 40, 96, 64
        A = g.standard_normal((b, Mp, K_)).astype(np.float16)
        B = (g.standard_normal((1, K_, N_)) * 0.1).astype(np.float16)
        C = g.standard_normal((1, Mp, N_)).astype(np.float16)
        want = oracle.gemm(A.reshape(-1, K_), B[0], np.tile(C[0], (b, 1)), beta=1.0, act="gelu_tanh")
        got = run_gemm(gpu, rt, A, B, C, np.zeros((b, Mp, N_), np.float16), knum(rt, tile, "gelutanh"), 1, beta=1.0)
        assert_close(got.reshape(-1, N_), want, **GEMM_TOL, what=f"{tile} shared source")
        # B as [N, K]
        name = [n for _, n, _, _ in rt.manifest() if f"_{tile}_" in n and n.endswith("_linear")][0]
        for (b, Mp, K_, N_, beta, sk) in [(2, 100, 136, 264, 1.0, 1), (1, 256, 128, 288, 0.0, 2)]:
            monkeypatch.setenv("HOM_NVTE_GEMM_KERNEL", f"{name},{sk}")
            A = g.standard_normal((b, Mp, K_)).astype(np.float16)
            Bt = (g.standard_normal((1, N_, K_)) * 0.05).astype(np.float16)
            X = g.standard_normal((b, Mp, N_)).astype(np.float16)
            want = oracle.gemm(A.reshape(-1, K_), Bt[0], X.reshape(-1, N_), beta=beta, b_is_nk=True)
            ta, tb, td = dev(A), dev(Bt), dev(X)
            gpu.nvteGemmF16(*M(ta).args(), False, *M(tb).args(), True, *M(td).args(), *M(td).args(),
                            0, 1.0, beta, 0, 0)
            assert_close(host(td).reshape(-1, N_), want, **GEMM_TOL, what=f"{tile} [N,K] {Mp}x{N_}x{K_} splitK={sk}")
        monkeypatch.delenv("HOM_NVTE_GEMM_KERNEL")


def test_gemm_fine_family(gpu, rt, oracle, monkeypatch):
    """The 16x16x32-MFMA kernels (tile sides in steps of 16)."""
    _gemm_family_cases(gpu, rt, oracle, monkeypatch, FINE_TILES, 41)


def test_gemm_dma_staged_family(gpu, rt, oracle, monkeypatch):
    """The q<d> kernels: same cases; K = 72 and 128 are shorter than the ring is deep, 136 and 392 end in a partial
    slab, 1100 x 2000 has more tiles than the chip holds workgroups."""
    _gemm_family_cases(gpu, rt, oracle, monkeypatch, DMA_STAGED_TILES, 43)


def test_gemm_more_tiles_than_resident_workgroups(gpu, rt, oracle):
    """Ragged problem whose tile count exceeds what the chip holds at once, so the
    persistent kernels walk several tiles per workgroup (with and without split-K)."""
    g = np.random.default_rng(35)
    M_, N_, K_ = 4100, 4104, 136
    A = g.standard_normal((1, M_, K_)).astype(np.float16)
    B = (g.standard_normal((1, K_, N_)) * 0.1).astype(np.float16)
    bias = g.standard_normal((1, 1, N_)).astype(np.float16)
    want = oracle.gemm(A[0], B[0], bias[0], beta=1.0, act="gelu_erf")
    for tile in ("64x64_64x2r2_w2x2", "128x128_64x2r2_w2x4", "256x256_64x2r1_w2x4", "64x64_64q3_w2x2",
                 "256x256_64q1_w2x4"):
        for sk in (1, 2):
            got = run_gemm(gpu, rt, A, B, bias, np.zeros((1, M_, N_), np.float16), knum(rt, tile, "gelu"), sk,
                           beta=1.0)
            assert_close(got[0], want, **GEMM_TOL, what=f"{tile} splitK={sk}, {M_}x{N_}x{K_}")


def test_gemm_even_n_not_multiple_of_8(gpu, rt, oracle):
    """N % 8 != 0 with K % 8 == 0: rows of B, C, D start at 4-byte boundaries only.
    The register-staged kernels take these directly (the reference's alignment-2
    CUTLASS instances); covers the BERT vocabulary projection width 30522."""
    g = np.random.default_rng(36)
    for (M_, N_, K_) in [(200, 250, 136), (64, 30522, 64), (130, 6, 72), (96, 1026, 768)]:
        A = g.standard_normal((1, M_, K_)).astype(np.float16)
        B = (g.standard_normal((1, K_, N_)) * 0.1).astype(np.float16)
        bias = g.standard_normal((1, 1, N_)).astype(np.float16)
        R = g.standard_normal((1, M_, N_)).astype(np.float16)
        want_bias = oracle.gemm(A[0], B[0], bias[0], beta=1.0, act="gelu_erf")
        want_res = oracle.gemm(A[0], B[0], R[0], beta=1.0)
        for tile in ("64x64_64x2r2_w2x2", "128x128_64x2r2_w2x4", "256x256_64x2r1_w2x4"):
            for sk in (1, 2):
                got = run_gemm(gpu, rt, A, B, bias, np.zeros((1, M_, N_), np.float16), knum(rt, tile, "gelu"),
                               sk, beta=1.0)
                assert_close(got[0], want_bias, **GEMM_TOL, what=f"{tile} splitK={sk} {M_}x{N_}x{K_} bias+gelu")
                got = run_gemm(gpu, rt, A, B, None, R, knum(rt, tile), sk, beta=1.0, in_place=True)
                assert_close(got[0], want_res, **GEMM_TOL, what=f"{tile} splitK={sk} {M_}x{N_}x{K_} residual")
        # the library's own choice (gemmNum 0) must not fall back to the scalar kernel
        idx, sk = ctypes.c_int64(), ctypes.c_int32()
        gpu.homGemmSelect(M_, N_, K_, 0, ctypes.byref(idx), ctypes.byref(sk))
        name = rt.manifest()[idx.value][1]
        assert "align8" in name and "r" in name.split("_64x2")[1][:2], name
        got = run_gemm(gpu, rt, A, B, None, R, 0, 1, beta=1.0, in_place=True)
        assert_close(got[0], want_res, **GEMM_TOL, what=f"auto {M_}x{N_}x{K_}")
    # a kernel of the DMA family still refuses such a problem
    A = g.standard_normal((1, 64, 64)).astype(np.float16)
    B = g.standard_normal((1, 64, 250)).astype(np.float16)
    gpu.homSetErrorMode(1)
    try:
        run_gemm(gpu, rt, A, B, None, np.zeros((1, 64, 250), np.float16), knum(rt, "128x128_64x4"), 1)
        assert b"multiples of 8" in gpu.homGetLastError()
    finally:
        gpu.homSetErrorMode(0)


def test_gemm_config1_bias_gelu(gpu, rt, oracle, synth):
    c = synth.gemm_bias_gelu()
    for form, act in (("gelu_tanh", 2), ("gelu_erf", 1)):
        want = oracle.gemm(c["A"][0], c["B"][0], c["bias"][0], beta=1.0, act=form)
        idx, sk = ctypes.c_int64(), ctypes.c_int32()
        gpu.homGemmSelect(1024, 3072, 768, act, ctypes.byref(idx), ctypes.byref(sk))
        got = run_gemm(gpu, rt, c["A"], c["B"], c["bias"], np.zeros((1, 1024, 3072), np.float16),
                       idx.value + 1, sk.value, beta=1.0)
        assert_close(got[0], want, **GEMM_TOL, what=f"config 1 {form}")
        # gemmNum 0: the library picks by the activation argument
        got0 = run_gemm(gpu, rt, c["A"], c["B"], c["bias"], np.zeros((1, 1024, 3072), np.float16),
                        0, 1, beta=1.0, act=act)
        assert_close(got0[0], want, **GEMM_TOL)


def test_gemm_residual_in_place_and_batch_folding(gpu, rt, oracle):
    """out-proj / FFN2 form: beta = 1 with D aliasing C, batch folded into rows."""
    g = np.random.default_rng(32)
    b, Mp, K_, N_ = 8, 128, 768, 768
    A = g.standard_normal((b, Mp, K_)).astype(np.float16)
    B = (g.standard_normal((1, K_, N_)) * 0.02).astype(np.float16)
    X = g.standard_normal((b, Mp, N_)).astype(np.float16)
    want = oracle.gemm(A.reshape(-1, K_), B[0], X.reshape(-1, N_), beta=1.0)
    for num in (knum(rt, "128x128_64x4"), knum(rt, "64x64_64x4"), knum(rt, "128x64_64x4"),
                knum(rt, "128x128_32x2")):
        for sk in (1, 2, 6):
            got = run_gemm(gpu, rt, A, B, None, X, num, sk, beta=1.0, in_place=True)
            assert_close(got.reshape(-1, N_), want, **GEMM_TOL, what=f"in-place kernel {num} splitK {sk}")
    # [1, M', N] source shared by every batch, alpha/beta other than 1
    C1 = g.standard_normal((1, Mp, N_)).astype(np.float16)
    want = oracle.gemm(A.reshape(-1, K_), B[0], C1[0], alpha=0.5, beta=-2.0)
    got = run_gemm(gpu, rt, A, B, C1, np.zeros((b, Mp, N_), np.float16), knum(rt, "128x128_64x4"), 1,
                   alpha=0.5, beta=-2.0)
    assert_close(got.reshape(-1, N_), want, **GEMM_TOL)


def test_gemm_split_k_is_deterministic_and_invariant(gpu, rt, oracle, synth):
    c = synth.skinny_gemm()  # M=64, K=4096, N=1024
    want = oracle.gemm(c["A"][0], c["B"][0])
    outs = {}
    num = knum(rt, "64x64_64x4")
    for sk in (1, 2, 5, 8, 16):
        a = run_gemm(gpu, rt, c["A"], c["B"], None, np.zeros((1, 64, 1024), np.float16), num, sk)
        b = run_gemm(gpu, rt, c["A"], c["B"], None, np.zeros((1, 64, 1024), np.float16), num, sk)
        assert np.array_equal(a, b), f"split-K {sk} not reproducible"
        assert_close(a[0], want, **GEMM_TOL, what=f"skinny splitK={sk}")
        outs[sk] = a
    # slices only reassociate the fp32 sum: results agree to fp16 rounding
    assert np.abs(outs[16].astype(np.float32) - outs[1].astype(np.float32)).max() < 4e-3


def test_gemm_exact_cases(gpu, rt, literals):
    g = np.random.default_rng(33)
    A = g.standard_normal((1, 128, 128)).astype(np.float16)
    eye = np.eye(128, dtype=np.float16)[None]
    for num in (knum(rt, "128x128_64x4"), knum(rt, "64x64_64x8"), knum(rt, "64x64_64x2"),
                knum(rt, "64x64_32x2_w2x2_nn_align1")):
        assert np.array_equal(run_gemm(gpu, rt, A, eye, None, np.zeros_like(A), num, 1), A)
        assert np.array_equal(run_gemm(gpu, rt, eye, A, None, np.zeros_like(A), num, 1), A)
    c = literals["gemm_const"]  # reference driver b.cu: 0.1 x 0.2 over K = 768
    A = np.full((1, c["m"], c["k"]), c["a"], np.float16)
    B = np.full((1, c["k"], c["n"]), c["b"], np.float16)
    out = run_gemm(gpu, rt, A, B, None, np.zeros((1, c["m"], c["n"]), np.float16),
                   knum(rt, "128x128_64x4"), 1)
    assert np.abs(out.astype(np.float64) - c["expect"]).max() < c["tol"]


def test_profiler_layout_sweep_and_table_preference(gpu, rt):
    """homGemmProfileLayout returns a kernel with the matching epilogue for either layout of B, and
    homGemmPrefersNvte only says yes for shapes the shipped table holds a [N, K] kernel for."""
    names = {i: n for i, n, _, _ in rt.manifest()}
    for nk in (0, 1):
        idx, sk, ms = ctypes.c_int64(), ctypes.c_int32(), ctypes.c_float()
        gpu.homGemmProfileLayout(256, 768, 768, 0, 1.0, 0.0, nk, ctypes.byref(idx), ctypes.byref(sk),
                                 ctypes.byref(ms))
        assert idx.value >= 0 and names[idx.value].endswith("_linear") and sk.value >= 1 and ms.value > 0
    assert gpu.homGemmPrefersNvte(7, 24, 40, 0) == 0   # not in the table
    assert gpu.homGemmPrefersNvte(1024, 768, 768, 0) in (0, 1)


def test_nvte_gemm_path(gpu, rt, oracle):
    g = np.random.default_rng(34)
    M = rt.MemRef.from_tensor
    for (b, Mp, K_, N_, act, beta) in [(8, 128, 768, 2304, 0, 0.0), (8, 128, 768, 3072, 1, 0.0),
                                       (8, 128, 3072, 768, 0, 1.0), (1, 50, 72, 24, 1, 1.0),
                                       (2, 9, 37, 21, 0, 0.0)]:
        A = g.standard_normal((b, Mp, K_)).astype(np.float16)
        Bt = (g.standard_normal((1, N_, K_)) * 0.05).astype(np.float16)
        X = g.standard_normal((b, Mp, N_)).astype(np.float16)
        want = oracle.gemm(A.reshape(-1, K_), Bt[0], X.reshape(-1, N_), beta=beta,
                           act="gelu_tanh" if act else "linear", b_is_nk=True)
        ta, tb, td = dev(A), dev(Bt), dev(X)
        gpu.nvteGemmF16(*M(ta).args(), False, *M(tb).args(), True, *M(td).args(), *M(td).args(),
                        act, 1.0, beta, 0, 0)
        assert_close(host(td).reshape(-1, N_), want, **GEMM_TOL, what=f"nvte {Mp}x{N_}x{K_}")


def test_ln_gemm_pair(gpu, rt, oracle, literals):
    """verify.py case: ab = a@b with row stats, then LN(ab) @ c."""
    a = np.array(literals["verify_a"], np.float16)[None]
    b = np.array(literals["verify_b"], np.float16)[None]
    c = np.array(literals["verify_c"], np.float16)[None]
    M = rt.MemRef.from_tensor
    ta, tb, tc = dev(a), dev(b), dev(c)
    ab = torch.zeros((1, 4, 8), dtype=torch.float16, device="cuda")
    var = torch.zeros((1, 4, 1), dtype=torch.float16, device="cuda")
    mean = torch.zeros((1, 4, 1), dtype=torch.float16, device="cuda")
    eps = literals["verify_eps_stats"]
    gpu.cutlassGemmWithVarMeanF16(*M(ta).args(), *M(tb).args(), *M(ab).args(), *M(ab).args(),
                                  *M(var).args(), *M(mean).args(), 1.0, 0.0, 0, eps)
    want_ab = oracle.gemm(a[0], b[0])
    assert_close(host(ab)[0], want_ab, **GEMM_TOL)
    v, m = oracle.row_stats(host(ab)[0].astype(np.float32), eps)
    assert_close(host(var).ravel(), v, rtol=2e-3, atol=1e-3)
    assert_close(host(mean).ravel(), m, rtol=2e-3, atol=2e-3)
    out = torch.zeros((1, 4, 16), dtype=torch.float16, device="cuda")
    gpu.cutlassLayernormGemmF16(*M(ab).args(), *M(tc).args(), *M(out).args(), *M(out).args(),
                                *M(var).args(), *M(mean).args(), 1.0, 0.0, 0)
    x = host(ab)[0].astype(np.float64)
    ln = x * host(var).reshape(4, 1).astype(np.float64) + host(mean).reshape(4, 1).astype(np.float64)
    assert_close(host(out)[0], ln @ c[0].astype(np.float64), rtol=1e-2, atol=2e-2)


@pytest.mark.parametrize("Mp,N1,K1,N2,beta", [
    (1024, 768, 768, 768, 0.0),      # 64x64 tiles for both halves
    (1024, 768, 768, 2304, 1.0),     # second half on 128x128 tiles, residual source
    (4096, 1024, 256, 2304, 0.0),    # second half on 256x256 tiles
    (1000, 776, 264, 520, 1.0),      # ragged rows and columns (still multiples of 8)
    (100, 250, 72, 30, 0.0),         # N not a multiple of 8: the unfused kernels
])
def test_ln_gemm_pair_shapes(gpu, rt, oracle, Mp, N1, K1, N2, beta):
    """GEMM + row statistics, then GEMM of the row-normalised result, at sizes that reach every fused tile
    (LayernormGemmRunner.h:17-361).  The second product is checked against the affine row transform applied in
    fp64 with the var/mean values the first call stored."""
    M = rt.MemRef.from_tensor
    g = np.random.default_rng(Mp + N1 + N2)
    a = g.standard_normal((1, Mp, K1)).astype(np.float16)
    b = (g.standard_normal((1, K1, N1)) * 0.05).astype(np.float16)
    c = (g.standard_normal((1, N1, N2)) * 0.05).astype(np.float16)
    # rows with a mean well away from zero make the colsum term matter
    src = (g.standard_normal((1, Mp, N1)) + 1.5).astype(np.float16)
    eps = 1e-5
    ta, tb, tc = dev(a), dev(b), dev(c)
    d1 = dev(src) if beta else torch.zeros((1, Mp, N1), dtype=torch.float16, device="cuda")
    var = torch.zeros((1, Mp, 1), dtype=torch.float16, device="cuda")
    mean = torch.zeros((1, Mp, 1), dtype=torch.float16, device="cuda")
    gpu.cutlassGemmWithVarMeanF16(*M(ta).args(), *M(tb).args(), *M(d1).args(), *M(d1).args(),
                                  *M(var).args(), *M(mean).args(), 1.0, beta, 0, eps)
    want_d1 = oracle.gemm(a[0], b[0], src[0] if beta else None, beta=beta)
    got_d1 = host(d1)[0]
    assert_close(got_d1, want_d1, **GEMM_TOL, what="first product")
    v, m = oracle.row_stats(got_d1.astype(np.float32), eps)
    assert_close(host(var).ravel(), v, rtol=2e-3, atol=1e-3, what="var")
    assert_close(host(mean).ravel(), m, rtol=2e-3, atol=2e-3, what="mean")

    res = (g.standard_normal((1, Mp, N2))).astype(np.float16)
    out = dev(res) if beta else torch.zeros((1, Mp, N2), dtype=torch.float16, device="cuda")
    gpu.cutlassLayernormGemmF16(*M(d1).args(), *M(tc).args(), *M(out).args(), *M(out).args(),
                                *M(var).args(), *M(mean).args(), 1.0, beta, 0)
    ln = got_d1.astype(np.float64) * host(var).reshape(Mp, 1).astype(np.float64) \
        + host(mean).reshape(Mp, 1).astype(np.float64)
    want = ln @ c[0].astype(np.float64) + (beta * res[0].astype(np.float64) if beta else 0.0)
    assert_close(host(out)[0], want, **GEMM_TOL, what="second product")


def test_ln_gemm_pair_constant_rows_stay_finite(gpu, rt):
    """Rows of D that are constant make E[x^2] - E[x]^2 cancel to zero or just below; with BERT's eps of
    1e-12 an unclamped difference gives NaN statistics that poison the second product."""
    M = rt.MemRef.from_tensor
    for (Mp, N1, K1) in [(128, 768, 64), (100, 250, 72)]:   # fused epilogue, separate statistics kernel
        a = np.full((1, Mp, K1), 0.25, np.float16)
        b = np.full((1, K1, N1), 0.125, np.float16)
        a[0, 1::2] = -0.5
        ta, tb = dev(a), dev(b)
        d1 = torch.zeros((1, Mp, N1), dtype=torch.float16, device="cuda")
        var = torch.zeros((1, Mp, 1), dtype=torch.float16, device="cuda")
        mean = torch.zeros((1, Mp, 1), dtype=torch.float16, device="cuda")
        gpu.cutlassGemmWithVarMeanF16(*M(ta).args(), *M(tb).args(), *M(d1).args(), *M(d1).args(),
                                      *M(var).args(), *M(mean).args(), 1.0, 0.0, 0, 1e-12)
        v, m = host(var).astype(np.float32), host(mean).astype(np.float32)
        assert not np.isnan(v).any() and not np.isnan(m).any(), (Mp, N1, K1)
        assert (v > 0).all()


@pytest.mark.parametrize("Mp,H,F,tile", [
    (1024, 768, 3072, None),                  # BERT-base sizes, library-chosen tiles
    (200, 264, 520, "64x64_64x2r2_w2x2"),     # ragged rows and columns (multiples of 8)
    (300, 264, 520, "128x128_64x2r2_w2x4"),
    (520, 520, 264, "256x256_64x2r1_w2x4"),
])
def test_folded_layernorm_gemm_chain(gpu, rt, oracle, Mp, H, F, tile):
    """x1 = a . Wo + r (+ partial row sums); f = GELU(LN(x1) . W1); x2 = f . W2 + LN(x1) (+ partial row sums);
    q = LN(x2) . Wq: the post-LN transformer block with both layer norms folded into the GEMMs around them
    (homGemmFoldedLayernormF16).  Every product is checked against fp64 arithmetic on the fp16 tensors the GPU
    stored, with the layer norm in its closed form (pinned for the oracle by test_oracle.py)."""
    M = rt.MemRef.from_tensor
    g = np.random.default_rng(Mp + H + F)
    eps = 1e-12
    num = knum(rt, tile) if tile else 0
    a = g.standard_normal((1, Mp, H)).astype(np.float16)
    wo = (g.standard_normal((1, H, H)) * 0.05).astype(np.float16)
    w1 = (g.standard_normal((1, H, F)) * 0.05).astype(np.float16)
    w2 = (g.standard_normal((1, F, H)) * 0.05).astype(np.float16)
    wq = (g.standard_normal((1, H, 3 * H)) * 0.05).astype(np.float16)
    r = (g.standard_normal((1, Mp, H)) + 0.75).astype(np.float16)   # rows with a mean away from zero
    ta, two, tw1, tw2, twq = dev(a), dev(wo), dev(w1), dev(w2), dev(wq)
    x = dev(r)                                                      # residual stream, updated in place
    f = torch.zeros((1, Mp, F), dtype=torch.float16, device="cuda")
    q = torch.zeros((1, Mp, 3 * H), dtype=torch.float16, device="cuda")
    cs1 = torch.zeros(F, dtype=torch.float32, device="cuda")
    csq = torch.zeros(3 * H, dtype=torch.float32, device="cuda")
    gpu.homColumnSumsF16(*M(tw1).args(), cs1.data_ptr())
    gpu.homColumnSumsF16(*M(twq).args(), csq.data_ptr())
    assert_close(cs1.cpu().numpy(), w1[0].astype(np.float64).sum(0), rtol=1e-5, atol=1e-4, what="column sums")
    pieces = gpu.homFoldedLayernormPieces(Mp, H, H, 0, num)
    assert pieces == gpu.homFoldedLayernormPieces(Mp, H, F, 0, num) or tile is None
    st1 = torch.full((pieces * Mp * 2,), float("nan"), dtype=torch.float32, device="cuda")

    def ln(v16):
        v = v16.astype(np.float64)
        mu = v.mean(-1, keepdims=True)
        return (v - mu) / np.sqrt(((v - mu) ** 2).mean(-1, keepdims=True) + eps)

    # x1 = a . Wo + r, in place over r, with the partial sums of x1
    gpu.homGemmFoldedLayernormF16(*M(ta).args(), *M(two).args(), *M(x).args(), *M(x).args(), 2, 0, 1.0, 1.0,
                                  None, 0, eps, None, st1.data_ptr(), num)
    x1 = host(x)[0]
    assert_close(x1, oracle.gemm(a[0], wo[0], r[0], beta=1.0), **GEMM_TOL, what="x1")
    part = st1.cpu().numpy().reshape(pieces, Mp, 2).astype(np.float64).sum(0)
    assert_close(part[:, 0], x1.astype(np.float64).sum(-1), rtol=1e-4, atol=1e-2, what="row sums")
    assert_close(part[:, 1], (x1.astype(np.float64) ** 2).sum(-1), rtol=1e-4, atol=1e-2, what="row sums of squares")
    # f = GELU(LN(x1) . W1)
    gpu.homGemmFoldedLayernormF16(*M(x).args(), *M(tw1).args(), *M(f).args(), *M(f).args(), 1, 1, 1.0, 0.0,
                                  st1.data_ptr(), pieces, eps, cs1.data_ptr(), None, num)
    f16 = host(f)[0]
    assert_close(f16, oracle.gelu(ln(x1) @ w1[0].astype(np.float64), "erf"), **GEMM_TOL, what="f")
    # x2 = f . W2 + LN(x1), in place over x1, with the partial sums of x2
    pieces2 = gpu.homFoldedLayernormPieces(Mp, H, F, 0, num)
    st2 = torch.full((pieces2 * Mp * 2,), float("nan"), dtype=torch.float32, device="cuda")
    gpu.homGemmFoldedLayernormF16(*M(f).args(), *M(tw2).args(), *M(x).args(), *M(x).args(), 2, 0, 1.0, 1.0,
                                  st1.data_ptr(), pieces, eps, None, st2.data_ptr(), num)
    x2 = host(x)[0]
    assert_close(x2, f16.astype(np.float64) @ w2[0].astype(np.float64) + ln(x1), **GEMM_TOL, what="x2")
    # q = LN(x2) . Wq
    gpu.homGemmFoldedLayernormF16(*M(x).args(), *M(twq).args(), *M(q).args(), *M(q).args(), 1, 0, 1.0, 0.0,
                                  st2.data_ptr(), pieces2, eps, csq.data_ptr(), None, num)
    assert_close(host(q)[0], ln(x2) @ wq[0].astype(np.float64), **GEMM_TOL, what="q")
    # without statistics the same entry point is the plain product
    gpu.homGemmFoldedLayernormF16(*M(x).args(), *M(twq).args(), *M(q).args(), *M(q).args(), 1, 0, 1.0, 0.0,
                                  None, 0, eps, None, None, num)
    assert_close(host(q)[0], oracle.gemm(x2, wq[0]), **GEMM_TOL, what="plain product")


# --------------------------------------------------------------- attention --
def run_attention(gpu, rt, qkv, lens, heads, scale):
    M = rt.MemRef.from_tensor
    bs, seq, w = qkv.shape
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    tq, tc = dev(qkv), dev(cu)
    out = torch.full((bs, seq, w // 3), 7.0, dtype=torch.float16, device="cuda")
    gpu.nvteBertAttentionF16(*M(tq).args(), *M(tc).args(), *M(out).args(), scale, heads)
    return host(out), cu


def test_attention_config3(gpu, rt, oracle, synth):
    c = synth.attention()
    got, cu = run_attention(gpu, rt, c["qkv"], c["lens"], 12, 0.125)
    want = oracle.attention(c["qkv"], cu, 12, 0.125)
    assert_close(got, want, **GEMM_TOL, what="attention config 3")
    for b, n in enumerate(c["lens"]):
        assert not got[b, n:].any(), "padded query rows must be zeros"


@pytest.mark.parametrize("bs,seq,heads,lens", [
    (2, 64, 2, [64, 1]), (3, 100, 1, [100, 37, 64]), (2, 512, 16, [512, 300]),
    (4, 128, 12, [0, 128, 65, 33]), (1, 40, 3, [17]), (32, 512, 2, None)])
def test_attention_shapes_and_edges(gpu, rt, oracle, bs, seq, heads, lens):
    g = np.random.default_rng(bs * 1000 + seq)
    qkv = g.standard_normal((bs, seq, 3 * heads * 64)).astype(np.float16)
    lens = np.array(lens if lens is not None else g.integers(1, seq + 1, size=bs), np.int32)
    got, cu = run_attention(gpu, rt, qkv, lens, heads, 0.125)
    assert_close(got, oracle.attention(qkv, cu, heads, 0.125), **GEMM_TOL, what=f"attention {bs}x{seq}x{heads}")


@pytest.mark.parametrize("d", [128, 192, 256])
@pytest.mark.parametrize("bs,seq,heads,lens", [
    (2, 64, 2, [64, 1]), (3, 100, 1, [100, 37, 64]), (2, 512, 8, [512, 300]),
    (4, 128, 6, [0, 128, 65, 33]), (1, 40, 3, [17]), (16, 512, 4, None)])
def test_attention_larger_head_sizes(gpu, rt, oracle, d, bs, seq, heads, lens):
    """Head sizes 128, 192 and 256 (the reference's contract is head size % 64 == 0): both kernel variants
    where they exist (d = 128: the larger shapes take 128 query rows per workgroup, the smaller ones the
    key-split form), padding, an empty sequence, ragged lengths; padded query rows are zeros."""
    g = np.random.default_rng(bs * 1000 + seq + 7 + d)
    qkv = g.standard_normal((bs, seq, 3 * heads * d)).astype(np.float16)
    lens = np.array(lens if lens is not None else g.integers(1, seq + 1, size=bs), np.int32)
    scale = 1.0 / np.sqrt(float(d))
    got, cu = run_attention(gpu, rt, qkv, lens, heads, scale)
    assert_close(got, oracle.attention(qkv, cu, heads, scale), **GEMM_TOL, what=f"attention d{d} {bs}x{seq}x{heads}")
    for b, n in enumerate(lens):
        assert not got[b, n:].any(), "padded query rows must be zeros"
    # layout: V one-hot in (head h, column d - 51) comes out in that column of every valid row
    col = d - 51
    z = np.zeros((1, 64, 3, heads, d), np.float16)
    z[:, :, 2, heads - 1, col] = 1.0
    one, _ = run_attention(gpu, rt, z.reshape(1, 64, -1), [64], heads, scale)
    want = np.zeros((1, 64, heads, d), np.float16)
    want[:, :, heads - 1, col] = 1.0
    assert np.array_equal(one.reshape(1, 64, heads, d), want)


def test_attention_rejects_other_head_sizes(gpu, rt):
    M = rt.MemRef.from_tensor
    qkv = torch.zeros((1, 64, 3 * 2 * 96), dtype=torch.float16, device="cuda")
    cu = torch.tensor([0, 64], dtype=torch.int32, device="cuda")
    out = torch.zeros((1, 64, 2 * 96), dtype=torch.float16, device="cuda")
    gpu.homSetErrorMode(1)
    try:
        gpu.homGetLastError()
        gpu.nvteBertAttentionF16(*M(qkv).args(), *M(cu).args(), *M(out).args(), 0.1, 2)
        msg = gpu.homGetLastError().decode()
    finally:
        gpu.homSetErrorMode(0)
    assert "head size" in msg, msg


@pytest.mark.parametrize("d,heads", [(64, 4), (128, 2), (256, 1)])
def test_attention_growing_scores(gpu, rt, oracle, d, heads):
    """Scores that keep growing along the keys: the softmax reference a wavefront fixed on its first key block
    has to move again and again (the probabilities of a later block would leave fp16's range against the old
    reference), in blocks of any position, with full and ragged lengths, in both kernel variants."""
    g = np.random.default_rng(d + heads)
    for bs, seq, lens in ((2, 512, [512, 301]), (32, 512, None), (3, 128, [128, 70, 9])):
        qkv = g.standard_normal((bs, seq, 3, heads, d)).astype(np.float32)
        ramp = 1.0 + 5.0 * np.arange(seq, dtype=np.float32) / seq        # keys 6 times larger at the end
        qkv[:, :, 1] *= ramp[None, :, None, None]
        qkv[:, seq // 2, 1] *= 2.0                                         # and a spike in the middle
        qkv = qkv.reshape(bs, seq, -1).astype(np.float16)
        lens_ = np.array(lens if lens is not None else g.integers(1, seq + 1, size=bs), np.int32)
        scale = 1.0 / np.sqrt(float(d))
        got, cu = run_attention(gpu, rt, qkv, lens_, heads, scale)
        assert np.isfinite(got.astype(np.float32)).all()
        assert_close(got, oracle.attention(qkv, cu, heads, scale), **GEMM_TOL,
                     what=f"attention d{d} {bs}x{seq}, growing scores")


def test_attention_layout_onehot(gpu, rt):
    """Pins the [3][heads][64] interleave: V one-hot in (head 5, d 9)."""
    heads, seq = 12, 64
    z = np.zeros((1, seq, 3, heads, 64), np.float16)
    z[:, :, 2, 5, 9] = 1.0
    got, _ = run_attention(gpu, rt, z.reshape(1, seq, -1), [seq], heads, 0.125)
    want = np.zeros((1, seq, heads, 64), np.float16)
    want[:, :, 5, 9] = 1.0
    assert np.array_equal(got.reshape(1, seq, heads, 64), want)


# ------------------------------------------------------------------ memory --
def test_alloc_family_and_constant_loader(gpu, rt, tmp_path, monkeypatch):
    m = gpu.alloc3DMemRefNVGPUF16(2, 3, 4)
    ptr, sizes, strides = rt.read_descriptor(m)
    assert m.rank == 3 and sizes == [2, 3, 4] and strides == [12, 4, 1] and ptr != 0
    gpu.deallocNVGPUF16(m.rank, m.descriptor)
    m = gpu.alloc1DMemRefNVGPUI32(9)
    assert rt.read_descriptor(m)[1:] == ([9], [1])
    gpu.deallocNVGPUI32(m.rank, m.descriptor)
    vals = np.arange(24, dtype=np.float32) * 0.37 - 3
    (tmp_path / "5.txt").write_text("2 3 4\n" + " ".join(repr(float(v)) for v in vals) + "\n")
    monkeypatch.setenv("HOM_CONSTANT_DIR", str(tmp_path))
    for fn, dt in [(gpu.allocConstantNVGPUF16, torch.float16), (gpu.allocConstantNVGPUF32, torch.float32)]:
        m = fn(5)
        ptr, sizes, _ = rt.read_descriptor(m)
        assert sizes == [2, 3, 4]
        out = torch.empty(24, dtype=dt, device="cuda")
        hip = ctypes.CDLL("libamdhip64.so")
        hip.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
        assert hip.hipMemcpy(out.data_ptr(), ptr, 24 * out.element_size(), 3) == 0
        want = vals.astype(np.float16 if dt == torch.float16 else np.float32)
        assert np.array_equal(host(out), want)
        gpu.deallocNVGPUF16(m.rank, m.descriptor)
    # binary files win over text ones; either element size feeds either entry point
    weights = importlib.import_module("hands-on-mlir_amd.weights")
    weights.write_binary(str(tmp_path), 5, (vals * 2).reshape(2, 3, 4).astype(np.float16))
    weights.write_binary(str(tmp_path), 6, (vals * 3).reshape(2, 3, 4).astype(np.float32))
    for idx, scale in ((5, 2), (6, 3)):
        for fn, dt in [(gpu.allocConstantNVGPUF16, torch.float16), (gpu.allocConstantNVGPUF32, torch.float32)]:
            m = fn(idx)
            ptr, sizes, _ = rt.read_descriptor(m)
            assert sizes == [2, 3, 4]
            out = torch.empty(24, dtype=dt, device="cuda")
            assert hip.hipMemcpy(out.data_ptr(), ptr, 24 * out.element_size(), 3) == 0
            src = (vals * scale).astype(np.float16 if idx == 5 else np.float32)
            assert np.array_equal(host(out), src.astype(np.float16 if dt == torch.float16 else np.float32))
            gpu.deallocNVGPUF16(m.rank, m.descriptor)


# ------------------------------------------------------ randomised sweeps --
def test_gemm_randomised_sweep(gpu, rt, oracle):
    """Seeded random problems over every manifest kernel: ragged M / N / K, whole numbers of slabs, split-K, and the
    four source forms (none, bias row, residual in place, separate full matrix) with alpha / beta other than 1.
    Problems an aligned kernel cannot take are refused by the library's argument check (the reference's
    can_implement) and skipped."""
    g = np.random.default_rng(2024)
    man = rt.manifest()
    M_ = rt.MemRef.from_tensor
    compared = 0
    gpu.homSetErrorMode(1)
    try:
        for _ in range(500):
            idx, name, act, align = man[g.integers(len(man))]
            epi = "gelu_tanh" if "gelutanh" in name else ("gelu_erf" if act else "linear")
            M, N, K = (int(g.integers(1, 520)) for _ in range(3))
            if align == 8 and g.random() < 0.8:
                N, K = max(8, N // 8 * 8), max(8, K // 8 * 8)
            if g.random() < 0.15:
                K = int(g.integers(1, 24)) * 64
            sk = int(g.choice([1, 1, 2, 3, 5]))
            mode = int(g.integers(4))
            alpha = float(g.choice([1.0, 1.0, 0.5, 2.0]))
            beta = 0.0 if mode == 0 else float(g.choice([1.0, 1.0, 0.5]))
            A = g.standard_normal((1, M, K)).astype(np.float16)
            B = (g.standard_normal((1, K, N)) * 0.1).astype(np.float16)
            C = None if mode == 0 else g.standard_normal((1, 1 if mode == 1 else M, N)).astype(np.float16)
            ta, tb = dev(A), dev(B)
            td = dev(C) if mode == 2 else torch.zeros((1, M, N), dtype=torch.float16, device="cuda")
            tc = td if mode in (0, 2) else dev(C)
            gpu.homGetLastError()
            gpu.cutlassGemmF16(*M_(ta).args(), False, *M_(tb).args(), False, *M_(tc).args(), *M_(td).args(),
                               act, alpha, beta, idx + 1, sk)
            err = gpu.homGetLastError().decode()
            if err:
                assert "multiples of" in err, err
                continue
            want = oracle.gemm(A[0], B[0], None if C is None else np.broadcast_to(C[0], (M, N)).astype(np.float16),
                               alpha=alpha, beta=beta, act=epi)
            assert_close(host(td)[0], want, **GEMM_TOL,
                         what=f"{name} {M}x{N}x{K} splitK={sk} source form {mode} alpha={alpha} beta={beta}")
            compared += 1
    finally:
        gpu.homSetErrorMode(0)
    assert compared >= 300


def test_attention_and_layernorm_randomised_sweep(gpu, rt, oracle):
    """Seeded random attention problems (every head size, ragged and empty sequences, larger score amplitudes) and
    layer norms (in place, and with residual and affine parameters; row lengths off the vector width)."""
    g = np.random.default_rng(2025)
    M_ = rt.MemRef.from_tensor
    for _ in range(150):
        d = int(g.choice([64, 64, 64, 128, 192, 256]))
        heads, bs, seq = int(g.integers(1, 5)), int(g.integers(1, 6)), int(g.integers(1, 300))
        amp = float(g.choice([1.0, 1.0, 3.0]))
        qkv = (g.standard_normal((bs, seq, 3 * heads * d)) * amp).astype(np.float16)
        lens = g.integers(0, seq + 1, size=bs).astype(np.int32)
        got, cu = run_attention(gpu, rt, qkv, lens, heads, float(1.0 / np.sqrt(d)))
        want = oracle.attention(qkv, cu, heads, float(1.0 / np.sqrt(d)))
        for b in range(bs):
            assert_close(got[b, :lens[b]], want[b, :lens[b]], **GEMM_TOL,
                         what=f"attention d={d} heads={heads} bs={bs} seq={seq} lens={lens.tolist()} amplitude {amp}")
            assert not got[b, lens[b]:].any()
    for _ in range(150):
        rows = int(g.integers(1, 300))
        hidden = int(g.choice([8, 64, 96, 128, 760, 768, 1000, 1024, 2048, 3000, 4096, 5000]))
        x = (g.standard_normal((rows, hidden)) * float(g.choice([1.0, 10.0])) + float(g.choice([0.0, 3.0])))
        x = x.astype(np.float16)
        eps = float(g.choice([1e-12, 1e-5]))
        if g.integers(2):
            res = g.standard_normal((rows, hidden)).astype(np.float16)
            gamma = (1 + 0.02 * g.standard_normal(hidden)).astype(np.float16)
            beta = (0.02 * g.standard_normal(hidden)).astype(np.float16)
            tx, tr, tg, tb = dev(x), dev(res), dev(gamma), dev(beta)
            to = torch.zeros_like(tx)
            gpu.homAddLayernormF16(*M_(tx).args(), *M_(tr).args(), *M_(tg).args(), *M_(tb).args(), *M_(to).args(), eps)
            got, want = host(to), oracle.layernorm_f16(x, eps, res, gamma, beta)
        else:
            tx = dev(x)
            gpu.nvteLayernormF16(*M_(tx).args(), eps)
            got, want = host(tx), oracle.layernorm_f16(x, eps)
        assert_close(got, want, **LN_TOL, what=f"layer norm rows={rows} hidden={hidden} eps={eps}")


def test_library_selected_gemm_randomised_sweep(gpu, rt, oracle):
    """Seeded random problems through the two entry points that let the library pick the kernel: cutlassGemmF16
    with gemmNum == 0 (activation 0 / 1 / 2) and nvteGemmF16 (B as [N, K]; beta 0 or 1 in place; activation 1 is
    the tanh form there).  Any M, N, K: the selection has to fall back to kernels that fit the alignment."""
    g = np.random.default_rng(2026)
    M_ = rt.MemRef.from_tensor
    for it in range(300):
        M, N, K = (int(g.integers(1, 600)) for _ in range(3))
        if g.random() < 0.6:
            N, K = max(8, N // 8 * 8), max(8, K // 8 * 8)
        A = g.standard_normal((1, M, K)).astype(np.float16)
        X = g.standard_normal((1, M, N)).astype(np.float16)
        ta, td = dev(A), dev(X)
        if it % 2 == 0:
            act = int(g.integers(3))
            B = (g.standard_normal((1, K, N)) * 0.1).astype(np.float16)
            bias = g.standard_normal((1, 1, N)).astype(np.float16)
            tb, tc = dev(B), dev(bias)
            gpu.cutlassGemmF16(*M_(ta).args(), False, *M_(tb).args(), False, *M_(tc).args(), *M_(td).args(),
                               act, 1.0, 1.0, 0, 1)
            want = oracle.gemm(A[0], B[0], np.broadcast_to(bias[0], (M, N)).astype(np.float16), beta=1.0,
                               act=("linear", "gelu_erf", "gelu_tanh")[act])
            what = f"cutlassGemmF16 gemmNum=0 act={act} {M}x{N}x{K}"
        else:
            act, beta = int(g.integers(2)), float(g.integers(2))
            Bt = (g.standard_normal((1, N, K)) * 0.1).astype(np.float16)
            tb = dev(Bt)
            gpu.nvteGemmF16(*M_(ta).args(), False, *M_(tb).args(), True, *M_(td).args(), *M_(td).args(),
                            act, 1.0, beta, 0, 0)
            want = oracle.gemm(A[0], Bt[0], X[0], beta=beta, act=("linear", "gelu_tanh")[act], b_is_nk=True)
            what = f"nvteGemmF16 act={act} beta={beta} {M}x{N}x{K}"
        assert_close(host(td)[0], want, **GEMM_TOL, what=what)


def test_gemm_split_k_summed_in_kernel_matches_second_kernel(gpu, rt, oracle):
    """The optional in-kernel split-K reduction (the last slice of a tile to finish adds the partial
    tiles) against the default second kernel: same sums in the same order, so outputs agree to the last
    bit of fp16 (the epilogue's rounding may differ), run to run identical, and within the GEMM
    tolerance of the oracle.  Launches whose grid does not keep a tile's slices on one XCD must stay on
    the second kernel."""
    g = np.random.default_rng(36)
    used0 = gpu.homSplitKInKernelLaunches()
    try:
        for (M, N, K) in ((64, 1024, 4096), (512, 512, 1024), (200, 328, 1000), (1024, 768, 768)):
            A = g.standard_normal((1, M, K)).astype(np.float16)
            B = (g.standard_normal((1, K, N)) * 0.1).astype(np.float16)
            C = g.standard_normal((1, M, N)).astype(np.float16)
            want = oracle.gemm(A[0], B[0])
            for tile in ("64x64_64q3_w2x2", "64x64_64x2r2_w2x2", "128x128_64x2r2_w2x4"):
                for epi, act, beta in (("linear", 0, 0.0), ("linear", 0, 1.0), ("gelu", 1, 1.0)):
                    num = knum(rt, tile, epi)
                    for sk in (2, 3, 8):
                        zero = np.zeros((1, M, N), np.float16)
                        gpu.homSetSplitKInKernel(0)
                        two = run_gemm(gpu, rt, A, B, C, zero, num, sk, beta=beta, act=act)
                        gpu.homSetSplitKInKernel(1)
                        before = gpu.homSplitKInKernelLaunches()
                        one = run_gemm(gpu, rt, A, B, C, zero, num, sk, beta=beta, act=act)
                        again = run_gemm(gpu, rt, A, B, C, zero, num, sk, beta=beta, act=act)
                        what = f"{M}x{N}x{K} {tile} {epi} beta={beta} splitK={sk}"
                        bm, bn = (int(v) for v in tile.split("_")[0].split("x"))
                        tiles_n = -(-N // bn) * -(-M // bm)
                        took = gpu.homSplitKInKernelLaunches() - before
                        assert took == (2 if tiles_n % 8 == 0 else 0), what
                        assert np.array_equal(one, again), what
                        a, b = one.astype(np.float32), two.astype(np.float32)
                        ulp = np.maximum(np.abs(b), 2.0 ** -14) * 2.0 ** -10
                        assert (np.abs(a - b) <= ulp).all(), what
                        if not beta and not act:
                            assert_close(one[0], want, **GEMM_TOL, what=what)
        # the default mode takes the in-kernel form only where it measured faster: small tiles,
        # at most 6 slices, at most 512 workgroups
        gpu.homSetSplitKInKernel(3)
        A = g.standard_normal((1, 64, 4096)).astype(np.float16)
        B = (g.standard_normal((1, 4096, 1024)) * 0.1).astype(np.float16)
        want = oracle.gemm(A[0], B[0])
        zero = np.zeros((1, 64, 1024), np.float16)
        for tile, sk, expect in (("64x64_64x2r2_w2x2", 4, 1), ("64x64_64x2r2_w2x2", 8, 0),
                                 ("128x128_64x2r2_w2x4", 2, 0), ("64x64_64q3_w2x2", 6, 1)):
            before = gpu.homSplitKInKernelLaunches()
            out = run_gemm(gpu, rt, A, B, None, zero, knum(rt, tile), sk)
            assert gpu.homSplitKInKernelLaunches() - before == expect, (tile, sk)
            assert_close(out[0], want, **GEMM_TOL, what=f"default mode {tile} splitK={sk}")
    finally:
        gpu.homSetSplitKInKernel(3)   # the default
    assert gpu.homSplitKInKernelLaunches() > used0


def test_gemm_split_k_in_kernel_reports_misplaced_slices(gpu, rt, oracle):
    """The device-side check behind the in-kernel split-K reduction.  Mode 2 drops the launcher's condition
    on the grid, so with 6 tiles the slices of a tile run on different XCDs: the last arriver of each tile
    must notice (the arrival word counts slices per XCD), the next split-K launch must report it, sum with
    the second kernel from then on, and still be right.  Nothing faults or waits: only the values of the
    misplaced launch are undefined."""
    g = np.random.default_rng(37)
    M, N, K = 200, 328, 1024
    A = g.standard_normal((1, M, K)).astype(np.float16)
    B = (g.standard_normal((1, K, N)) * 0.1).astype(np.float16)
    want = oracle.gemm(A[0], B[0])
    num = knum(rt, "128x128_64x2r2_w2x4")   # 2 x 3 tiles
    zero = np.zeros((1, M, N), np.float16)
    gpu.homSetErrorMode(1)
    try:
        gpu.homSetSplitKInKernel(2)
        before = gpu.homSplitKInKernelLaunches()
        run_gemm(gpu, rt, A, B, None, zero, num, 3)          # misplaced on purpose; output not looked at
        assert gpu.homSplitKInKernelLaunches() == before + 1
        assert gpu.homGetLastError() == b""
        out = run_gemm(gpu, rt, A, B, None, zero, num, 3)    # finds the report, falls back
        assert b"different XCDs" in gpu.homGetLastError()
        assert gpu.homSplitKInKernelLaunches() == before + 1
        assert_close(out[0], want, **GEMM_TOL, what="launch that reported the misplaced slices")
        out = run_gemm(gpu, rt, A, B, None, zero, num, 3)    # stays on the second kernel, silently
        assert gpu.homGetLastError() == b"" and gpu.homSplitKInKernelLaunches() == before + 1
        assert_close(out[0], want, **GEMM_TOL, what="launch after the report")
        # switching the form on again measures the placement afresh and uses it where the grid allows
        gpu.homSetSplitKInKernel(1)
        A2 = g.standard_normal((1, 256, K)).astype(np.float16)
        B2 = (g.standard_normal((1, K, 512)) * 0.1).astype(np.float16)
        out = run_gemm(gpu, rt, A2, B2, None, np.zeros((1, 256, 512), np.float16), num, 3)   # 2 x 4 tiles
        assert gpu.homGetLastError() == b"" and gpu.homSplitKInKernelLaunches() == before + 2
        assert_close(out[0], oracle.gemm(A2[0], B2[0]), **GEMM_TOL, what="after re-arming")
    finally:
        gpu.homSetSplitKInKernel(3)   # the default
        gpu.homSetErrorMode(0)
