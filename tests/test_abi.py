"""CPU-side checks of the drop-in boundary: the library loads, exports every
symbol the header declares, and rejects bad arguments before touching the GPU."""
import ctypes
import importlib
import json
import os
import re
import subprocess
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "hom_amdgpu_runner_utils.h")


def declared_symbols():
    text = open(HEADER).read()
    names = set(re.findall(r"HOM_EXPORT\s+[\w\s\*]+?\b(\w+)\s*\(", text))
    for op, sfx in re.findall(r"HOM_ELEMENTWISE_DECL\((\w+), (\w+)\)", text):
        names.add(f"thrustElementwise{op}{sfx}")
    names.discard("thrustElementwiseopsuffix")
    return names


def test_header_symbols_all_exported(rt):
    lib = rt.load_runtime()
    names = declared_symbols()
    assert len(names) >= 45
    for n in sorted(names):
        assert hasattr(lib, n), f"{n} declared in the header but not exported"
    # and the ctypes table covers exactly the header
    assert names == set(rt.SIGNATURES), names ^ set(rt.SIGNATURES)


def test_reference_symbol_names_present(rt):
    """Names the compiler emits calls to (include/Conversions/Function/FunctionUtils.h:12-49)."""
    lib = rt.load_runtime()
    for n in ["cutlassGemmF16", "cutlassGemmF32", "nvteGemmF16", "nvteLayernormF16", "nvteLayernormF32",
              "nvteBertAttentionF16", "nvteBertAttentionF32", "alloc3DMemRefNVGPUF16",
              "alloc3DMemRefNVGPUF32", "alloc1DMemRefNVGPUI32", "allocConstantNVGPUF16",
              "allocConstantNVGPUF32", "deallocNVGPUF16", "deallocNVGPUF32", "deallocNVGPUI32",
              "thrustElementwiseAddF16", "thrustElementwiseSubF32", "thrustGatherF16",
              "thrustCuSeqLenI64", "thrustCuSeqLenI32", "cutlassGemmWithVarMeanF16",
              "cutlassLayernormGemmF16", "cutlassLayernormGemmF32", "printMemrefSizeF16"]:
        assert hasattr(lib, n)


def test_unranked_memref_is_16_byte_pod(rt):
    assert ctypes.sizeof(rt.CUnrankedMemRef) == 16


def test_manifest_is_well_formed(rt):
    man = rt.manifest()
    assert len(man) >= 30
    names = [m[1] for m in man]
    assert len(set(names)) == len(names)
    lib = rt.load_runtime()
    for idx, name, act, align in man:
        # activation is derived from the name the way the reference's runner does
        # (GemmRunner.h:200-206): "gelu" -> 1, "linear" -> 0
        assert act == (1 if "gelu" in name else 0)
        assert ("linear" in name) != ("gelu" in name)
        assert align in (1, 8)
        assert lib.homGemmManifestFind(name.encode()) == idx
    assert lib.homGemmManifestFind(b"no_such_kernel") == -1
    assert lib.homGemmManifestName(-1) == b"" and lib.homGemmManifestActivation(10**6) == -1
    # every (epilogue) has an unaligned fallback
    assert any(a == 1 and "linear" in n for _, n, _, a in man)


def test_select_returns_compatible_kernel(rt):
    lib = rt.load_runtime()
    man = rt.manifest()
    idx, sk = ctypes.c_int64(), ctypes.c_int32()
    for (M, N, K, act) in [(1024, 2304, 768, 0), (1024, 3072, 768, 1), (1024, 3072, 768, 2),
                           (1024, 768, 3072, 0), (64, 1024, 4096, 0), (7, 13, 5, 0), (16384, 4096, 1024, 1),
                           (1024, 30522, 768, 0), (64, 250, 72, 1), (64, 251, 72, 0), (64, 256, 76, 0)]:
        lib.homGemmSelect(M, N, K, act, ctypes.byref(idx), ctypes.byref(sk))
        _, name, a, align = man[idx.value]
        assert a == (1 if act else 0)
        assert ("gelutanh" in name) == (act == 2)
        assert sk.value >= 1 and sk.value <= max(1, min(16, K // 128))
        if N % 2 or K % 8:
            assert align == 1
        elif N % 8:
            # even N: only the register-staged family reads rows that start at 4-byte boundaries
            assert align == 8 and "_64x2r" in name


def test_selection_model_without_the_tuned_table():
    """The timing model that answers for untuned shapes, asked about shapes the autotuner measured: it must land on
    the tile class the measurements favour (its own process: the switch is read once)."""
    code = r"""
import ctypes, importlib, json, sys
sys.path.insert(0, %r)
rt = importlib.import_module("hands-on-mlir_amd.hom_runtime")
lib = rt.load_runtime(); man = rt.manifest()
idx, sk = ctypes.c_int64(), ctypes.c_int32()
out = {}
for shape in [(16384, 1024, 4096, 0), (16384, 4096, 1024, 1), (1024, 768, 768, 0), (1024, 2304, 768, 0),
              (128, 1024, 4096, 0), (1024, 30522, 768, 0), (4096, 768, 3072, 0)]:
    lib.homGemmSelect(*shape, ctypes.byref(idx), ctypes.byref(sk))
    out["x".join(map(str, shape))] = [man[idx.value][1], sk.value]
print(json.dumps(out))
""" % ROOT
    env = dict(os.environ, HOM_GEMM_IGNORE_TUNED_TABLE="1")
    res = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=120)
    assert res.returncode == 0, res.stderr
    picks = json.loads(res.stdout.strip().splitlines()[-1])
    assert "_256x256_64x2r1_w2x4_" in picks["16384x1024x4096x0"][0]
    assert "_256x256_64x2r1_w2x4_" in picks["16384x4096x1024x1"][0] and picks["16384x4096x1024x1"][0].endswith("_gelu")
    assert "_64x64_64x2r2_" in picks["1024x768x768x0"][0] and picks["1024x768x768x0"][1] == 1
    assert "_128x128_64x2r2_w2x4_" in picks["1024x2304x768x0"][0]
    assert "_128x128_64x2r2_w2x4_" in picks["4096x768x3072x0"][0]
    assert "_64x64_" in picks["128x1024x4096x0"][0] and picks["128x1024x4096x0"][1] > 1    # skinny: split-K
    assert "_64x2r" in picks["1024x30522x768x0"][0] and picks["1024x30522x768x0"][1] == 1  # even N: pipe family


def build_autotune_usage(tmp_path):
    exe = str(tmp_path / "autotune_pass_usage")
    lib_dir = os.path.join(ROOT, "hands-on-mlir_amd", "lib")
    cmd = ["g++", "-std=c++17", "-O1", "-Wall", "-I", os.path.join(ROOT, "include"),
           os.path.join(ROOT, "tests", "modules", "autotune_pass_usage.cpp"),
           "-L", lib_dir, "-lhom_amdgpu_runner_utils", f"-Wl,-rpath,{lib_dir}", "-o", exe]
    res = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stderr
    return exe


def test_autotune_pass_source_compiles_against_the_profiler_header(rt, tmp_path):
    """The reference's pass includes NVGPUKernels/GemmProfiler.h and calls GemmProfiler::profile;
    its library-facing code must compile and link unchanged against this repo's header and library."""
    rt.load_runtime()
    exe = build_autotune_usage(tmp_path)
    res = subprocess.run([exe], capture_output=True, text=True, timeout=60)
    assert res.returncode == 0, res.stderr
    assert int(res.stdout.strip()) == len(rt.manifest())


@pytest.mark.gpu
def test_autotune_pass_usage_runs_on_the_gpu(rt, tmp_path):
    rt.load_runtime()
    exe = build_autotune_usage(tmp_path)
    res = subprocess.run([exe, "run"], capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stdout + res.stderr
    num, split, name = res.stdout.strip().splitlines()[-1].split()
    assert 0 <= int(num) <= len(rt.manifest()) and int(split) >= 1
    # 0 = the [N, K] path of nvteGemmF16 was the fastest (the reference's profiler returns -1 then)
    assert name == "nvte" if int(num) == 0 else name.endswith("_linear")


# ---- argument checking: runs without a GPU because every check precedes the
# first HIP call.  Default mode aborts (reference: assert / exit(1)); mode 1
# records the message instead.
def _errors(rt, fn):
    lib = rt.load_runtime()
    lib.homSetErrorMode(1)
    try:
        lib.homGetLastError()
        fn(lib)
        return lib.homGetLastError().decode()
    finally:
        lib.homSetErrorMode(0)


def test_gemm_argument_checks(rt):
    M = rt.MemRef
    a, b, d = M(256, [1, 16, 32]), M(256, [1, 32, 8]), M(256, [1, 16, 8])

    def call(A, B, C, D, num=1, sk=1, beta=0.0):
        return lambda lib: lib.cutlassGemmF16(*A.args(), False, *B.args(), False, *C.args(), *D.args(),
                                              0, 1.0, beta, num, sk)
    assert "rank 3" in _errors(rt, call(M(256, [16, 32]), b, d, d))
    assert "K mismatch" in _errors(rt, call(a, M(256, [1, 31, 8]), d, d))
    assert "D is" in _errors(rt, call(a, b, d, M(256, [1, 16, 9])))
    assert "outside the manifest" in _errors(rt, call(a, b, d, d, num=10**6))
    assert "negative kernel number" in _errors(rt, call(a, b, d, d, num=-1))
    assert "split-K" in _errors(rt, call(a, b, d, d, sk=0))
    assert "not broadcastable" in _errors(rt, call(a, b, M(256, [1, 3, 8]), d, beta=1.0))
    assert "contiguous" in _errors(rt, call(M(256, [1, 16, 32], [1024, 64, 1]), b, d, d))
    # aligned kernels reject odd K/N the way can_implement() does
    odd = call(M(256, [1, 16, 31]), M(256, [1, 31, 8]), d, d)
    assert "multiples of 8" in _errors(rt, odd)


def test_nvte_gemm_argument_checks(rt):
    M = rt.MemRef
    a, bt, d = M(256, [1, 16, 32]), M(256, [1, 8, 32]), M(256, [1, 16, 8])

    def call(transa=False, transb=True, alpha=1.0, beta=0.0, C=d, D=d):
        return lambda lib: lib.nvteGemmF16(*a.args(), transa, *bt.args(), transb, *C.args(), *D.args(),
                                           0, alpha, beta, 0, 0)
    assert "transa" in _errors(rt, call(transa=True))
    assert "transb" in _errors(rt, call(transb=False))
    assert "alpha must be 1" in _errors(rt, call(alpha=2.0))
    assert "beta must be 0 or 1" in _errors(rt, call(beta=0.5))
    assert "C must alias D" in _errors(rt, call(beta=1.0, C=M(512, [1, 16, 8])))


def test_other_argument_checks(rt):
    M = rt.MemRef
    assert "rank must be 2 or 3" in _errors(rt, lambda lib: lib.nvteLayernormF16(4, M(256, [1, 2, 3, 4]).descriptor, 1e-5))
    qkv, cu, out = M(256, [2, 64, 2304]), M(256, [3]), M(256, [2, 64, 768])
    att = lambda q, c, o, heads=12: (lambda lib: lib.nvteBertAttentionF16(*q.args(), *c.args(), *o.args(), 0.125, heads))
    assert "multiple of 3 * heads" in _errors(rt, att(qkv, cu, out, heads=7))
    assert "cu_seqlens" in _errors(rt, att(qkv, M(256, [2]), out))
    assert "Out is" in _errors(rt, att(qkv, cu, M(256, [2, 64, 767])))
    assert "head size" in _errors(rt, att(M(256, [2, 64, 2304]), cu, out, heads=24))
    ew = lambda a, b, o: (lambda lib: lib.thrustElementwiseAddF16(*a.args(), *b.args(), *o.args()))
    assert "only B can broadcast" in _errors(rt, ew(M(256, [3, 1, 3]), M(256, [3, 3, 3]), M(256, [3, 1, 3])))
    assert "ranks differ" in _errors(rt, ew(M(256, [3, 3]), M(256, [3, 3, 3]), M(256, [3, 3])))
    ga = lambda i, v, o: (lambda lib: lib.thrustGatherF16(*i.args(), *v.args(), *o.args()))
    assert "value must be" in _errors(rt, ga(M(256, [2, 4]), M(256, [2, 10, 8]), M(256, [2, 4, 8])))
    cs = lambda i, o: (lambda lib: lib.thrustCuSeqLenI64(*i.args(), *o.args()))
    assert "expected 9" in _errors(rt, cs(M(256, [8, 128]), M(256, [8])))
    assert "fp32 attention" in _errors(rt, lambda lib: lib.nvteBertAttentionF32(*qkv.args(), *cu.args(), *out.args(), 0.125, 12))


def test_default_error_mode_aborts(rt):
    """Reference behaviour: a failed check kills the process (assert / exit(1))."""
    code = (
        "import importlib, sys; sys.path.insert(0, %r);"
        "rt = importlib.import_module('hands-on-mlir_amd.hom_runtime');"
        "lib = rt.load_runtime();"
        "m = rt.MemRef(256, [1, 2, 3, 4]);"
        "lib.nvteLayernormF16(4, m.descriptor, 1e-5); print('survived')" % ROOT)
    p = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True)
    assert p.returncode != 0 and "survived" not in p.stdout
    assert "rank must be 2 or 3" in p.stderr


def test_constant_loader_rejects_bad_files(rt, tmp_path, monkeypatch):
    monkeypatch.setenv("HOM_CONSTANT_DIR", str(tmp_path))
    (tmp_path / "1.txt").write_text("2 3\n1 2 3 4 5 6\n")
    (tmp_path / "2.txt").write_text("1 2 3\n1 2 3 4 5\n")
    assert "cannot open" in _errors(rt, lambda lib: lib.allocConstantNVGPUF16(99))
    assert "expected 3" in _errors(rt, lambda lib: lib.allocConstantNVGPUF16(1))
    assert "holds 5 values, expected 6" in _errors(rt, lambda lib: lib.allocConstantNVGPUF16(2))


def test_binary_constant_files(rt, tmp_path, monkeypatch):
    """Writer layout (40-byte header, raw values) and the loader's header checks."""
    import struct
    weights = importlib.import_module("hands-on-mlir_amd.weights")
    a = (np.arange(24, dtype=np.float32) * 0.37 - 3).reshape(2, 3, 4).astype(np.float16)
    path = weights.write_binary(str(tmp_path), 7, a)
    raw = open(path, "rb").read()
    assert len(raw) == 40 + 48
    assert struct.unpack("<4sIIIqqq", raw[:40]) == (b"HOMW", 1, 2, 3, 2, 3, 4)
    assert np.array_equal(np.frombuffer(raw[40:], np.float16).reshape(2, 3, 4), a)
    text = open(weights.write_text(str(tmp_path), 8, a[0])).read().split("\n")
    assert text[0] == "1 3 4"
    assert np.array_equal(np.array(text[1].split(), np.float32).astype(np.float16), a[0].ravel())
    monkeypatch.setenv("HOM_CONSTANT_DIR", str(tmp_path))
    (tmp_path / "3.bin").write_bytes(b"NOPE" + raw[4:])
    (tmp_path / "4.bin").write_bytes(raw[:-2])
    assert "not a HOMW v1 rank-3 file" in _errors(rt, lambda lib: lib.allocConstantNVGPUF16(3))
    assert "holds 23 values, expected 24" in _errors(rt, lambda lib: lib.allocConstantNVGPUF16(4))



def test_folded_layernorm_gemm_argument_checks(rt):
    """The folded layer norm + GEMM entry point refuses what its kernels do not implement, before any launch."""
    M = rt.MemRef
    a, b, d = M(256, [1, 64, 128]), M(256, [1, 128, 64]), M(256, [1, 64, 64])
    stats = ctypes.c_void_p(4096)

    def call(mode, act=0, beta=0.0, stats_in=None, col=None, stats_out=None, pieces=1, A=a, B=b):
        return lambda lib: lib.homGemmFoldedLayernormF16(*A.args(), *B.args(), *d.args(), *d.args(), mode, act, 1.0,
                                                         beta, stats_in, pieces, 1e-5, col, stats_out, 0)
    assert "mode must be 1" in _errors(rt, call(3))
    assert "0 pieces" in _errors(rt, call(1, stats_in=stats, col=stats, pieces=0))
    assert "not supported" in _errors(rt, call(1, stats_in=stats))                 # normalising A needs colsum(B)
    assert "not supported" in _errors(rt, call(1, stats_out=stats))                # mode 1 emits no sums
    assert "not supported" in _errors(rt, call(2, act=1, beta=1.0))                # no activation after the residual
    assert "not supported" in _errors(rt, call(2, stats_in=stats, beta=0.0))       # nothing to normalise
    assert "K mismatch" in _errors(rt, call(1, B=M(256, [1, 120, 64])))
    assert "column sums" in _errors(rt, lambda lib: lib.homColumnSumsF16(2, M(256, [128, 64]).descriptor, stats))
    lib = rt.load_runtime()
    for (m, n, k) in [(1024, 768, 768), (16384, 1024, 1024), (64, 64, 64)]:
        pieces = lib.homFoldedLayernormPieces(m, n, k, 0, 0)
        assert 1 <= pieces <= (n + 63) // 64 and pieces in {-(-n // e) for e in (64, 128, 256)}
