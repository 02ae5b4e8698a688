"""Autotune the GEMM shapes of BERT-base / BERT-large on the current GPU and
write csrc/gemm_tuned_table.inc (rebuild the library afterwards).

This is the MI355X counterpart of the reference's compile-time autotune pass
(lib/Dialect/HOMNVGPU/HOMNVGPUAutotunePass.cpp:52-92 -> GemmProfiler::profile):
for every (M, N, K, activation) it times each eligible manifest kernel x
split-K factor through homGemmProfile and records the winner by NAME, so the
table survives manifest reordering.

    python hands-on-mlir_amd/tune_gemm.py [output.inc]     # needs a GPU
"""
import ctypes
import importlib
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))


def bert_shapes():
    shapes = []
    for (hidden, ffn, rows) in [(768, 3072, (128, 1024, 2048, 4096)),      # base: b1..b32 x s128
                                (1024, 4096, (128, 1024, 4096, 16384))]:  # large, up to b32 x s512
        for m in rows:
            for act_gelu in (1, 2):
                shapes.append((m, ffn, hidden, act_gelu))
            shapes += [(m, 3 * hidden, hidden, 0), (m, hidden, hidden, 0), (m, hidden, ffn, 0)]
    shapes.append((64, 1024, 4096, 0))  # skinny split-K stress case
    return shapes


def main():
    sys.path.insert(0, os.path.dirname(HERE))
    rt = importlib.import_module("hands-on-mlir_amd.hom_runtime")
    lib = rt.load_runtime()
    names = {i: n for i, n, _, _ in rt.manifest()}
    lines = []
    for (M, N, K, act) in bert_shapes():
        idx, sk, ms = ctypes.c_int64(), ctypes.c_int32(), ctypes.c_float()
        beta = 1.0 if (act == 0 and N in (768, 1024) and K != N // 3) else 0.0
        lib.homGemmProfile(M, N, K, act, 1.0, beta, ctypes.byref(idx), ctypes.byref(sk), ctypes.byref(ms))
        if idx.value < 0:
            continue
        tf = 2.0 * M * N * K / (ms.value * 1e9)
        lines.append(f'    {{{M}, {N}, {K}, {act}, "{names[idx.value]}", {sk.value}}}, '
                     f'// {ms.value * 1e3:.2f} us, {tf:.1f} TFLOP/s')
        print(lines[-1], flush=True)
    out = sys.argv[1] if len(sys.argv) > 1 else os.path.join(HERE, "csrc", "gemm_tuned_table.inc")
    with open(out, "w") as f:
        f.write("// (M, N, K, activation: 0 linear / 1 GELU erf / 2 GELU tanh, kernel name, split-K)\n"
                "// Written by hands-on-mlir_amd/tune_gemm.py on an MI355X; do not edit by hand.\n")
        f.write("\n".join(lines) + "\n")
    print("wrote", out)


if __name__ == "__main__":
    main()
