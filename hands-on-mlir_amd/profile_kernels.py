"""Tiny single-kernel workloads to run under rocprofv3 (kernel trace or --pmc).

    python3 hands-on-mlir_amd/profile_kernels.py <what> [iters] [tile]

tile (GEMM workloads only): run the manifest kernel whose name holds `_<tile>_`
(e.g. 256x256_64x2r1_w2x2) instead of the tuned one.

what:  gemm1      FFN1 GEMM + bias + tanh-GELU, M=1024 K=768 N=3072 (tuned kernel)
       gemm5      BERT-large FFN2 GEMM, M=16384 K=4096 N=1024
       gemm5g     BERT-large FFN1 GEMM + bias + erf-GELU, M=16384 K=1024 N=4096
       gemm_skinny  the skinny split-K stress case, M=64 K=4096 N=1024, as the
                  library runs it (tuned kernel and split factor)
       splitk_ab  the two forms of the split-K reduction side by side (a second
                  kernel / the last slice to finish, inside the GEMM kernel), in
                  a replayed HIP graph, over split factors 1..16 of the skinny
                  case and of two BERT-base shapes
       layernorm  in-place layer norm, 16384 x 1024, the same tensor launch after
                  launch (it stays in the 256 MB Infinity Cache: a cache rate)
       layernorm_cold  the same over 24 tensors walked round-robin (805 MB:
                  every launch reads from and writes to HBM)
       add_cold   elementwise add 16384 x 1024 over 8 (a, b, out) triples
                  walked round-robin (805 MB)
       attention  packed-QKV attention, b8 s128 h12
       attention5 packed-QKV attention, b32 s512 h16, full-length sequences
       lnpair     the layer-norm pair at BERT-large size: GEMM + row statistics
                  16384x1024x1024, then the GEMM of the normalised rows
                  16384x4096x1024, next to the two plain GEMMs
       copy       plain device copy of 256 MiB (counter calibration: reads and
                  writes exactly 268435456 bytes each)
       operands   gemm5 and gemm5g on random operands and on operands that are
                  all zero (same instructions and traffic, no switching in the
                  data paths): what the chip's power management costs the kernel
       mfma_ceiling  v_mfma_f32_32x32x16_f16 back to back on register operands,
                  no memory access in the loop, 8 wavefronts per CU: the rate the
                  matrix cores sustain on zero and on random operands, alone and
                  with 4 / 8 independent fp32 FMAs behind every MFMA
Each call goes through the C-ABI via the C++ driver's timing helpers.
"""
import ctypes
import importlib
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def main():
    what = sys.argv[1]
    iters = int(sys.argv[2]) if len(sys.argv) > 2 else 20
    rt = importlib.import_module("hands-on-mlir_amd.hom_runtime")
    drv, lib = rt.load_driver(), rt.load_runtime()
    idx, sk = ctypes.c_int64(), ctypes.c_int32()
    tile = sys.argv[3] if len(sys.argv) > 3 else None

    def pick(m, n, k, act):
        lib.homGemmSelect(m, n, k, act, ctypes.byref(idx), ctypes.byref(sk))
        if tile:
            want = {0: "_linear", 1: "_gelu", 2: "_gelutanh"}[act]
            hits = [i for i, name, _, _ in rt.manifest() if f"_{tile}_" in name and name.endswith(want)]
            assert hits, f"no manifest kernel matches {tile}"
            idx.value, sk.value = hits[0], 1

    if what == "gemm1":
        pick(1024, 3072, 768, 2)
        ms = drv.homTimeGemm(1024, 3072, 768, 2, 1, idx.value + 1, sk.value, iters, 3)
        print(f"gemm1 {lib.homGemmManifestName(idx.value).decode()} splitK {sk.value}: {ms * 1e3:.2f} us")
    elif what == "gemm5":
        pick(16384, 1024, 4096, 0)
        ms = drv.homTimeGemm(16384, 1024, 4096, 0, 0, idx.value + 1, sk.value, iters, 3)
        print(f"gemm5 {lib.homGemmManifestName(idx.value).decode()} splitK {sk.value}: {ms * 1e3:.2f} us")
    elif what == "gemm5g":
        pick(16384, 4096, 1024, 1)
        ms = drv.homTimeGemm(16384, 4096, 1024, 1, 1, idx.value + 1, sk.value, iters, 3)
        print(f"gemm5g {lib.homGemmManifestName(idx.value).decode()} splitK {sk.value}: {ms * 1e3:.2f} us")
    elif what == "gemm_skinny":
        pick(64, 1024, 4096, 0)
        ms = drv.homTimeGemm(64, 1024, 4096, 0, 0, idx.value + 1, sk.value, iters, 3)
        print(f"gemm_skinny {lib.homGemmManifestName(idx.value).decode()} splitK {sk.value}: {ms * 1e3:.2f} us")
    elif what == "splitk_ab":
        num = {n: i + 1 for i, n, _, _ in rt.manifest()}
        stem = "hom_gfx950_mfma_f16_s32x32x16gemm_f16_%s_nn_align8_linear"
        try:
            for (m, n, k) in ((64, 1024, 4096), (1024, 768, 3072), (1024, 768, 768)):
                for tile in ("64x64_64q3_w2x2", "64x64_64x2r2_w2x2", "128x128_64q3_w2x4"):
                    row = []
                    for sk in (1, 2, 3, 4, 6, 8, 12, 16):
                        if k // 64 < 2 * sk:
                            continue
                        us = []
                        for on in (0, 1):
                            lib.homSetSplitKInKernel(on)
                            us.append(min(drv.homTimeGemmInGraph(m, n, k, 0, 0, num[stem % tile], sk, 1000, 100)
                                          for _ in range(2)) * 1e3)
                        row.append(f"splitK {sk}: {us[0]:.2f} / {us[1]:.2f}")
                    print(f"splitk_ab {m}x{n}x{k} {tile} (us, second kernel / in kernel)  " + "  ".join(row),
                          flush=True)
        finally:
            lib.homSetSplitKInKernel(3)  # the default
    elif what == "layernorm":
        print(f"layernorm 16384x1024: {drv.homTimeLayernorm(16384, 1024, 0, iters, 3) * 1e3:.2f} us")
    elif what == "layernorm_cold":
        ms = drv.homTimeLayernormRotating(16384, 1024, 0, 24, iters, 3)
        print(f"layernorm 16384x1024 over 24 rotating tensors: {ms * 1e3:.2f} us")
    elif what == "add_cold":
        ms = drv.homTimeElementwiseAddRotating(16384, 1024, 8, iters, 3)
        print(f"add 16384x1024 over 8 rotating triples: {ms * 1e3:.2f} us")
    elif what == "attention":
        lens = (ctypes.c_int32 * 8)(83, 128, 57, 101, 32, 120, 64, 99)
        print(f"attention b8 s128 h12: {drv.homTimeAttention(8, 128, 12, lens, iters, 3) * 1e3:.2f} us")
    elif what == "attention5":
        lens = (ctypes.c_int32 * 32)(*([512] * 32))
        print(f"attention b32 s512 h16: {drv.homTimeAttention(32, 512, 16, lens, iters, 3) * 1e3:.2f} us")
    elif what == "lnpair":
        import torch
        M = rt.MemRef.from_tensor
        g = torch.Generator(device="cuda").manual_seed(0)
        rnd = lambda *shape, scale=1.0: (torch.randn(shape, device="cuda", generator=g) * scale).half()
        x, w1, w2 = rnd(1, 16384, 1024), rnd(1, 1024, 1024, scale=0.03), rnd(1, 1024, 4096, scale=0.03)
        d1 = torch.zeros((1, 16384, 1024), dtype=torch.float16, device="cuda")
        d2 = torch.zeros((1, 16384, 4096), dtype=torch.float16, device="cuda")
        var = torch.zeros((1, 16384, 1), dtype=torch.float16, device="cuda")
        mean = torch.zeros_like(var)
        mx, mw1, mw2, md1, md2, mv, mm = (M(t) for t in (x, w1, w2, d1, d2, var, mean))
        for _ in range(iters):
            lib.cutlassGemmF16(*mx.args(), False, *mw1.args(), False, *md1.args(), *md1.args(), 0, 1.0, 0.0, 0, 1)
            lib.cutlassGemmF16(*md1.args(), False, *mw2.args(), False, *md2.args(), *md2.args(), 0, 1.0, 0.0, 0, 1)
            lib.cutlassGemmWithVarMeanF16(*mx.args(), *mw1.args(), *md1.args(), *md1.args(), *mv.args(), *mm.args(),
                                          1.0, 0.0, 0, 1e-5)
            lib.cutlassLayernormGemmF16(*md1.args(), *mw2.args(), *md2.args(), *md2.args(), *mv.args(), *mm.args(),
                                        1.0, 0.0, 0)
        torch.cuda.synchronize()
        print("ln pair 16384x1024x1024 -> 16384x4096x1024 x", iters)
    elif what == "operands":
        for (m, n, k, act, bias, label) in ((16384, 1024, 4096, 0, 0, "gemm5"), (16384, 4096, 1024, 1, 1, "gemm5g")):
            pick(m, n, k, act)
            for rep in range(2):
                rnd = drv.homTimeGemm(m, n, k, act, bias, idx.value + 1, sk.value, iters, 3) * 1e3
                zero = drv.homTimeGemmZeroOperands(m, n, k, act, bias, idx.value + 1, sk.value, iters, 3) * 1e3
                tf = lambda us: 2.0 * m * n * k / us / 1e6
                print(f"{label} {lib.homGemmManifestName(idx.value).decode()}: random operands {rnd:.2f} us "
                      f"({tf(rnd):.0f} TFLOP/s), zero operands {zero:.2f} us ({tf(zero):.0f} TFLOP/s)", flush=True)
    elif what == "mfma_ceiling":
        for valu in (0, 4, 8):
            for rnd in (0, 1, 0, 1):
                tf = drv.homMfmaCeilingProbe(rnd, valu)
                print(f"mfma only loop, {valu} fp32 FMAs per MFMA, {'random' if rnd else 'zero'} operands: "
                      f"{tf:.0f} TFLOP/s = {tf / 2500:.3f} of the 2.5 PFLOP/s peak", flush=True)
    elif what == "copy":
        import torch
        src = torch.ones(128 * 1024 * 1024, dtype=torch.float16, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(iters):
            dst.copy_(src)
        torch.cuda.synchronize()
        print("copy 268435456 bytes x", iters)
    else:
        sys.exit(__doc__)


if __name__ == "__main__":
    main()
