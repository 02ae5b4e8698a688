"""What the vendor libraries reach on the same GPU for the shapes this library
is measured on (a yardstick for the figures in bench.py, not part of any
product path): torch.matmul (hipBLASLt / rocBLAS), torch's fused
scaled_dot_product_attention and layer_norm, timed with events over
back-to-back launches.  The small GEMMs are dominated by PyTorch's per-call
host cost (~17 us) and say nothing about the kernels; the BERT-large sizes do.

    python hands-on-mlir_amd/vendor_yardstick.py        # needs a GPU
"""
import torch


def timed_us(fn, iters):
    for _ in range(5):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    best = float("inf")
    for _ in range(3):
        start.record()
        for _ in range(iters):
            fn()
        stop.record()
        torch.cuda.synchronize()
        best = min(best, start.elapsed_time(stop) / iters)
    return best * 1e3


def main():
    for (M, N, K) in [(1024, 3072, 768), (16384, 1024, 4096), (16384, 4096, 1024), (16384, 3072, 1024),
                      (16384, 1024, 1024)]:
        a = torch.randn(M, K, device="cuda").half()
        b = (torch.randn(K, N, device="cuda") * 0.05).half()
        out = torch.empty(M, N, device="cuda", dtype=torch.float16)
        us = timed_us(lambda: torch.matmul(a, b, out=out), 200 if M <= 1024 else 30)
        print(f"torch.matmul {M}x{N}x{K}: {us:.1f} us, {2 * M * N * K / us / 1e6:.0f} TFLOP/s", flush=True)
    q = torch.randn(32, 16, 512, 64, device="cuda").half()
    k, v = torch.randn_like(q), torch.randn_like(q)
    us = timed_us(lambda: torch.nn.functional.scaled_dot_product_attention(q, k, v), 30)
    print(f"scaled_dot_product_attention b32 h16 s512 d64: {us:.1f} us, "
          f"{4 * 32 * 16 * 512 * 512 * 64 / us / 1e6:.0f} TFLOP/s dense", flush=True)
    x = torch.randn(16384, 1024, device="cuda").half()
    us = timed_us(lambda: torch.nn.functional.layer_norm(x, (1024,)), 100)
    print(f"layer_norm 16384x1024: {us:.1f} us, {2 * 2 * 16384 * 1024 / us / 1e3:.0f} GB/s", flush=True)


if __name__ == "__main__":
    main()
