"""Times torch.matmul (hipBLASLt / rocBLAS behind it) on fp16 and bf16 operands at the shapes of config 5, for
context beside this library's MFMA GEMM figures: the program behind profiles/gemm_vendor_library_context.txt.
Not a test and not part of the product; torch is only the way to reach the vendor library here."""
import torch, time
torch.backends.cuda.matmul.allow_fp16_reduced_precision_reduction = False
dev = "cuda"
def bench(M, N, K, dtype=torch.float16):
    x = torch.randn(M, K, device=dev, dtype=dtype)
    w = torch.randn(N, K, device=dev, dtype=dtype) * 0.02
    for _ in range(10): y = x @ w.t()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    best = 1e9
    for _ in range(5):
        e0.record()
        for _ in range(50): y = x @ w.t()
        e1.record(); torch.cuda.synchronize()
        best = min(best, e0.elapsed_time(e1) / 50)
    fl = 2.0 * M * N * K
    print(f"torch {dtype} M={M} N={N} K={K}: {best*1e3:.2f} us  {fl/best/1e9:.1f} TFLOP/s  frac {fl/best/1e9/2500:.3f}", flush=True)
for shp in [(2048, 4864, 896), (2048, 896, 4864), (512, 4864, 896), (8192, 8192, 8192), (4096, 4864, 896), (16384, 4864, 896)]:
    bench(*shp)
    bench(*shp, dtype=torch.bfloat16)
