"""Library GEMM yardstick: the vendor bf16 GEMM (hipBLASLt through torch.matmul) on dense operands of
the benchmark shape 8192 x 4096 x 14336, i.e. what the reference's dequantize-then-matmul forward
(src/Metis/Metis/bitlinear.py:435) costs on this part once the operands are already dequantized.

    python3 fp4-post_amd/metis_hip/tools/library_gemm_reference.py
"""
import torch


def main(M=8192, K=4096, N=14336, reps=20):
    g = torch.Generator().manual_seed(1003)
    x = torch.randn(M, K, generator=g).bfloat16().cuda()
    w = (torch.randn(N, K, generator=g) * 0.02).bfloat16().cuda()
    for _ in range(5):
        torch.matmul(x, w.T)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        torch.matmul(x, w.T)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / reps
    print(f"torch.matmul bf16 {M}x{K}x{N}: {ms * 1e3:.1f} us  {2.0 * M * N * K / ms / 1e9:.1f} TFLOP/s")


if __name__ == "__main__":
    main()
