"""Usage example: fp16 preshuffle GEMM, the problem of the reference's tutorial (examples/04-preshuffle_gemm.py:190-204):
C[4096,4096] = A[4096,4096] @ B[4096,4096]^T with B preshuffled on the host, checked with the tutorial's tolerance
``1e-3 + 1e-3*|expected|`` against ``A @ B.T``.

    python -m flydsl_amd.examples.preshuffle_gemm_fp16
"""

from __future__ import annotations

import torch

from flydsl_amd.kernels.gemm.preshuffle_gemm import compile_preshuffle_gemm
from flydsl_amd.layout import shuffle_weight


def main(M: int = 4096, N: int = 4096, K: int = 4096, iters: int = 20) -> bool:
    A = torch.randn(M, K, dtype=torch.float16).cuda()
    B = torch.randn(N, K, dtype=torch.float16).cuda()
    C = torch.zeros(M, N, dtype=torch.float16).cuda()
    preshuffle_B = shuffle_weight(B, layout=(16, 16))

    gemm = compile_preshuffle_gemm(N=N, K=K, tile_m=128, tile_n=128, tile_k=64, in_dtype="fp16", out_dtype="fp16")
    none = torch.empty(0, dtype=torch.float32, device="cuda")
    bias = torch.empty(0, dtype=torch.float16, device="cuda")
    gemm(C, A, preshuffle_B, none, none, bias, M, N, torch.cuda.current_stream())
    torch.cuda.synchronize()

    expected = (A @ B.T).to(torch.float32)
    actual = C.to(torch.float32)
    tol = 1e-3 + 1e-3 * expected.abs()
    max_violation = ((actual - expected).abs() - tol).max().item()
    is_correct = max_violation <= 0
    print("Result correct:", is_correct)
    if not is_correct:
        print("Max violation:", max_violation)

    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        gemm(C, A, preshuffle_B, none, none, bias, M, N, torch.cuda.current_stream())
    stop.record()
    torch.cuda.synchronize()
    us = start.elapsed_time(stop) * 1e3 / iters
    print(f"Throughput: {us:.1f} us, {2 * M * N * K / us / 1e6:.2f} TFLOPS")
    return is_correct


if __name__ == "__main__":
    raise SystemExit(0 if main() else 1)
