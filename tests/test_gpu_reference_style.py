"""The reference's harness flow (tests/kernels/test_preshuffle_gemm.py:116-314, 342-466), written against the
reference's own module names through ``flydsl_amd.compat.install()``: quantise on the device, preshuffle, run through
``flyc.compile`` + ``run_perftest`` (eager and graph), accept with ``verify_output(rtol=0.1, atol=0.1)``, and check
the sentinel guard rows.  The aliases are removed again afterwards so that they do not leak into the other tests."""

import sys
import textwrap

import pytest

pytestmark = pytest.mark.gpu

SCRIPT = textwrap.dedent('''
    import torch

    import flydsl.compiler as flyc
    import flydsl.expr as fx
    from flydsl.runtime.device import get_rocm_arch
    from kernels.gemm.mxfp4_preshuffle import launch_gemm
    from kernels.gemm.preshuffle_gemm import compile_preshuffle_gemm
    from tests.kernels.utils import gemm_common_utils
    from tests.test_common import run_perftest, verify_output
    from tests.utils import pertoken_quant, shuffle_weight

    assert get_rocm_arch() == "gfx950"
    DTYPE_FP8 = torch.float8_e4m3fn

    def run_torch(a, b, scale_a, scale_b, dtype=torch.float32):
        if scale_a is not None:
            a_f32 = a.to(torch.float32) * scale_a.view(-1, 1); b_f32 = b.to(torch.float32) * scale_b.view(-1, 1)
        else:
            a_f32, b_f32 = a.to(torch.float32), b.to(torch.float32)
        return torch.mm(a_f32, b_f32.T).to(dtype)

    def a8_case(in_dtype, M, N, K, tile_m, tile_n, tile_k, test_graph):
        launch_fn = compile_preshuffle_gemm(N=N, K=K, tile_m=tile_m, tile_n=tile_n, tile_k=tile_k, in_dtype=in_dtype, out_dtype="bf16")
        device = torch.device("cuda")
        a_fp32 = torch.randn(M, K, device=device); b_fp32_t = torch.randn(N, K, device=device)
        if in_dtype in ("fp16", "bf16"):
            dt = torch.float16 if in_dtype == "fp16" else torch.bfloat16
            a_q, b_q, scale_a, scale_b = a_fp32.to(dt), b_fp32_t.to(dt), None, None
        else:
            qd = torch.int8 if in_dtype == "int8" else DTYPE_FP8
            a_q, scale_a = pertoken_quant(a_fp32, quant_dtype=qd); b_q, scale_b = pertoken_quant(b_fp32_t, quant_dtype=qd)
        b_shuffled = shuffle_weight(b_q.contiguous(), layout=(16, 16))
        c_ref = run_torch(a_q, b_q, scale_a, scale_b)
        grid_rows = ((M + tile_m - 1) // tile_m) * tile_m
        sentinel = torch.tensor(-8192.0, dtype=torch.bfloat16, device=device)
        c_alloc = torch.full((grid_rows, N), sentinel, dtype=torch.bfloat16, device=device)
        c_out = c_alloc[:M]
        sa = scale_a.contiguous().view(-1) if scale_a is not None else torch.empty(0, device=device)
        sb = scale_b.contiguous().view(-1) if scale_b is not None else torch.empty(0, device=device)
        as_i8 = lambda t: t.view(torch.int8) if "float8" in str(t.dtype) else t
        bias = torch.empty(0, dtype=torch.bfloat16, device=device)
        def gemm_args(c, a, b, sa_, sb_):
            return (c.contiguous().view(-1), as_i8(a.contiguous().view(-1)), as_i8(b.contiguous().view(-1)), sa_, sb_, bias, M, N,
                    torch.cuda.current_stream())
        compiled = flyc.compile(launch_fn, *gemm_args(c_out, a_q, b_shuffled, sa, sb))
        _, us = run_perftest(lambda c, a, b, s1, s2: compiled(*gemm_args(c, a, b, s1, s2)), c_out, a_q, b_shuffled, sa, sb,
                             num_iters=6, num_warmup=2, testGraph=test_graph)
        torch.cuda.synchronize()
        assert verify_output(c_out.to(torch.float32), c_ref, rtol=0.1, atol=0.1), (in_dtype, M, N, K)
        assert int((c_alloc[M:] != sentinel).sum().item()) == 0
        print(f"[flyc] {in_dtype} {M}x{N}x{K} Throughput: {us:.1f} us, {2*M*N*K/us/1e6:.2f} TFLOPS")

    for in_dtype in ("fp8", "int8", "fp16", "bf16"):
        for graph in (False, True):
            a8_case(in_dtype, 16, 5120, 8192, 16, 64, 512, graph)
            a8_case(in_dtype, 33, 1024, 2048, 32, 64, 512, graph)
    a8_case("fp8", 5133, 5120, 8320, 64, 256, 128, False)

    def w4_case(M, N, K, tile_m, tile_n, tile_k):
        ptr = lambda t: flyc.from_c_void_p(fx.Uint8, t.contiguous().data_ptr())
        device = torch.device("cuda")
        M32 = (M + 31) // 32 * 32
        a = torch.zeros(M32, K, device=device); a[:M] = torch.randn(M, K, device=device)
        b = torch.randn(N, K, device=device)
        a_q, sa_orig, _ = gemm_common_utils.per_1x32_f4_quant(a); a_q = a_q[:M]
        sa = gemm_common_utils.shuffle_scale_w4(sa_orig.view(torch.uint8), 1, False)
        b_q, sb_orig, _ = gemm_common_utils.per_1x32_f4_quant(b)
        x = gemm_common_utils.mxfp4_to_f32(a_q) * gemm_common_utils.e8m0_to_f32(sa_orig[:M].view(torch.uint8).repeat_interleave(32, dim=1))
        w = gemm_common_utils.mxfp4_to_f32(b_q) * gemm_common_utils.e8m0_to_f32(sb_orig.view(torch.uint8).repeat_interleave(32, dim=1))
        c_ref = torch.mm(x, w.T)
        b_sh = gemm_common_utils.shuffle_weight_w4(b_q.view(torch.uint8), 16, False, False)
        sb = gemm_common_utils.shuffle_scale_w4(sb_orig.view(torch.uint8), 1, False)
        c = torch.zeros(M, N, dtype=torch.bfloat16, device=device)
        launch_gemm(ptr(c), ptr(a_q.view(torch.uint8)), ptr(b_sh), ptr(sa), ptr(sb), M, N, torch.cuda.current_stream(), N, K, tile_m, tile_n,
                    tile_k, "fp4", "bf16", "fp4", 1, -1, -1, -1, -1, -1, -1, 0, 0)
        torch.cuda.synchronize()
        assert verify_output(c.to(torch.float32), c_ref, rtol=0.1, atol=0.1), (M, N, K)
        print(f"[flyc] mxfp4 {M}x{N}x{K} ok")

    w4_case(64, 8192, 8192, 64, 128, 128)
    w4_case(32, 8192, 8192, 32, 128, 256)
    w4_case(133, 1024, 2048, 64, 256, 256)
    DONE = True
''')


def test_reference_style_harness_runs_unchanged():
    import flydsl_amd.compat as compat

    added = compat.install()
    try:
        assert "flydsl.compiler" in added and "tests.utils" in added, added
        scope = {}
        exec(compile(SCRIPT, "<reference-style harness>", "exec"), scope)
        assert scope.get("DONE") is True
    finally:
        for name in added:
            sys.modules.pop(name, None)
