"""The row-scale fp8 GEMM call shapes (reference: compile_fp8_gemm_8w kernels/gemm/fp8_gemm_8wave.py:148,
compile_fp8_gemm_4w kernels/gemm/fp8_gemm_4wave.py:162) on the native kernels, with W plain row-major and preshuffled,
mirroring the reference's tests/kernels/test_fp8_gemm_rowscale.py: uniform [0,1) inputs, per-row fp8 quantisation,
``flyc.compile`` then launch, oracle = fp32 dequantised matmul.  Tolerance: 1e-2*|ref| + 1e-2*max|ref|."""

import numpy as np
import pytest
import torch

from helpers import np_bytes
from oracle import psg_oracle as O

pytestmark = pytest.mark.gpu


def _case(M, N, K, use_8w, tile_m, tile_n, b_preshuffled, seed=0):
    import flydsl_amd.compiler as flyc
    from flydsl_amd.quant import pertoken_quant
    from kernels.gemm.fp8_gemm_4wave import compile_fp8_gemm_4w
    from kernels.gemm.fp8_gemm_8wave import compile_fp8_gemm_8w
    from kernels.gemm.fp8_gemm_utils import preshuffle_b

    g = torch.Generator().manual_seed(seed)
    a_q, sa = pertoken_quant(torch.rand(M, K, generator=g), quant_dtype=torch.float8_e4m3fn)
    b_q, sb = pertoken_quant(torch.rand(N, K, generator=g), quant_dtype=torch.float8_e4m3fn)
    sa, sb = sa.squeeze().contiguous(), sb.squeeze().contiguous()
    ref = O.run_torch(np_bytes(a_q), np_bytes(b_q), sa.numpy(), sb.numpy(), "fp8")
    dev = torch.device("cuda")
    b_kernel = preshuffle_b(b_q.view(torch.uint8)) if b_preshuffled else b_q
    if use_8w:
        fn = compile_fp8_gemm_8w(K=K, BLOCK_M=tile_m, BLOCK_N=tile_n, b_preshuffled=b_preshuffled)
    else:
        fn = compile_fp8_gemm_4w(K=K, BLOCK_M=tile_m, BLOCK_N=tile_n, b_preshuffled=b_preshuffled)
    c = torch.full((M + 8, N), -8192.0, dtype=torch.bfloat16, device=dev)
    args = (a_q.view(torch.int8).to(dev).view(-1), b_kernel.view(torch.int8).to(dev).view(-1), c[:M].view(-1), sa.to(dev), sb.to(dev),
            M, N, torch.cuda.current_stream())
    compiled = flyc.compile(fn, *args)
    c[:M].zero_()
    compiled(*args)
    torch.cuda.synchronize()
    ok, ratio = O.within_north_star_tolerance(c[:M].float().cpu().numpy(), ref, 1e-2)
    assert ok, f"outside tolerance (worst ratio {ratio:.3f})"
    assert (c[M:] == -8192.0).all()


@pytest.mark.parametrize("b_preshuffled", [False, True], ids=["rowmajor", "preshuffle_b"])
@pytest.mark.parametrize("M,N,K,tile_m,tile_n", [(512, 2112, 7168, 64, 64), (1000, 1040, 1152, 256, 256), (16, 2112, 7168, 64, 64),
                                                 (31, 272, 640, 64, 64)])
def test_fp8_gemm_4wave(M, N, K, tile_m, tile_n, b_preshuffled):
    _case(M, N, K, False, tile_m, tile_n, b_preshuffled)


@pytest.mark.parametrize("b_preshuffled", [False, True], ids=["rowmajor", "preshuffle_b"])
@pytest.mark.parametrize("M,N,K,tile_m,tile_n", [(512, 2112, 7168, 128, 256), (5120, 5120, 8320, 256, 256)])
def test_fp8_gemm_8wave(M, N, K, tile_m, tile_n, b_preshuffled):
    _case(M, N, K, True, tile_m, tile_n, b_preshuffled, seed=1)


def test_rowmajor_and_preshuffled_weights_give_the_same_bits_for_int8():
    """The row-major W path through the C ABI (b_layout = 1) against the preshuffled one: same accumulators, so the
    int8 outputs must be bit-identical, in both regimes and with ragged shapes."""
    import ctypes

    from flydsl_amd import _lib
    from flydsl_amd.synthetic import make_a8w8

    handle = _lib.lib()
    dev = torch.device("cuda")
    for (M, N, K) in [(16, 1040, 1088), (32, 272, 192), (300, 528, 2368), (1000, 2000, 128)]:
        d = make_a8w8(M, N, K, "int8", seed=M)
        t = {k: d[k].to(dev) for k in ("a_q", "b_q", "b_shuf", "sa", "sb")}
        outs = []
        for layout, b in ((0, t["b_shuf"]), (1, t["b_q"])):
            c = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
            a = _lib.A8W8Args()
            a.c, a.a, a.b = c.data_ptr(), t["a_q"].data_ptr(), b.data_ptr()
            a.scale_a, a.scale_b = t["sa"].data_ptr(), t["sb"].data_ptr()
            a.M, a.N, a.K, a.in_dtype, a.b_layout = M, N, K, 0, layout
            assert handle.psg_gemm_a8w8(ctypes.byref(a), _lib.stream_handle(None)) == 0, handle.psg_last_error()
            torch.cuda.synchronize()
            outs.append(c.view(torch.int16).cpu().numpy())
        assert np.array_equal(outs[0], outs[1]), (M, N, K)
