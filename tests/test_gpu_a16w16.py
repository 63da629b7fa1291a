"""GPU parity of the fp16 / bf16 preshuffle GEMM (same entry point, no scales) and of its fused epilogues,
against the fp32 matmul of the same 16-bit operands.  Bar: |out-ref| <= 1e-2*|ref| + 1e-2*max|ref|."""

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from helpers import make_a16w16, np_u16
from oracle import psg_oracle as O

pytestmark = pytest.mark.gpu

SENTINEL = -8192.0


def _launch(d, M, N, K, *, force_path=0, tile=None, epilogue="none", bias=None, guard_rows=0, out_dtype="bf16", acc=False, wave_layout=0):
    from kernels.gemm.preshuffle_gemm import compile_preshuffle_gemm

    dev = torch.device("cuda")
    fn = compile_preshuffle_gemm(N=N, K=K, tile_m=128, tile_n=256, tile_k=32, in_dtype=d["kind"], out_dtype=out_dtype,
                                 epilogue=epilogue)
    tdt = torch.bfloat16 if out_dtype == "bf16" else torch.float16
    a, b = d["a_q"].to(dev), d["b_shuf"].to(dev)
    empty = torch.empty(0, dtype=torch.float32, device=dev)
    if acc:
        out = torch.full((M, N), -7.0, dtype=torch.float32, device=dev)
        fn.accumulators(out, a, b, M, N, torch.cuda.current_stream(), force_path=force_path, tile=tile, wave_layout=wave_layout)
        torch.cuda.synchronize()
        return out.cpu().numpy()
    c_alloc = torch.full((M + guard_rows, N), SENTINEL, dtype=tdt, device=dev)
    bias_t = bias.to(dev) if bias is not None else torch.empty(0, dtype=tdt, device=dev)
    fn.launch_forced(c_alloc[:M].view(-1), a.view(-1), b.view(-1), empty, empty, bias_t, M, N, torch.cuda.current_stream(),
                     force_path=force_path, tile=tile, wave_layout=wave_layout)
    torch.cuda.synchronize()
    return c_alloc


def _ref(d):
    return O.run_torch(np_u16(d["a_q"]), np_u16(d["b_q"]), None, None, d["kind"])


def _check(out, ref):
    ok, ratio = O.within_north_star_tolerance(out, ref, 1e-2)
    assert ok, f"outside tolerance (worst ratio {ratio:.3f})"


@pytest.mark.parametrize("kind", ["bf16", "fp16"])
@pytest.mark.parametrize("M,N,K", [(1, 512, 256), (16, 1024, 2048), (33, 1024, 2048), (200, 272, 96), (512, 1024, 2048)])
def test_a16w16_shapes(kind, M, N, K):
    d = make_a16w16(M, N, K, kind, seed=M, w_std=0.05)
    ref = _ref(d)
    paths = [(1, t) for t in ((256, 256), (128, 256), (64, 256), (32, 256), (128, 128), (64, 64))]
    if M <= 64:
        paths.append((2, None))
    for force_path, tile in paths:
        c = _launch(d, M, N, K, force_path=force_path, tile=tile, guard_rows=40)
        _check(c[:M].float().cpu().numpy(), ref)
        assert (c[M:] == SENTINEL).all(), f"path {force_path} tile {tile}: rows past M were written"
    acc = _launch(d, M, N, K, acc=True)
    assert np.allclose(acc, ref, rtol=1e-4, atol=1e-4 * np.abs(ref).max())


# ---- the 256x256 tile of eight wavefronts (A by LDS DMA; what the planner takes for problems that fill the GPU), forced on
# ragged shapes: rows past M, columns past N in the last tile, K from half a step to 33 and a half steps
@pytest.mark.parametrize("kind", ["bf16", "fp16"])
@pytest.mark.parametrize("M,N,K", [(200, 272, 96), (257, 48, 32), (700, 528, 160), (300, 992, 2144)])
def test_a16w16_eight_wavefront_tile_ragged(kind, M, N, K):
    d = make_a16w16(M, N, K, kind, seed=M + K, w_std=0.05)
    ref = _ref(d)
    for _ in range(2):
        c = _launch(d, M, N, K, force_path=1, tile=(256, 256), guard_rows=40, wave_layout=8)
        _check(c[:M].float().cpu().numpy(), ref)
        assert (c[M:] == SENTINEL).all()
    acc = _launch(d, M, N, K, force_path=1, tile=(256, 256), acc=True, wave_layout=8)
    assert np.allclose(acc, ref, rtol=1e-4, atol=1e-4 * np.abs(ref).max())
    # same K order as the four-wavefront build of the tile: the same accumulator bits
    assert np.array_equal(acc, _launch(d, M, N, K, force_path=1, tile=(256, 256), acc=True))


@pytest.mark.parametrize("epilogue", ["bias", "bias_relu", "bias_silu", "bias_gelu"])
def test_fused_epilogue_reference_shape(epilogue):
    # the reference's own epilogue test: bf16, M=16, N=5120, K=8192, seed 0, atol 2.0 / rtol 0.05
    M, N, K = 16, 5120, 8192
    g = torch.Generator().manual_seed(0)
    a = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = torch.randn(N, K, generator=g).to(torch.bfloat16)
    bias = torch.randn(N, generator=g).to(torch.bfloat16)
    from flydsl_amd import layout

    d = {"kind": "bf16", "a_q": a, "b_q": w, "b_shuf": layout.shuffle_weight(w.contiguous())}
    ref = a.float() @ w.float().T + bias.float()
    ref = {"bias": ref, "bias_relu": F.relu(ref), "bias_silu": F.silu(ref), "bias_gelu": F.gelu(ref, approximate="tanh")}[epilogue]
    ref = ref.to(torch.bfloat16)
    for force_path in (0, 1):
        c = _launch(d, M, N, K, force_path=force_path, epilogue=epilogue, bias=bias)[:M].cpu()
        assert not torch.isnan(c).any() and not torch.isinf(c).any()
        assert torch.allclose(c, ref, atol=2.0, rtol=0.05)
        # and the build's own tighter bar against the fp32 result
        act = {"bias": "none", "bias_relu": "relu", "bias_silu": "silu", "bias_gelu": "gelu"}[epilogue]
        want = O.apply_bias_act(O.run_torch(np_u16(a), np_u16(w), None, None, "bf16"), bias.float().numpy(), act)
        _check(c.float().numpy(), want)


def test_example_shape_fp16():
    # the tutorial's problem (examples/04-preshuffle_gemm.py): fp16, tolerance 1e-3 + 1e-3*|ref| on its own data
    M = N = K = 1024
    d = make_a16w16(M, N, K, "fp16", seed=5, w_std=0.02)
    ref = _ref(d)
    c = _launch(d, M, N, K, out_dtype="fp16")
    _check(c[:M].float().cpu().numpy(), ref)


def test_usage_example_runs_and_is_correct():
    from flydsl_amd.examples import preshuffle_gemm_fp16

    assert preshuffle_gemm_fp16.main(M=1024, N=2048, K=4096, iters=3)
