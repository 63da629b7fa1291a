"""GPU parity of the MXFP4 preshuffle GEMM against the CPU oracle, through the C ABI.

Bar: bf16 outputs within |out-ref| <= 1e-2*|ref| + 1e-2*max|ref| of the fp32 dequantised matmul;
fp32 accumulators within 1e-5 relative of the float64 block-scaled sum (the products and the
power-of-two scales are exact, only the summation order differs)."""

import numpy as np
import pytest
import torch

from helpers import make_mxfp4
from oracle import c_oracle as C
from oracle import psg_oracle as O

pytestmark = pytest.mark.gpu

SENTINEL = -8192.0


def _ptr(t):
    import flydsl_amd.compiler as flyc
    import flydsl_amd.expr as fx

    return flyc.from_c_void_p(fx.Uint8, t.contiguous().data_ptr())


def _run(d, M, N, K, *, force_path=0, tile=None, guard_rows=0, acc=False, out_dtype="bf16", tile_args=(32, 128, 256), wave_layout=0):
    from kernels.gemm.mxfp4_preshuffle import launch_gemm

    dev = torch.device("cuda")
    a, b = d["a_q"].to(dev), d["b_shuf"].to(dev)
    sa, sb = d["sa_shuf"].to(dev), d["sb_shuf"].to(dev)
    tdt = torch.bfloat16 if out_dtype == "bf16" else torch.float16
    c_alloc = torch.full((M + guard_rows, N), SENTINEL, dtype=tdt, device=dev)
    accbuf = torch.full((M, N), -7.0, dtype=torch.float32, device=dev) if acc else None
    tm, tn, tk = tile_args
    launch_gemm(_ptr(c_alloc), _ptr(a), _ptr(b), _ptr(sa), _ptr(sb), M, N, torch.cuda.current_stream(), N, K, tm, tn, tk,
                "fp4", out_dtype, "fp4", 1, -1, -1, -1, -1, -1, -1, 0, 0, _force_path=force_path, _tile=tile,
                _acc=accbuf, _wave_layout=wave_layout)
    torch.cuda.synchronize()
    return accbuf.cpu().numpy() if acc else c_alloc


def _check(out, ref):
    ok, ratio = O.within_north_star_tolerance(out, ref, 1e-2)
    assert ok, f"outside tolerance (worst ratio {ratio:.3f})"


@pytest.mark.parametrize("M", [1, 16, 31, 32, 33, 47, 48, 49, 64])
@pytest.mark.parametrize("N,K", [(256, 512), (7168, 2048)])
def test_mxfp4_small_m(M, N, K):
    d = make_mxfp4(M, N, K, seed=M)
    ref = O.run_torch_w4(d["a_q"].numpy(), d["b_q"].numpy(), d["sa"].numpy(), d["sb"].numpy())
    want = C.mxfp4(d["a_q"].numpy(), d["b_shuf"].numpy(), d["sa_shuf"].numpy(), d["sb_shuf"].numpy(), M, N, K)["out_f32"]
    for force_path in (2, 1):
        c = _run(d, M, N, K, force_path=force_path, guard_rows=33)
        _check(c[:M].float().cpu().numpy(), ref)
        assert (c[M:] == SENTINEL).all()
        acc = _run(d, M, N, K, force_path=force_path, acc=True)
        assert np.allclose(acc, want, rtol=1e-5, atol=1e-5 * np.abs(want).max())


@pytest.mark.parametrize("tile", [(256, 256), (128, 256), (64, 256), (32, 256), (64, 128), (32, 128)])
@pytest.mark.parametrize("M,N,K", [(64, 512, 512), (133, 288, 768), (300, 1056, 256)])
def test_mxfp4_tiled_shapes(tile, M, N, K):
    d = make_mxfp4(M, N, K, seed=7)
    ref = O.run_torch_w4(d["a_q"].numpy(), d["b_q"].numpy(), d["sa"].numpy(), d["sb"].numpy())
    c = _run(d, M, N, K, force_path=1, tile=tile, guard_rows=64)
    _check(c[:M].float().cpu().numpy(), ref)
    assert (c[M:] == SENTINEL).all()
    want = C.mxfp4(d["a_q"].numpy(), d["b_shuf"].numpy(), d["sa_shuf"].numpy(), d["sb_shuf"].numpy(), M, N, K)["out_f32"]
    acc = _run(d, M, N, K, force_path=1, tile=tile, acc=True)
    assert np.allclose(acc, want, rtol=1e-5, atol=1e-5 * np.abs(want).max())


# ---- the 256x256 tile of eight wavefronts (A and the scale dwords by LDS DMA), which the planner only takes for problems that
# fill the GPU: forced here on ragged shapes (rows and scale chunks past M, columns past N in the last tile, one to nine K steps)
@pytest.mark.parametrize("M,N,K", [(64, 512, 512), (133, 288, 768), (300, 1056, 256), (257, 32, 1280), (700, 544, 2304)])
def test_mxfp4_eight_wavefront_tile_ragged(M, N, K):
    d = make_mxfp4(M, N, K, seed=M + K)
    ref = O.run_torch_w4(d["a_q"].numpy(), d["b_q"].numpy(), d["sa"].numpy(), d["sb"].numpy())
    want = C.mxfp4(d["a_q"].numpy(), d["b_shuf"].numpy(), d["sa_shuf"].numpy(), d["sb_shuf"].numpy(), M, N, K)["out_f32"]
    for _ in range(2):
        c = _run(d, M, N, K, force_path=1, tile=(256, 256), guard_rows=64, wave_layout=8)
        _check(c[:M].float().cpu().numpy(), ref)
        assert (c[M:] == SENTINEL).all()
        acc = _run(d, M, N, K, force_path=1, tile=(256, 256), acc=True, wave_layout=8)
        assert np.allclose(acc, want, rtol=1e-5, atol=1e-5 * np.abs(want).max())
    # the same K order as the four-wavefront build of the tile: the same accumulator bits
    assert np.array_equal(acc, _run(d, M, N, K, force_path=1, tile=(256, 256), acc=True, wave_layout=0))


def test_mxfp4_config5_prefill():
    M, N, K = 4096, 7168, 2048
    d = make_mxfp4(M, N, K, seed=0)
    x = torch.from_numpy(O.mxfp4_to_f32(d["a_q"].numpy()) * O.e8m0_to_f32(np.repeat(d["sa"].numpy()[:M], 32, axis=1)))
    w = torch.from_numpy(O.mxfp4_to_f32(d["b_q"].numpy()) * O.e8m0_to_f32(np.repeat(d["sb"].numpy()[:N], 32, axis=1)))
    ref = torch.mm(x, w.T).numpy()
    c = _run(d, M, N, K, tile_args=(64, 256, 256))
    _check(c[:M].float().cpu().numpy(), ref)


def test_mxfp4_fp16_out_and_scale_extremes():
    # scales spanning many binades: exercises the opsel byte selection harder than N(0,1) data does
    M, N, K = 48, 128, 1024
    g = torch.Generator().manual_seed(4)
    d = make_mxfp4(M, N, K, seed=4, w_std=1.0)
    sa = torch.randint(110, 140, d["sa"].shape, generator=g, dtype=torch.uint8)
    sb = torch.randint(110, 140, d["sb"].shape, generator=g, dtype=torch.uint8)
    from flydsl_amd import layout

    d["sa"], d["sb"] = sa, sb
    d["sa_shuf"], d["sb_shuf"] = layout.shuffle_scale_w4(sa, 1, False), layout.shuffle_scale_w4(sb, 1, False)
    want = C.mxfp4(d["a_q"].numpy(), d["b_shuf"].numpy(), d["sa_shuf"].numpy(), d["sb_shuf"].numpy(), M, N, K)["out_f32"]
    for fp in (1,):
        acc = _run(d, M, N, K, force_path=fp, acc=True)
        assert np.allclose(acc, want, rtol=1e-5, atol=1e-6 * np.abs(want).max())
    acc = _run(d, 32, N, K, force_path=2, acc=True)
    assert np.allclose(acc, want[:32], rtol=1e-5, atol=1e-6 * np.abs(want).max())


@pytest.mark.parametrize("K", [256, 512])
def test_mxfp4_short_k_every_tile(K):
    # one or two mainloop steps: the accumulators are read right after the last MFMA
    M, N = 256, 512
    d = make_mxfp4(M, N, K, seed=K)
    want = C.mxfp4(d["a_q"].numpy(), d["b_shuf"].numpy(), d["sa_shuf"].numpy(), d["sb_shuf"].numpy(), M, N, K)["out_f32"]
    for tile in [(256, 256), (128, 256), (64, 256), (32, 256), (64, 128), (32, 128)]:
        for _ in range(3):
            acc = _run(d, M, N, K, force_path=1, tile=tile, acc=True)
            assert np.allclose(acc, want, rtol=1e-5, atol=1e-5 * np.abs(want).max()), f"tile {tile}"


def test_mxfp4_strided_batched_default_strides():
    # batch > 1 with the reference's default strides: contiguous [B,M,*] operands, one result slab per batch
    from kernels.gemm.mxfp4_preshuffle import launch_gemm

    B, M, N, K = 3, 40, 256, 512
    dev = torch.device("cuda")
    ds = [make_mxfp4(M, N, K, seed=20 + b) for b in range(B)]
    cat = lambda k: torch.cat([d[k].reshape(-1) for d in ds]).to(dev)
    a, w, sa, sb = cat("a_q"), cat("b_shuf"), cat("sa_shuf"), cat("sb_shuf")
    c = torch.zeros(B, M, N, dtype=torch.bfloat16, device=dev)
    launch_gemm(c, a, w, sa, sb, M, N, torch.cuda.current_stream(), N, K, 64, 128, 256, "fp4", "bf16", "fp4", B, -1, -1, -1, -1, -1, -1, 0, 0)
    torch.cuda.synchronize()
    for b, d in enumerate(ds):
        ref = O.run_torch_w4(d["a_q"].numpy(), d["b_q"].numpy(), d["sa"].numpy(), d["sb"].numpy())
        _check(c[b].float().cpu().numpy(), ref)
