"""GPU parity of the general MX preshuffle GEMM (fp4 / fp6 / fp8 A against fp4 / fp8 W, caller strides, batch over
grid.z) against the CPU oracle, through the reference's launch_gemm call shape.

Mirrors tests/kernels/test_preshuffle_gemm.py test_mfma_a6w4_preshuffle (:472-576) and test_mfma_a8w8_preshuffle
(:582-700) at sizes the oracle finishes in seconds, plus ragged shapes.  Bar: bf16 / fp16 outputs within
|out-ref| <= 1e-2*|ref| + 1e-2*max|ref| of the fp32 dequantised matmul (the reference's own check is
rtol = atol = 0.1); fp32 accumulators within 1e-5*max|ref| for fp4 / fp6 pairs (products and power-of-two scales are
exact, only the summation order differs) and 1e-4*max|ref| when an operand is fp8 (the same bar as the row-scale fp8
GEMM's accumulators: the MFMA sums fp8 products with fewer guard bits)."""

import numpy as np
import pytest
import torch

from helpers import make_mx
from oracle import psg_oracle as O

pytestmark = pytest.mark.gpu

SENTINEL = -8192.0
PAIRS = [("fp6", "fp4"), ("fp8", "fp8"), ("fp8", "fp4"), ("fp4", "fp8"), ("fp6", "fp8"), ("fp4", "fp4")]


def _ref(d):
    return O.run_torch_mx(d["a_q"].numpy(), d["b_q"].numpy(), d["sa"].numpy(), d["sb"].numpy(), d["a_dtype"], d["b_dtype"])


def _acc_atol(d, ref):
    return (1e-4 if "fp8" in (d["a_dtype"], d["b_dtype"]) else 1e-5) * np.abs(ref).max()


def _check(out, ref):
    ok, ratio = O.within_north_star_tolerance(out, ref, 1e-2)
    assert ok, f"outside tolerance (worst ratio {ratio:.3f})"


def _launch(d, M, N, K, *, out_dtype="bf16", tile=(64, 128, 256), guard_rows=0, acc=False, force_path=0, xcd_swizzle=0):
    from kernels.gemm.mxfp4_preshuffle import launch_gemm

    dev = torch.device("cuda")
    tdt = torch.bfloat16 if out_dtype == "bf16" else torch.float16
    c = torch.full((M + guard_rows, N), SENTINEL, dtype=tdt, device=dev)
    accbuf = torch.full((M, N), -7.0, dtype=torch.float32, device=dev) if acc else None
    launch_gemm(c, d["a_q"].to(dev), d["b_shuf"].to(dev), d["sa_shuf"].to(dev), d["sb_shuf"].to(dev), M, N, torch.cuda.current_stream(),
                N, K, *tile, d["a_dtype"], out_dtype, d["b_dtype"], 1, -1, -1, -1, -1, -1, -1, 0, xcd_swizzle,
                _acc=accbuf, _force_path=force_path)
    torch.cuda.synchronize()
    return accbuf.cpu().numpy() if acc else c


@pytest.mark.parametrize("a_dtype,b_dtype", PAIRS)
@pytest.mark.parametrize("M,N,K", [(64, 512, 512), (32, 256, 1024), (1, 128, 256), (133, 288, 768), (300, 1056, 256)])
def test_mx_format_pairs(a_dtype, b_dtype, M, N, K):
    d = make_mx(M, N, K, a_dtype, b_dtype, seed=M + N)
    ref = _ref(d)
    force = 3 if (a_dtype, b_dtype) == ("fp4", "fp4") else 0
    c = _launch(d, M, N, K, guard_rows=40, force_path=force)
    _check(c[:M].float().cpu().numpy(), ref)
    assert (c[M:] == SENTINEL).all()
    acc = _launch(d, M, N, K, acc=True, force_path=force)
    assert np.allclose(acc, ref, rtol=1e-4, atol=_acc_atol(d, ref))


@pytest.mark.parametrize("out_dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("M,N,K,tile", [(64, 2048, 2048, (64, 128, 128)), (32, 2048, 2048, (32, 128, 256))])
def test_mfma_a6w4_preshuffle(out_dtype, M, N, K, tile):
    d = make_mx(M, N, K, "fp6", "fp4", seed=1, w_std=1.0)
    c = _launch(d, M, N, K, out_dtype=out_dtype, tile=tile)
    ref = _ref(d)
    _check(c.float().cpu().numpy(), ref)
    assert O.verify_output(c.float().cpu().numpy(), ref, rtol=0.1, atol=0.1)


@pytest.mark.parametrize("xcd_swizzle", [0, 4])
@pytest.mark.parametrize("out_dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("M,N,K,tile", [(64, 2048, 2048, (64, 128, 128)), (32, 2048, 2048, (32, 128, 256))])
def test_mfma_a8w8_preshuffle(out_dtype, M, N, K, tile, xcd_swizzle):
    d = make_mx(M, N, K, "fp8", "fp8", seed=2, w_std=1.0)
    c = _launch(d, M, N, K, out_dtype=out_dtype, tile=tile, xcd_swizzle=xcd_swizzle)
    ref = _ref(d)
    _check(c.float().cpu().numpy(), ref)
    assert O.verify_output(c.float().cpu().numpy(), ref, rtol=0.1, atol=0.1)


def test_general_kernel_agrees_with_the_fp4_kernels_bit_for_bit():
    # same K order (ascending 128-element steps into one accumulator), so the unsplit fp4 x fp4 results carry the same bits
    M, N, K = 96, 512, 1024
    d = make_mx(M, N, K, "fp4", "fp4", seed=5)
    a = _launch(d, M, N, K, acc=True, force_path=3)
    from kernels.gemm.mxfp4_preshuffle import launch_gemm

    dev = torch.device("cuda")
    accbuf = torch.zeros(M, N, dtype=torch.float32, device=dev)
    launch_gemm(0, d["a_q"].to(dev), d["b_shuf"].to(dev), d["sa_shuf"].to(dev), d["sb_shuf"].to(dev), M, N, torch.cuda.current_stream(),
                N, K, 64, 128, 256, "fp4", "bf16", "fp4", 1, -1, -1, -1, -1, -1, -1, 0, 0, _acc=accbuf, _force_path=1, _tile=(64, 128))
    torch.cuda.synchronize()
    assert np.array_equal(a, accbuf.cpu().numpy())


def test_scale_extremes_select_the_right_scale_byte():
    # scales spanning 30 binades make a wrong byte selection (K half or row half) visible at once
    from flydsl_amd import layout

    M, N, K = 48, 128, 1024
    g = torch.Generator().manual_seed(4)
    for a_dtype, b_dtype in PAIRS[:4]:
        d = make_mx(M, N, K, a_dtype, b_dtype, seed=4, w_std=1.0)
        d["sa"] = torch.randint(110, 140, d["sa"].shape, generator=g, dtype=torch.uint8)
        d["sb"] = torch.randint(110, 140, d["sb"].shape, generator=g, dtype=torch.uint8)
        d["sa_shuf"], d["sb_shuf"] = layout.shuffle_scale_w4(d["sa"], 1, False), layout.shuffle_scale_w4(d["sb"], 1, False)
        x = O.mx_operand_to_f32(d["a_q"].numpy(), a_dtype).astype(np.float64) * np.repeat(O.e8m0_to_f32(d["sa"].numpy()[:M]), 32, axis=1)
        w = O.mx_operand_to_f32(d["b_q"].numpy(), b_dtype).astype(np.float64) * np.repeat(O.e8m0_to_f32(d["sb"].numpy()[:N]), 32, axis=1)
        ref = x @ w.T  # float64: the fp32 matmul's own rounding is visible at this dynamic range
        acc = _launch(d, M, N, K, acc=True, force_path=3)
        assert np.allclose(acc, ref, rtol=1e-4, atol=_acc_atol(d, ref) * 0.1), (a_dtype, b_dtype)


@pytest.mark.parametrize("a_dtype,b_dtype", [("fp8", "fp8"), ("fp6", "fp4")])
def test_split_k_of_the_general_kernel(a_dtype, b_dtype):
    # decode-like shape: few tiles, long K -> K is split over workgroups, partials reduced in a fixed order
    from flydsl_amd import _lib
    from kernels.gemm.mxfp4_preshuffle import launch_gemm

    M, N, K = 32, 512, 8192
    need = _lib.lib().psg_workspace_bytes(M, N, K, 5)
    assert need == 4 * M * N * 4  # four splits
    d = make_mx(M, N, K, a_dtype, b_dtype, seed=9, w_std=1.0)
    ref = _ref(d)
    dev = torch.device("cuda")
    outs = []
    for no_split in (False, True):
        c = torch.full((M + 8, N), SENTINEL, dtype=torch.bfloat16, device=dev)
        for _ in range(2):  # the second call reuses the parked workspace
            launch_gemm(c, d["a_q"].to(dev), d["b_shuf"].to(dev), d["sa_shuf"].to(dev), d["sb_shuf"].to(dev), M, N, torch.cuda.current_stream(),
                        N, K, 32, 128, 256, a_dtype, "bf16", b_dtype, 1, -1, -1, -1, -1, -1, -1, 0, 0, _no_split=no_split)
        torch.cuda.synchronize()
        _check(c[:M].float().cpu().numpy(), ref)
        assert (c[M:] == SENTINEL).all()
        outs.append(c[:M].float().cpu().numpy())
    # split and unsplit sums differ only by fp32 summation order
    assert np.abs(outs[0] - outs[1]).max() <= 2e-2 * np.abs(ref).max()


def test_fp6_padding_bytes_are_not_read():
    M, N, K = 40, 128, 512
    d = make_mx(M, N, K, "fp6", "fp4", seed=6)
    want = _launch(d, M, N, K, acc=True)
    a = d["a_q"].clone().view(M, K // 32, 32)
    a[:, :, 24:] = 0xFF
    d["a_q"] = a.view(M, K).contiguous()
    assert np.array_equal(_launch(d, M, N, K, acc=True), want)


@pytest.mark.parametrize("a_dtype,b_dtype", [("fp4", "fp4"), ("fp6", "fp4"), ("fp8", "fp8")])
def test_strided_batched_default_strides(a_dtype, b_dtype):
    # contiguous [B,M,*] operands, one launch over grid.z (kernels/gemm/mxfp4_preshuffle.py:177-196)
    from kernels.gemm.mxfp4_preshuffle import launch_gemm

    B, M, N, K = 3, 40, 256, 512
    dev = torch.device("cuda")
    ds = [make_mx(M, N, K, a_dtype, b_dtype, seed=20 + b) for b in range(B)]
    cat = lambda k: torch.cat([d[k].reshape(-1) for d in ds]).to(dev)
    c = torch.full((B, M, N), SENTINEL, dtype=torch.bfloat16, device=dev)
    launch_gemm(c, cat("a_q"), cat("b_shuf"), cat("sa_shuf"), cat("sb_shuf"), M, N, torch.cuda.current_stream(), N, K, 64, 128, 256,
                a_dtype, "bf16", b_dtype, B, -1, -1, -1, -1, -1, -1, 0, 0)
    torch.cuda.synchronize()
    for b, d in enumerate(ds):
        _check(c[b].float().cpu().numpy(), _ref(d))


@pytest.mark.parametrize("a_dtype,b_dtype", [("fp4", "fp4"), ("fp8", "fp4"), ("fp6", "fp8")])
def test_strided_batched_mbn_layout(a_dtype, b_dtype):
    # every stride set: A, scale_a and C interleaved [M, B, *] (row stride = B rows, batch stride = one row), the
    # layout the reference's docstring calls mbn (kernels/gemm/mxfp4_preshuffle.py:88-91)
    from kernels.gemm.mxfp4_preshuffle import launch_gemm

    B, M, N, K = 2, 64, 256, 512
    dev = torch.device("cuda")
    ds = [make_mx(M, N, K, a_dtype, b_dtype, seed=30 + b) for b in range(B)]
    a_row = ds[0]["a_q"].shape[1]
    chunk = (K // 256) * 256
    a = torch.stack([d["a_q"] for d in ds], dim=1).contiguous().to(dev)  # [M, B, a_row]
    sa = torch.stack([d["sa_shuf"].reshape(M // 32, chunk) for d in ds], dim=1).contiguous().to(dev)  # [M/32, B, chunk]
    w = torch.cat([d["b_shuf"].reshape(-1) for d in ds]).to(dev)
    sb = torch.cat([d["sb_shuf"].reshape(-1) for d in ds]).to(dev)
    c = torch.full((M, B, N), SENTINEL, dtype=torch.bfloat16, device=dev)
    launch_gemm(c, a, w, sa, sb, M, N, torch.cuda.current_stream(), N, K, 64, 128, 256, a_dtype, "bf16", b_dtype, B,
                B * a_row, a_row, B * chunk // 4, chunk, B * N, N * 2, 0, 0)
    torch.cuda.synchronize()
    for b, d in enumerate(ds):
        _check(c[:, b].float().cpu().numpy(), _ref(d))


def test_c_row_stride_leaves_the_gap_untouched():
    # c_row_stride applies with batch == 1 too (kernels/gemm/mxfp4_preshuffle.py:435-440)
    from kernels.gemm.mxfp4_preshuffle import launch_gemm

    M, N, K, ld = 50, 128, 256, 192
    dev = torch.device("cuda")
    for a_dtype, b_dtype in (("fp4", "fp4"), ("fp8", "fp8")):
        d = make_mx(M, N, K, a_dtype, b_dtype, seed=41)
        c = torch.full((M, ld), SENTINEL, dtype=torch.bfloat16, device=dev)
        launch_gemm(c, d["a_q"].to(dev), d["b_shuf"].to(dev), d["sa_shuf"].to(dev), d["sb_shuf"].to(dev), M, N, torch.cuda.current_stream(),
                    N, K, 64, 128, 256, a_dtype, "bf16", b_dtype, 1, -1, -1, -1, -1, ld, -1, 0, 0)
        torch.cuda.synchronize()
        _check(c[:, :N].float().cpu().numpy(), _ref(d))
        assert (c[:, N:] == SENTINEL).all()


def test_bad_arguments_are_rejected():
    from kernels.gemm.mxfp4_preshuffle import launch_gemm

    base = [0, 0, 0, 0, 0, 32, 128, None, 128, 256, 32, 128, 256, "fp4", "bf16", "fp4", 1, -1, -1, -1, -1, -1, -1, 0]
    for idx, val in ((13, "fp5"), (15, "fp6"), (16, 0), (16, 70000), (14, "fp32"), (12, 64)):
        args = list(base)
        args[idx] = val
        with pytest.raises(ValueError):
            launch_gemm(*args)
    dev = torch.device("cuda")
    d = make_mx(32, 128, 256, "fp8", "fp8", seed=1)
    c = torch.zeros(32, 128, dtype=torch.bfloat16, device=dev)
    with pytest.raises(ValueError, match="needs at least"):  # A given as fp4-sized bytes for an fp8 call
        launch_gemm(c, d["a_q"][:, :128].contiguous().to(dev), d["b_shuf"].to(dev), d["sa_shuf"].to(dev), d["sb_shuf"].to(dev), 32, 128,
                    torch.cuda.current_stream(), 128, 256, 32, 128, 256, "fp8", "bf16", "fp8", 1, -1, -1, -1, -1, -1, -1, 0, 0)
    with pytest.raises(ValueError, match="c_row_stride"):  # a row stride below N comes back from the C ABI
        launch_gemm(c, d["a_q"].to(dev), d["b_shuf"].to(dev), d["sa_shuf"].to(dev), d["sb_shuf"].to(dev), 32, 128,
                    torch.cuda.current_stream(), 128, 256, 32, 128, 256, "fp8", "bf16", "fp8", 1, -1, -1, -1, -1, 64, -1, 0, 0)


# ---- fp8 x fp8 on the tiled mainloop (problems with enough tiles; forced here on small shapes) -------------------------
@pytest.mark.parametrize("tile", [(256, 256), (128, 512), (128, 256), (64, 256), (32, 256), (64, 128), (32, 128)])
@pytest.mark.parametrize("M,N,K", [(64, 512, 512), (133, 288, 768), (300, 1056, 256)])
def test_mxfp8_tiled_shapes(tile, M, N, K):
    from kernels.gemm.mxfp4_preshuffle import launch_gemm

    d = make_mx(M, N, K, "fp8", "fp8", seed=8)
    ref = _ref(d)
    dev = torch.device("cuda")
    ops = [d[k].to(dev) for k in ("a_q", "b_shuf", "sa_shuf", "sb_shuf")]
    for wave_layout in ((0, 8, 2) if tile == (256, 256) else (0,)):
        c = torch.full((M + 40, N), SENTINEL, dtype=torch.bfloat16, device=dev)
        launch_gemm(c, *ops, M, N, torch.cuda.current_stream(), N, K, 64, 128, 256, "fp8", "bf16", "fp8", 1, -1, -1, -1, -1, -1, -1, 0, 0,
                    _force_path=1, _tile=tile, _wave_layout=wave_layout)
        torch.cuda.synchronize()
        _check(c[:M].float().cpu().numpy(), ref)
        assert (c[M:] == SENTINEL).all()
        # same K order as the general kernel (one MFMA per 128-element step, ascending): the same accumulator bits
        acc = torch.zeros(M, N, dtype=torch.float32, device=dev)
        launch_gemm(0, *ops, M, N, torch.cuda.current_stream(), N, K, 64, 128, 256, "fp8", "bf16", "fp8", 1, -1, -1, -1, -1, -1, -1, 0, 0,
                    _acc=acc, _force_path=1, _tile=tile, _wave_layout=wave_layout)
        torch.cuda.synchronize()
        assert np.array_equal(acc.cpu().numpy(), _launch(d, M, N, K, acc=True, force_path=3)), (tile, wave_layout)


def test_mxfp8_large_problem_takes_the_tiled_path_and_scale_extremes_hold():
    from flydsl_amd import layout

    M, N, K = 1024, 8192, 512  # 8 x 32 tiles of 128x256: routed to the tiled mainloop
    d = make_mx(M, N, K, "fp8", "fp8", seed=12, w_std=1.0)
    g = torch.Generator().manual_seed(12)
    d["sa"] = torch.randint(115, 135, d["sa"].shape, generator=g, dtype=torch.uint8)
    d["sb"] = torch.randint(115, 135, d["sb"].shape, generator=g, dtype=torch.uint8)
    d["sa_shuf"], d["sb_shuf"] = layout.shuffle_scale_w4(d["sa"], 1, False), layout.shuffle_scale_w4(d["sb"], 1, False)
    ref = _ref(d)
    for out_dtype in ("bf16", "fp16"):
        if out_dtype == "fp16" and np.abs(ref).max() > 6e4:
            continue
        c = _launch(d, M, N, K, out_dtype=out_dtype)
        _check(c.float().cpu().numpy(), ref)
    assert np.array_equal(_launch(d, M, N, K, acc=True), _launch(d, M, N, K, acc=True, force_path=3))


@pytest.mark.parametrize("a_dtype,b_dtype", [("fp6", "fp4"), ("fp8", "fp4"), ("fp4", "fp8")])
def test_general_kernel_large_tile(a_dtype, b_dtype):
    # enough 128x256 tiles to give every CU one: the general kernel's large tile, ragged in M and N
    M, N, K = 1000, 8224, 256
    d = make_mx(M, N, K, a_dtype, b_dtype, seed=14)
    ref = _ref(d)
    c = _launch(d, M, N, K, guard_rows=8)
    _check(c[:M].float().cpu().numpy(), ref)
    assert (c[M:] == SENTINEL).all()
    # the small tile through the same kernel (forced by a batch of one narrow problem) gives the same accumulators
    acc = _launch(d, M, N, K, acc=True)
    assert np.allclose(acc, ref, rtol=1e-4, atol=_acc_atol(d, ref))
