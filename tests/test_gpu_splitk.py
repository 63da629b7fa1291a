"""GPU parity of the split-K variant of the tiled path (few tiles, long K): int32 partial sums are exact, so int8
outputs stay bit-identical to the oracle for every split count; fp8 / bf16 / MXFP4 stay inside the tolerance.  Also
checks the automatic plan (workspace supplied by the launcher) and that a missing workspace falls back to the
unsplit kernel with the same result."""

import ctypes

import numpy as np
import pytest
import torch

from helpers import bf16_bits, make_a8w8, make_a16w16, make_mxfp4, np_bytes, np_u16
from oracle import c_oracle as C
from oracle import psg_oracle as O

pytestmark = pytest.mark.gpu


def _fn(kind, N, K):
    from kernels.gemm.preshuffle_gemm import compile_preshuffle_gemm

    return compile_preshuffle_gemm(N=N, K=K, tile_m=128, tile_n=256, tile_k=64 if kind in ("int8", "fp8") else 32, in_dtype=kind)


@pytest.mark.parametrize("splits", [2, 3, 4, 8, 16])
@pytest.mark.parametrize("tile", [(64, 64), (128, 128), (64, 256), (256, 256)])
def test_int8_splitk_bit_exact(splits, tile):
    M, N, K = 100, 528, 2368  # ragged M, N not a tile multiple, K % 128 == 64, uneven steps per split
    d = make_a8w8(M, N, K, "int8", seed=splits)
    dev = torch.device("cuda")
    fn = _fn("int8", N, K)
    c = torch.full((M + 8, N), -8192.0, dtype=torch.bfloat16, device=dev)
    fn.launch_forced(c[:M], d["a_q"].to(dev), d["b_shuf"].to(dev), d["sa"].to(dev), d["sb"].to(dev),
                     torch.empty(0, dtype=torch.bfloat16, device=dev), M, N, None, force_path=1, tile=tile, splits=splits)
    torch.cuda.synchronize()
    ref = C.a8w8(np_bytes(d["a_q"]), np_bytes(d["b_shuf"]), d["sa"].numpy(), d["sb"].numpy(), "int8")
    assert np.array_equal(bf16_bits(c[:M]), ref["c_bf16_bits"])
    assert (c[M:] == -8192.0).all()


@pytest.mark.parametrize("kind", ["fp8", "bf16"])
@pytest.mark.parametrize("epilogue", ["none", "bias_gelu"])
def test_float_splitk(kind, epilogue):
    from kernels.gemm.preshuffle_gemm import compile_preshuffle_gemm

    M, N, K = 72, 384, 4096
    dev = torch.device("cuda")
    g = torch.Generator().manual_seed(3)
    bias = (torch.randn(N, generator=g) * 0.3).to(torch.bfloat16)
    if kind == "fp8":
        d = make_a8w8(M, N, K, kind, seed=1, w_std=0.05)
        sa, sb = d["sa"].to(dev), d["sb"].to(dev)
        ref = O.run_torch(np_bytes(d["a_q"]), np_bytes(d["b_q"]), d["sa"].numpy(), d["sb"].numpy(), kind)
    else:
        d = make_a16w16(M, N, K, kind, seed=1, w_std=0.05)
        sa = sb = torch.empty(0, dtype=torch.float32, device=dev)
        ref = O.run_torch(np_u16(d["a_q"]), np_u16(d["b_q"]), None, None, kind)
    if epilogue != "none":
        ref = O.apply_bias_act(ref, bias.float().numpy(), "gelu")
    fn = compile_preshuffle_gemm(N=N, K=K, tile_m=128, tile_n=256, tile_k=64, in_dtype=kind, epilogue=epilogue)
    for splits in (1, 4):
        c = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
        fn.launch_forced(c, d["a_q"].to(dev), d["b_shuf"].to(dev), sa, sb, bias.to(dev), M, N, None, force_path=1,
                         tile=(64, 64), splits=splits)
        torch.cuda.synchronize()
        ok, ratio = O.within_north_star_tolerance(c.float().cpu().numpy(), ref)
        assert ok, (splits, ratio)


def test_automatic_plan_uses_and_survives_without_workspace():
    from flydsl_amd import _lib

    M, N, K = 80, 2048, 8192  # few tiles, long K: the planner splits
    handle = _lib.lib()
    need = handle.psg_workspace_bytes(M, N, K, 0)
    assert need > 0 and need % (M * N * 4) == 0
    assert handle.psg_workspace_bytes(16, N, K, 0) == 0  # streaming kernel
    assert handle.psg_workspace_bytes(8192, 4096, 4096, 1) == 0  # enough tiles
    d = make_a8w8(M, N, K, "int8", seed=5)
    dev = torch.device("cuda")
    fn = _fn("int8", N, K)
    ref = C.a8w8(np_bytes(d["a_q"]), np_bytes(d["b_shuf"]), d["sa"].numpy(), d["sb"].numpy(), "int8")["c_bf16_bits"]
    t = {k: d[k].to(dev) for k in ("a_q", "b_shuf", "sa", "sb")}
    bias = torch.empty(0, dtype=torch.bfloat16, device=dev)
    c = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
    fn(c, t["a_q"], t["b_shuf"], t["sa"], t["sb"], bias, M, N, None)  # launcher supplies the workspace
    torch.cuda.synchronize()
    assert np.array_equal(bf16_bits(c), ref)
    # same call straight through the C ABI with no workspace: runs unsplit, same bits
    args = fn._fill(c, t["a_q"], t["b_shuf"], t["sa"], t["sb"], bias, M, N)
    args.workspace, args.workspace_bytes = None, 0
    c.zero_()
    assert handle.psg_gemm_a8w8(ctypes.byref(args), _lib.stream_handle(None)) == 0
    torch.cuda.synchronize()
    assert np.array_equal(bf16_bits(c), ref)
    # graph replay of the split path (two kernels, shared workspace) matches eager
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s):
        fn(c, t["a_q"], t["b_shuf"], t["sa"], t["sb"], bias, M, N, torch.cuda.current_stream())
    for _ in range(3):
        c.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert np.array_equal(bf16_bits(c), ref)


def test_mxfp4_splitk():
    from kernels.gemm.mxfp4_preshuffle import launch_gemm

    M, N, K = 64, 512, 4096
    d = make_mxfp4(M, N, K, seed=2)
    dev = torch.device("cuda")
    t = {k: d[k].to(dev) for k in ("a_q", "b_shuf", "sa_shuf", "sb_shuf")}
    ref = O.run_torch_w4(d["a_q"].numpy(), d["b_q"].numpy(), d["sa"].numpy(), d["sb"].numpy())
    for splits in (1, 2, 4):
        c = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
        launch_gemm(c, t["a_q"], t["b_shuf"], t["sa_shuf"], t["sb_shuf"], M, N, None, N, K, 64, 128, 256, "fp4", "bf16", "fp4", 1,
                    -1, -1, -1, -1, -1, -1, 0, 0, _force_path=1, _tile=(64, 128), _splits=splits)
        torch.cuda.synchronize()
        ok, ratio = O.within_north_star_tolerance(c.float().cpu().numpy(), ref)
        assert ok, (splits, ratio)


def test_two_streams_take_the_split_plan_without_sharing_a_workspace():
    """Two launchers on two streams, both on the split-K plan, enqueued back to back so that they may overlap: each
    stream has its own workspace, so both int8 results stay bit-exact."""
    from flydsl_amd import _lib

    M, N, K = 80, 2048, 8192
    assert _lib.lib().psg_workspace_bytes(M, N, K, 0) > 0
    dev = torch.device("cuda")
    bias = torch.empty(0, dtype=torch.bfloat16, device=dev)
    work = []
    for seed in (11, 12):
        d = make_a8w8(M, N, K, "int8", seed=seed)
        t = {k: d[k].to(dev) for k in ("a_q", "b_shuf", "sa", "sb")}
        ref = C.a8w8(np_bytes(d["a_q"]), np_bytes(d["b_shuf"]), d["sa"].numpy(), d["sb"].numpy(), "int8")["c_bf16_bits"]
        work.append((t, ref, torch.zeros(M, N, dtype=torch.bfloat16, device=dev), torch.cuda.Stream(), _fn("int8", N, K)))
    torch.cuda.synchronize()
    for rep in range(4):
        for t, ref, c, s, fn in work:
            fn(c, t["a_q"], t["b_shuf"], t["sa"], t["sb"], bias, M, N, s)
    torch.cuda.synchronize()
    bufs = [_lib._pool._live[(w[4]._ws_owner, torch.cuda.current_device(), _lib.stream_handle(w[3]))] for w in work]
    assert bufs[0] is not bufs[1]
    # one launcher on two streams: separate buffers as well
    t, ref, c, s, fn = work[0]
    c2 = torch.zeros_like(c)
    s2 = torch.cuda.Stream()
    fn(c, t["a_q"], t["b_shuf"], t["sa"], t["sb"], bias, M, N, s)
    fn(c2, t["a_q"], t["b_shuf"], t["sa"], t["sb"], bias, M, N, s2)
    torch.cuda.synchronize()
    assert _lib._pool._live[(fn._ws_owner, torch.cuda.current_device(), _lib.stream_handle(s2))] is not bufs[0]
    assert np.array_equal(bf16_bits(c2), ref)
    for t, ref, c, s, fn in work:
        assert np.array_equal(bf16_bits(c), ref)


def test_workspace_growth_during_capture_is_refused():
    M, N, K = 128, 1024, 8192
    d = make_a8w8(M, N, K, "int8", seed=3)
    dev = torch.device("cuda")
    t = {k: d[k].to(dev) for k in ("a_q", "b_shuf", "sa", "sb")}
    c = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
    bias = torch.empty(0, dtype=torch.bfloat16, device=dev)
    fn = _fn("int8", N, K)  # a launcher that has no workspace yet
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    g = torch.cuda.CUDAGraph()
    with pytest.raises(RuntimeError, match="graph capture"):
        with torch.cuda.graph(g, stream=s):
            fn(c, t["a_q"], t["b_shuf"], t["sa"], t["sb"], bias, M, N, torch.cuda.current_stream())
    torch.cuda.synchronize()


@pytest.mark.parametrize("M,N,K", [(65, 2048, 4096), (128, 4096, 4096), (300, 1040, 2048), (512, 4096, 1024), (200, 4112, 5120), (384, 5120, 5120),
                                   (512, 5120, 5120), (96, 4096, 14336), (33, 28672, 4096)])
def test_mid_m_plans_stay_bit_exact_for_int8(M, N, K):
    """The automatic plan between the streaming kernel and GPU-filling problems: 64x64 tiles on short rows (with and without two K
    splits), 128x128 tiles with up to eight splits on long rows, and the shapes on either side of each rule's border.  int8 sums are
    exact, so whatever the plan the bf16 output equals the C oracle bit for bit; guard rows behind M stay untouched."""
    d = make_a8w8(M, N, K, "int8", seed=M + N)
    dev = torch.device("cuda")
    fn = _fn("int8", N, K)
    ref = C.a8w8(np_bytes(d["a_q"]), np_bytes(d["b_shuf"]), d["sa"].numpy(), d["sb"].numpy(), "int8")["c_bf16_bits"]
    t = {k: d[k].to(dev) for k in ("a_q", "b_shuf", "sa", "sb")}
    bias = torch.empty(0, dtype=torch.bfloat16, device=dev)
    c = torch.full((M + 3, N), 7.0, dtype=torch.bfloat16, device=dev)
    fn(c, t["a_q"], t["b_shuf"], t["sa"], t["sb"], bias, M, N, None)
    torch.cuda.synchronize()
    assert np.array_equal(bf16_bits(c[:M]), ref)
    assert torch.all(c[M:] == 7.0)
