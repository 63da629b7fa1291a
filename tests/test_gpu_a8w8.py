"""GPU parity of the 8-bit preshuffle GEMM against the CPU oracle, through the C ABI.

Bars: int32 accumulators bit-exact; int8 bf16 outputs bit-exact against the C oracle (same
arithmetic order in the epilogue); fp8 bf16 outputs within |out-ref| <= 1e-2*|ref| + 1e-2*max|ref|
of the fp32 dequantised matmul."""

import numpy as np
import pytest
import torch

from helpers import bf16_bits, make_a8w8, np_bytes
from oracle import c_oracle as C
from oracle import psg_oracle as O

pytestmark = pytest.mark.gpu

SENTINEL = -8192.0


def _launch(d, M, N, K, *, force_path=0, tile=None, epilogue="none", bias=None, guard_rows=0, out_dtype="bf16", wave_layout=0):
    from kernels.gemm.preshuffle_gemm import compile_preshuffle_gemm

    dev = torch.device("cuda")
    fn = compile_preshuffle_gemm(N=N, K=K, tile_m=128, tile_n=256, tile_k=64, in_dtype=d["kind"], out_dtype=out_dtype,
                                 epilogue=epilogue)
    tdt = torch.bfloat16 if out_dtype == "bf16" else torch.float16
    c_alloc = torch.full((M + guard_rows, N), SENTINEL, dtype=tdt, device=dev)
    a = d["a_q"].to(dev)
    if guard_rows:
        # poison the rows behind A: they must never be read into the result
        a_alloc = torch.full((M + guard_rows, K), 0x7F, dtype=torch.uint8, device=dev)
        a_alloc[:M] = a.view(torch.uint8)
        a = a_alloc[:M]
    b = d["b_shuf"].to(dev)
    sa, sb = d["sa"].to(dev), d["sb"].to(dev)
    bias_t = bias.to(dev) if bias is not None else torch.empty(0, dtype=tdt, device=dev)
    fn.launch_forced(c_alloc[:M].view(-1), a.view(-1), b.view(-1), sa, sb, bias_t, M, N, torch.cuda.current_stream(),
                     force_path=force_path, tile=tile, wave_layout=wave_layout)
    torch.cuda.synchronize()
    return c_alloc


def _acc(d, M, N, K, *, force_path=0, tile=None, wave_layout=0):
    from kernels.gemm.preshuffle_gemm import compile_preshuffle_gemm

    dev = torch.device("cuda")
    fn = compile_preshuffle_gemm(N=N, K=K, tile_m=128, tile_n=256, tile_k=64, in_dtype=d["kind"])
    dt = torch.int32 if d["kind"] == "int8" else torch.float32
    acc = torch.full((M, N), -7, dtype=dt, device=dev)
    fn.accumulators(acc, d["a_q"].to(dev), d["b_shuf"].to(dev), M, N, torch.cuda.current_stream(), force_path=force_path,
                    tile=tile, wave_layout=wave_layout)
    torch.cuda.synchronize()
    return acc.cpu().numpy()


def _check_fp(out_f32, ref):
    ok, ratio = O.within_north_star_tolerance(out_f32, ref, 1e-2)
    assert ok, f"outside 1e-2*|ref| + 1e-2*max|ref| (worst ratio {ratio:.3f})"


# ---- config 1: int8 128x1024x1024 --------------------------------------------------------------
@pytest.mark.parametrize("force_path,tile", [(1, (128, 256)), (1, (32, 256)), (1, (64, 64)), (1, (256, 256)), (1, (128, 128)),
                                             (1, (64, 256))])
def test_int8_config1_bit_exact(force_path, tile):
    M, N, K = 128, 1024, 1024
    d = make_a8w8(M, N, K, "int8", seed=0)
    want = O.int32_accumulators(np_bytes(d["a_q"]), np_bytes(d["b_q"]))
    got = _acc(d, M, N, K, force_path=force_path, tile=tile)
    assert np.array_equal(got, want)
    c = _launch(d, M, N, K, force_path=force_path, tile=tile)
    ref = C.a8w8(np_bytes(d["a_q"]), np_bytes(d["b_shuf"]), d["sa"].numpy(), d["sb"].numpy(), "int8")
    assert np.array_equal(bf16_bits(c[:M]), ref["c_bf16_bits"])
    _check_fp(c[:M].float().cpu().numpy(), O.run_torch(np_bytes(d["a_q"]), np_bytes(d["b_q"]), d["sa"].numpy(), d["sb"].numpy(), "int8"))


@pytest.mark.parametrize("kind", ["int8", "fp8"])
@pytest.mark.parametrize("M", [1, 7, 16, 17, 32, 33, 47, 48, 49, 64])
def test_small_m_paths(kind, M):
    N, K = 1024, 2048
    d = make_a8w8(M, N, K, kind, seed=M)
    ref = O.run_torch(np_bytes(d["a_q"]), np_bytes(d["b_q"]), d["sa"].numpy(), d["sb"].numpy(), kind)
    for force_path in (2, 1):
        c = _launch(d, M, N, K, force_path=force_path, guard_rows=40)
        _check_fp(c[:M].float().cpu().numpy(), ref)
        assert (c[M:] == SENTINEL).all(), "rows past M were written"
        if kind == "int8":
            got = _acc(d, M, N, K, force_path=force_path)
            assert np.array_equal(got, O.int32_accumulators(np_bytes(d["a_q"]), np_bytes(d["b_q"])))
            cref = C.a8w8(np_bytes(d["a_q"]), np_bytes(d["b_shuf"]), d["sa"].numpy(), d["sb"].numpy(), "int8")
            assert np.array_equal(bf16_bits(c[:M]), cref["c_bf16_bits"])


@pytest.mark.parametrize("kind", ["int8", "fp8"])
@pytest.mark.parametrize("M,N,K", [(33, 1040, 1088), (48, 272, 192), (50, 48, 64), (64, 528, 320), (41, 992, 4160), (64, 6144, 4096)])
def test_streaming_kernel_above_32_rows_ragged(kind, M, N, K):
    # three and four 16-row blocks, N % 128 != 0, K % 128 == 64, a single K step, the long-row plan (8 wavefronts)
    d = make_a8w8(M, N, K, kind, seed=M + N)
    c = _launch(d, M, N, K, force_path=2, guard_rows=24)
    assert (c[M:] == SENTINEL).all(), "rows past M were written"
    _check_fp(c[:M].float().cpu().numpy(), O.run_torch(np_bytes(d["a_q"]), np_bytes(d["b_q"]), d["sa"].numpy(), d["sb"].numpy(), kind))
    if kind == "int8":
        assert np.array_equal(_acc(d, M, N, K, force_path=2), O.int32_accumulators(np_bytes(d["a_q"]), np_bytes(d["b_q"])))
        cref = C.a8w8(np_bytes(d["a_q"]), np_bytes(d["b_shuf"]), d["sa"].numpy(), d["sb"].numpy(), "int8")
        assert np.array_equal(bf16_bits(c[:M]), cref["c_bf16_bits"])
        # the automatic plan (streaming or tiled, whichever the planner takes for the shape) gives the same bits
        assert np.array_equal(bf16_bits(_launch(d, M, N, K)[:M]), cref["c_bf16_bits"])


def test_small_m_no_ksplit():
    # N/16 >= 2048 n-blocks: the dispatcher keeps K whole (ksplit 1), 8 n-blocks per workgroup
    M, N, K = 32, 32768, 256
    d = make_a8w8(M, N, K, "int8", seed=1)
    got = _acc(d, M, N, K, force_path=2)
    assert np.array_equal(got, O.int32_accumulators(np_bytes(d["a_q"]), np_bytes(d["b_q"])))


# ---- config 2: fp8 decode, N=6144 K=4096 -------------------------------------------------------
@pytest.mark.parametrize("M", [1, 16, 32])
def test_fp8_config2_decode(M):
    N, K = 6144, 4096
    d = make_a8w8(M, N, K, "fp8", seed=0)
    ref = O.run_torch(np_bytes(d["a_q"]), np_bytes(d["b_q"]), d["sa"].numpy(), d["sb"].numpy(), "fp8")
    c = _launch(d, M, N, K)
    _check_fp(c[:M].float().cpu().numpy(), ref)
    # accumulators against the float64 sum of exact products (C oracle, wire format)
    acc = _acc(d, M, N, K)
    want = C.a8w8(np_bytes(d["a_q"]), np_bytes(d["b_shuf"]), d["sa"].numpy(), d["sb"].numpy(), "fp8")["acc_f32"]
    assert np.allclose(acc, want, rtol=1e-4, atol=1e-4 * np.abs(want).max())


# ---- ragged shapes: reference's (33, 1024, 2048) OOB case, odd K/64, N not a multiple of the tile ----
@pytest.mark.parametrize("kind", ["int8", "fp8"])
@pytest.mark.parametrize("M,N,K", [(33, 1024, 2048), (129, 1040, 1088), (300, 272, 192), (257, 48, 64)])
def test_ragged(kind, M, N, K):
    d = make_a8w8(M, N, K, kind, seed=3)
    ref = O.run_torch(np_bytes(d["a_q"]), np_bytes(d["b_q"]), d["sa"].numpy(), d["sb"].numpy(), kind)
    for tile in [(256, 256), (128, 256), (64, 256), (32, 256), (128, 128), (64, 64)]:
        c = _launch(d, M, N, K, force_path=1, tile=tile, guard_rows=64)
        _check_fp(c[:M].float().cpu().numpy(), ref)
        assert (c[M:] == SENTINEL).all(), f"tile {tile}: rows past M were written"
        if kind == "int8":
            got = _acc(d, M, N, K, force_path=1, tile=tile)
            assert np.array_equal(got, O.int32_accumulators(np_bytes(d["a_q"]), np_bytes(d["b_q"]))), f"tile {tile}"


# ---- config 3: fp8 prefill 8192x4096x4096 ------------------------------------------------------
def test_fp8_config3_prefill():
    M, N, K = 8192, 4096, 4096
    d = make_a8w8(M, N, K, "fp8", seed=0)
    c = _launch(d, M, N, K)
    a32 = torch.from_numpy(O.e4m3fn_to_f32(np_bytes(d["a_q"]))) * d["sa"].view(-1, 1)
    b32 = torch.from_numpy(O.e4m3fn_to_f32(np_bytes(d["b_q"]))) * d["sb"].view(-1, 1)
    ref = torch.mm(a32, b32.T).numpy()  # the reference's run_torch on CPU tensors
    _check_fp(c[:M].float().cpu().numpy(), ref)


# ---- config 4: int8 4096x28672x8192, accumulators bit-exact on a row sample at full size ---------
def test_int8_config4_large_ffn():
    M, N, K = 4096, 28672, 8192
    d = make_a8w8(M, N, K, "int8", seed=0)
    acc = _acc(d, M, N, K)
    rows = np.array(sorted({(i * 131 + 7) % M for i in range(192)} | {0, 255, 256, M - 1}))
    want = O.int32_accumulators(np_bytes(d["a_q"])[rows], np_bytes(d["b_q"]))
    assert np.array_equal(acc[rows], want)
    # size-independent property over ALL rows: column sums of the accumulators equal (sum_m A[m,:]) . W[n,:]
    colsum = acc.astype(np.int64).sum(axis=0)
    a_sum = np_bytes(d["a_q"]).view(np.int8).astype(np.int64).sum(axis=0)
    want_sum = np_bytes(d["b_q"]).view(np.int8).astype(np.int64) @ a_sum
    assert np.array_equal(colsum, want_sum)
    c = _launch(d, M, N, K)
    ref_rows = C.a8w8(np_bytes(d["a_q"])[rows], np_bytes(d["b_shuf"]), d["sa"].numpy()[rows], d["sb"].numpy(), "int8")
    assert np.array_equal(bf16_bits(c[:M])[rows], ref_rows["c_bf16_bits"])


# ---- fused epilogues (bias / relu / silu / gelu) -------------------------------------------------
@pytest.mark.parametrize("epilogue", ["bias", "bias_relu", "bias_silu", "bias_gelu"])
@pytest.mark.parametrize("M,force_path", [(16, 2), (200, 1)])
def test_epilogues(epilogue, M, force_path):
    N, K = 512, 1024
    d = make_a8w8(M, N, K, "int8", seed=11, w_std=0.05)
    g = torch.Generator().manual_seed(5)
    bias = (torch.randn(N, generator=g) * 0.5).to(torch.bfloat16)
    c = _launch(d, M, N, K, force_path=force_path, epilogue=epilogue, bias=bias)
    acc = O.int32_accumulators(np_bytes(d["a_q"]), np_bytes(d["b_q"]))
    act = {"bias": "none", "bias_relu": "relu", "bias_silu": "silu", "bias_gelu": "gelu"}[epilogue]
    ref = O.epilogue_a8w8(acc, d["sa"].numpy(), d["sb"].numpy(), bias.float().numpy(), act)
    out = c[:M].float().cpu().numpy()
    assert np.allclose(out, ref, rtol=1e-2, atol=1e-2), np.abs(out - ref).max()


def test_fp16_output():
    M, N, K = 64, 256, 512
    d = make_a8w8(M, N, K, "fp8", seed=2)
    ref = O.run_torch(np_bytes(d["a_q"]), np_bytes(d["b_q"]), d["sa"].numpy(), d["sb"].numpy(), "fp8")
    c = _launch(d, M, N, K, out_dtype="fp16")
    _check_fp(c[:M].float().cpu().numpy(), ref)


# ---- HIP-graph capture, mirroring the reference's graph test (M=1, N=K=8192, fp8) ---------------
def test_graph_capture_matches_eager():
    from kernels.gemm.preshuffle_gemm import compile_preshuffle_gemm

    M, N, K = 1, 8192, 8192
    d = make_a8w8(M, N, K, "fp8", seed=9, w_std=1.0)
    dev = torch.device("cuda")
    fn = compile_preshuffle_gemm(N=N, K=K, tile_m=16, tile_n=64, tile_k=256, in_dtype="fp8")
    a, b, sa, sb = d["a_q"].to(dev), d["b_shuf"].to(dev), d["sa"].to(dev), d["sb"].to(dev)
    c = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
    bias = torch.empty(0, dtype=torch.bfloat16, device=dev)

    def run():
        fn(c.view(-1), a.view(-1), b.view(-1), sa, sb, bias, M, N, torch.cuda.current_stream())

    run()
    torch.cuda.synchronize()
    eager = c.clone()
    assert eager.abs().max().item() > 0
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        run()
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    c.zero_()
    with torch.cuda.graph(g, stream=s):
        run()
    torch.cuda.synchronize()
    for _ in range(3):
        c.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(c, eager)


# ---- very short K (one or two mainloop steps): the accumulators are read right after the last MFMA ------------
@pytest.mark.parametrize("K", [64, 128, 256])
def test_short_k_every_tile(K):
    M, N = 256, 512
    d = make_a8w8(M, N, K, "int8", seed=K)
    want = O.int32_accumulators(np_bytes(d["a_q"]), np_bytes(d["b_q"]))
    ref = C.a8w8(np_bytes(d["a_q"]), np_bytes(d["b_shuf"]), d["sa"].numpy(), d["sb"].numpy(), "int8")["c_bf16_bits"]
    for tile in [(256, 256), (128, 512), (128, 256), (64, 256), (32, 256), (128, 128), (64, 64)]:
        for _ in range(3):
            c = _launch(d, M, N, K, force_path=1, tile=tile)
            assert np.array_equal(bf16_bits(c[:M]), ref), f"tile {tile}"
            assert np.array_equal(_acc(d, M, N, K, force_path=1, tile=tile), want), f"tile {tile}"


# ---- the 256x256 tile of eight wavefronts (what the planner picks for problems that fill the GPU) and the 2x2 form ----
@pytest.mark.parametrize("wave_layout", [8, 2])
@pytest.mark.parametrize("M,N,K", [(128, 1024, 1024), (300, 272, 192), (257, 48, 64), (700, 528, 320), (600, 992, 4160)])
def test_int8_wavefront_layouts_bit_exact(wave_layout, M, N, K):
    d = make_a8w8(M, N, K, "int8", seed=M)
    want = O.int32_accumulators(np_bytes(d["a_q"]), np_bytes(d["b_q"]))
    ref = C.a8w8(np_bytes(d["a_q"]), np_bytes(d["b_shuf"]), d["sa"].numpy(), d["sb"].numpy(), "int8")["c_bf16_bits"]
    assert np.array_equal(_acc(d, M, N, K, force_path=1, tile=(256, 256), wave_layout=wave_layout), want)
    c = _launch(d, M, N, K, force_path=1, tile=(256, 256), guard_rows=32, wave_layout=wave_layout)
    assert np.array_equal(bf16_bits(c[:M]), ref)
    assert (c[M:] == SENTINEL).all()


@pytest.mark.parametrize("epilogue", ["none", "bias_silu"])
def test_fp8_eight_wavefront_tile(epilogue):
    M, N, K = 520, 784, 2112
    d = make_a8w8(M, N, K, "fp8", seed=4, w_std=0.05)
    g = torch.Generator().manual_seed(1)
    bias = (torch.randn(N, generator=g) * 0.2).to(torch.bfloat16)
    ref = O.run_torch(np_bytes(d["a_q"]), np_bytes(d["b_q"]), d["sa"].numpy(), d["sb"].numpy(), "fp8")
    if epilogue != "none":
        ref = O.apply_bias_act(ref, bias.float().numpy(), "silu")
    c = _launch(d, M, N, K, force_path=1, tile=(256, 256), epilogue=epilogue, bias=bias, wave_layout=8)
    _check_fp(c[:M].float().cpu().numpy(), ref)
