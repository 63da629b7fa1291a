"""Seeded sweep over irregular shapes through the automatic dispatcher (streaming kernel, tiled kernel, split-K plan):
every dtype against the CPU oracle.  int8 outputs must be bit-identical whatever plan the library picks."""

import numpy as np
import pytest
import torch

from helpers import bf16_bits, make_a8w8, make_a16w16, make_mxfp4, np_bytes, np_u16
from oracle import c_oracle as C
from oracle import psg_oracle as O

pytestmark = pytest.mark.gpu


def _shapes(seed, n, k_unit, n_unit, k_max):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(n):
        m = int(rng.choice([1, 2, 15, 16, 17, 31, 32, 33, 47, 48, 49, 63, 64, 65, 100, 128, 129, 255, 256, 300, 513]))
        nn = int(rng.integers(1, 40)) * n_unit
        k = int(rng.integers(1, k_max // k_unit + 1)) * k_unit
        out.append((m, nn, k))
    # long-K few-tile cases that trigger the split-K plan, and the extremes of M
    out += [(40, 16 * n_unit, 8192 if k_unit <= 64 else 8192), (96, 32 * n_unit, 6144), (2048, n_unit, k_unit), (1, n_unit, k_unit)]
    return out


@pytest.mark.parametrize("kind", ["int8", "fp8"])
def test_fuzz_a8w8(kind):
    from kernels.gemm.preshuffle_gemm import compile_preshuffle_gemm

    dev = torch.device("cuda")
    for i, (M, N, K) in enumerate(_shapes(1 if kind == "int8" else 2, 24, 64, 16, 2048)):
        d = make_a8w8(M, N, K, kind, seed=100 + i)
        fn = compile_preshuffle_gemm(N=N, K=K, tile_m=64, tile_n=64, tile_k=64, in_dtype=kind)
        c = torch.full((M + 3, N), -8192.0, dtype=torch.bfloat16, device=dev)
        fn(c[:M], d["a_q"].to(dev), d["b_shuf"].to(dev), d["sa"].to(dev), d["sb"].to(dev), torch.empty(0, dtype=torch.bfloat16, device=dev),
           M, N, None)
        torch.cuda.synchronize()
        assert (c[M:] == -8192.0).all(), (M, N, K)
        if kind == "int8":
            ref = C.a8w8(np_bytes(d["a_q"]), np_bytes(d["b_shuf"]), d["sa"].numpy(), d["sb"].numpy(), "int8")["c_bf16_bits"]
            assert np.array_equal(bf16_bits(c[:M]), ref), (M, N, K)
        else:
            ref = O.run_torch(np_bytes(d["a_q"]), np_bytes(d["b_q"]), d["sa"].numpy(), d["sb"].numpy(), kind)
            ok, ratio = O.within_north_star_tolerance(c[:M].float().cpu().numpy(), ref)
            assert ok, (M, N, K, ratio)


def test_fuzz_bf16():
    from kernels.gemm.preshuffle_gemm import compile_preshuffle_gemm

    dev = torch.device("cuda")
    for i, (M, N, K) in enumerate(_shapes(3, 16, 32, 16, 1024)):
        d = make_a16w16(M, N, K, "bf16", seed=200 + i, w_std=0.05)
        fn = compile_preshuffle_gemm(N=N, K=K, tile_m=128, tile_n=64, tile_k=32, in_dtype="bf16")
        c = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
        none = torch.empty(0, dtype=torch.float32, device=dev)
        fn(c, d["a_q"].to(dev), d["b_shuf"].to(dev), none, none, torch.empty(0, dtype=torch.bfloat16, device=dev), M, N, None)
        torch.cuda.synchronize()
        ref = O.run_torch(np_u16(d["a_q"]), np_u16(d["b_q"]), None, None, "bf16")
        ok, ratio = O.within_north_star_tolerance(c.float().cpu().numpy(), ref)
        assert ok, (M, N, K, ratio)


def test_fuzz_mxfp4():
    from kernels.gemm.mxfp4_preshuffle import launch_gemm

    dev = torch.device("cuda")
    for i, (M, N, K) in enumerate(_shapes(4, 16, 256, 32, 2048)):
        d = make_mxfp4(M, N, K, seed=300 + i)
        t = {k: d[k].to(dev) for k in ("a_q", "b_shuf", "sa_shuf", "sb_shuf")}
        c = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
        launch_gemm(c, t["a_q"], t["b_shuf"], t["sa_shuf"], t["sb_shuf"], M, N, None, N, K, 32, 128, 256, "fp4", "bf16", "fp4", 1,
                    -1, -1, -1, -1, -1, -1, 0, 0)
        torch.cuda.synchronize()
        ref = O.run_torch_w4(d["a_q"].numpy(), d["b_q"].numpy(), d["sa"].numpy(), d["sb"].numpy())
        ok, ratio = O.within_north_star_tolerance(c.float().cpu().numpy(), ref)
        assert ok, (M, N, K, ratio)


@pytest.mark.parametrize("a_dtype,b_dtype", [("fp8", "fp8"), ("fp6", "fp4"), ("fp8", "fp4"), ("fp4", "fp8")])
def test_fuzz_mx_formats(a_dtype, b_dtype):
    # the general MX kernel through the automatic dispatcher (split-K plan included), ragged M, any N % 32, K % 256
    from helpers import make_mx
    from kernels.gemm.mxfp4_preshuffle import launch_gemm

    dev = torch.device("cuda")
    for i, (M, N, K) in enumerate(_shapes(7, 10, 256, 32, 2048) + [(32, 512, 8192), (64, 1024, 4096)]):
        d = make_mx(M, N, K, a_dtype, b_dtype, seed=300 + i)
        c = torch.full((M + 3, N), -8192.0, dtype=torch.bfloat16, device=dev)
        launch_gemm(c, d["a_q"].to(dev), d["b_shuf"].to(dev), d["sa_shuf"].to(dev), d["sb_shuf"].to(dev), M, N, None, N, K, 64, 128, 256,
                    a_dtype, "bf16", b_dtype, 1, -1, -1, -1, -1, -1, -1, 0, 0)
        torch.cuda.synchronize()
        assert (c[M:] == -8192.0).all(), (M, N, K)
        ref = O.run_torch_mx(d["a_q"].numpy(), d["b_q"].numpy(), d["sa"].numpy(), d["sb"].numpy(), a_dtype, b_dtype)
        ok, ratio = O.within_north_star_tolerance(c[:M].float().cpu().numpy(), ref)
        assert ok, (M, N, K, ratio)
