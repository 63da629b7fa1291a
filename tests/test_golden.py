"""Golden fixtures (tests/golden/*.npz, written by tests/golden/gen_golden.py from this repository's
pinned oracle): the oracle and the package's host helpers must reproduce them byte for byte on the CPU,
and the GPU kernels must reproduce their known answers."""

import os

import numpy as np
import pytest
import torch

from flydsl_amd import layout, quant
from oracle import c_oracle as C
from oracle import psg_oracle as O

G = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _load(name):
    return dict(np.load(os.path.join(G, name)))


@pytest.mark.parametrize("name,kind", [("a8w8_int8_m20_n48_k192.npz", "int8"), ("a8w8_fp8_m33_n64_k128.npz", "fp8")])
def test_oracle_and_package_reproduce_a8w8_fixture(name, kind):
    g = _load(name)
    x, w = g["x"].astype(np.float32), g["w"].astype(np.float32)
    aq, sa = O.pertoken_quant(x, kind)
    bq, sb = O.pertoken_quant(w, kind)
    assert np.array_equal(aq.view(np.uint8), g["a_q"]) and np.array_equal(bq.view(np.uint8), g["b_q"])
    assert np.array_equal(sa, g["sa"]) and np.array_equal(sb, g["sb"])
    assert np.array_equal(O.shuffle_weight(bq.view(np.uint8)), g["b_shuf"])
    assert np.array_equal(O.run_torch(aq, bq, sa, sb, kind), g["c_ref"])
    qd = torch.int8 if kind == "int8" else torch.float8_e4m3fn
    ta, tsa = quant.pertoken_quant(torch.from_numpy(x), quant_dtype=qd)
    tb, _ = quant.pertoken_quant(torch.from_numpy(w), quant_dtype=qd)
    assert np.array_equal(ta.view(torch.uint8).numpy(), g["a_q"]) and np.array_equal(tsa.numpy(), g["sa"])
    assert np.array_equal(layout.shuffle_weight(tb).view(torch.uint8).numpy(), g["b_shuf"])
    r = C.a8w8(g["a_q"], g["b_shuf"], g["sa"], g["sb"], kind, want_acc_i32=(kind == "int8"))
    if kind == "int8":
        assert np.array_equal(r["acc_i32"], g["acc"]) and np.array_equal(r["c_bf16_bits"], g["c_bf16_bits"])


def test_oracle_and_package_reproduce_mxfp4_fixture():
    g = _load("mxfp4_m40_n64_k512.npz")
    x, w = g["x"].astype(np.float32), g["w"].astype(np.float32)
    xp = np.zeros((64, x.shape[1]), np.float32)
    xp[:40] = x
    ap, sa = O.per_1x32_f4_quant(xp)
    bp, sb = O.per_1x32_f4_quant(w)
    assert np.array_equal(ap[:40], g["a_q"]) and np.array_equal(bp, g["b_q"])
    assert np.array_equal(sa, g["sa"]) and np.array_equal(sb, g["sb"])
    assert np.array_equal(O.shuffle_weight_w4(bp), g["b_shuf"])
    assert np.array_equal(O.shuffle_scale_w4(sa), g["sa_shuf"]) and np.array_equal(O.shuffle_scale_w4(sb), g["sb_shuf"])
    assert np.array_equal(O.run_torch_w4(ap[:40], bp, sa, sb), g["c_ref"])
    tp, ts, _ = quant.per_1x32_f4_quant(torch.from_numpy(xp))
    assert np.array_equal(tp.view(torch.uint8).numpy()[:40], g["a_q"]) and np.array_equal(ts.view(torch.uint8).numpy(), g["sa"])
    assert np.array_equal(layout.shuffle_scale_w4(ts.view(torch.uint8), 1, False).numpy(), g["sa_shuf"])


@pytest.mark.gpu
@pytest.mark.parametrize("name,kind", [("a8w8_int8_m20_n48_k192.npz", "int8"), ("a8w8_fp8_m33_n64_k128.npz", "fp8")])
@pytest.mark.parametrize("force_path", [1, 2])
def test_gpu_reproduces_a8w8_fixture(name, kind, force_path):
    from kernels.gemm.preshuffle_gemm import compile_preshuffle_gemm

    g = _load(name)
    M, K = g["a_q"].shape
    N = g["b_q"].shape[0]
    dev = torch.device("cuda")
    fn = compile_preshuffle_gemm(N=N, K=K, tile_m=64, tile_n=64, tile_k=64, in_dtype=kind)
    a = torch.from_numpy(g["a_q"]).to(dev)
    b = torch.from_numpy(g["b_shuf"]).to(dev)
    sa = torch.from_numpy(g["sa"]).reshape(-1).to(dev)
    sb = torch.from_numpy(g["sb"]).reshape(-1).to(dev)
    c = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
    fn.launch_forced(c, a, b, sa, sb, torch.empty(0, dtype=torch.bfloat16, device=dev), M, N, None, force_path=force_path)
    torch.cuda.synchronize()
    ok, ratio = O.within_north_star_tolerance(c.float().cpu().numpy(), g["c_ref"])
    assert ok, ratio
    if kind == "int8":
        assert np.array_equal(c.view(torch.int16).cpu().numpy().view(np.uint16), g["c_bf16_bits"])
        acc = torch.zeros(M, N, dtype=torch.int32, device=dev)
        fn.accumulators(acc, a, b, M, N, None, force_path=force_path)
        torch.cuda.synchronize()
        assert np.array_equal(acc.cpu().numpy(), g["acc"])


@pytest.mark.gpu
def test_gpu_reproduces_mxfp4_fixture():
    from kernels.gemm.mxfp4_preshuffle import launch_gemm

    g = _load("mxfp4_m40_n64_k512.npz")
    M, N, K = 40, 64, 512
    dev = torch.device("cuda")
    t = {k: torch.from_numpy(g[k]).to(dev) for k in ("a_q", "b_shuf", "sa_shuf", "sb_shuf")}
    c = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
    launch_gemm(c, t["a_q"], t["b_shuf"], t["sa_shuf"], t["sb_shuf"], M, N, None, N, K, 64, 128, 256, "fp4", "bf16", "fp4", 1,
                -1, -1, -1, -1, -1, -1, 0, 0)
    torch.cuda.synchronize()
    ok, ratio = O.within_north_star_tolerance(c.float().cpu().numpy(), g["c_ref"])
    assert ok, ratio
