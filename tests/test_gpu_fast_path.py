"""The launcher's validated-once path (the counterpart of the positional fast path the reference's ``flyc.compile``
returns, python/flydsl/compiler/jit_function.py:1613-1690): same bits as the path that checks every call, and a change of
operands goes through the checks again, so a too-small C is still refused."""

import numpy as np
import pytest
import torch

from helpers import bf16_bits, make_a8w8, np_bytes
from oracle import c_oracle as C

pytestmark = pytest.mark.gpu


def _operands(M, N, K, kind, seed):
    d = make_a8w8(M, N, K, kind, seed=seed)
    dev = torch.device("cuda")
    t = {k: d[k].to(dev) for k in ("a_q", "b_shuf", "sa", "sb")}
    ref = C.a8w8(np_bytes(d["a_q"]), np_bytes(d["b_shuf"]), d["sa"].numpy(), d["sb"].numpy(), kind)["c_bf16_bits"]
    return t, ref


@pytest.mark.parametrize("M,N,K", [(16, 1024, 2048), (96, 2048, 8192), (300, 512, 1024)])
def test_fast_path_gives_the_bits_of_the_checked_path(M, N, K):
    """int8, so both are also bit-exact against the C oracle; (96, 2048, 8192) takes the split-K plan with its workspace."""
    from flydsl_amd import compiler as flyc
    from kernels.gemm.preshuffle_gemm import compile_preshuffle_gemm

    fn = compile_preshuffle_gemm(N=N, K=K, tile_m=128, tile_n=256, tile_k=64, in_dtype="int8")
    t, ref = _operands(M, N, K, "int8", seed=5)
    dev = torch.device("cuda")
    bias = torch.empty(0, dtype=torch.bfloat16, device=dev)
    stream = torch.cuda.current_stream()
    c_checked = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
    fn.launch_checked(c_checked, t["a_q"], t["b_shuf"], t["sa"], t["sb"], bias, M, N, stream)
    c_fast = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
    compiled = flyc.compile(fn, c_fast, t["a_q"], t["b_shuf"], t["sa"], t["sb"], bias, M, N, stream)  # first call: checked, cached
    before = len(fn._fast)
    for _ in range(3):
        c_fast.zero_()
        compiled(c_fast, t["a_q"], t["b_shuf"], t["sa"], t["sb"], bias, M, N, stream)  # looked up
    torch.cuda.synchronize()
    assert len(fn._fast) == before
    assert np.array_equal(bf16_bits(c_fast), bf16_bits(c_checked))
    assert np.array_equal(bf16_bits(c_fast), ref)
    # other operands at other addresses: a new entry, still the right bits
    t2, ref2 = _operands(M, N, K, "int8", seed=6)
    c2 = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
    compiled(c2, t2["a_q"], t2["b_shuf"], t2["sa"], t2["sb"], bias, M, N, stream)
    torch.cuda.synchronize()
    assert len(fn._fast) == before + 1
    assert np.array_equal(bf16_bits(c2), ref2)


def test_fast_path_still_refuses_a_too_small_c():
    from kernels.gemm.preshuffle_gemm import compile_preshuffle_gemm

    M, N, K = 64, 512, 1024
    fn = compile_preshuffle_gemm(N=N, K=K, tile_m=128, tile_n=256, tile_k=64, in_dtype="int8")
    t, ref = _operands(M, N, K, "int8", seed=7)
    dev = torch.device("cuda")
    bias = torch.empty(0, dtype=torch.bfloat16, device=dev)
    stream = torch.cuda.current_stream()
    c = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
    for _ in range(2):
        fn(c, t["a_q"], t["b_shuf"], t["sa"], t["sb"], bias, M, N, stream)
    torch.cuda.synchronize()
    assert np.array_equal(bf16_bits(c), ref)
    # the same storage seen through a smaller tensor: same address, fewer elements -> not in the table -> checked -> refused
    with pytest.raises(ValueError, match="at least"):
        fn(c.view(-1)[: M * N - 8], t["a_q"], t["b_shuf"], t["sa"], t["sb"], bias, M, N, stream)
    # a larger M on the cached operands: another key, refused by the checks as well
    with pytest.raises(ValueError, match="at least"):
        fn(c, t["a_q"], t["b_shuf"], t["sa"], t["sb"], bias, M + 1, N, stream)
    # and the cached entry is still good
    c.zero_()
    fn(c, t["a_q"], t["b_shuf"], t["sa"], t["sb"], bias, M, N, stream)
    torch.cuda.synchronize()
    assert np.array_equal(bf16_bits(c), ref)
