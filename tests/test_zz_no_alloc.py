"""The entry point that allocates nothing (psg_gemm_a8w8_static) against psg_gemm_a8w8 with a caller workspace:
same plan, same kernels, so the outputs must be the same bits (int8: exact integer partial sums; fp8: the partial
sums are added in a fixed order).  Two calls in a row through the C ABI, the second on a smaller problem, so that
stale partial sums of the first call sit in the shared scratch while the second runs."""

import ctypes

import numpy as np
import pytest
import torch

from helpers import bf16_bits, make_a8w8, np_bytes
from oracle import c_oracle as C

pytestmark = pytest.mark.gpu


def _args(kind, d, c, M, N, K, dev):
    from flydsl_amd import _lib

    t = {k: d[k].to(dev) for k in ("a_q", "b_shuf", "sa", "sb")}
    a = _lib.A8W8Args()
    a.c, a.a, a.b = c.data_ptr(), t["a_q"].data_ptr(), t["b_shuf"].data_ptr()
    a.scale_a, a.scale_b = t["sa"].data_ptr(), t["sb"].data_ptr()
    a.M, a.N, a.K = M, N, K
    a.in_dtype = _lib.IN_DTYPE[kind]
    return a, t  # t keeps the operands alive


@pytest.mark.parametrize("kind", ["int8", "fp8"])
def test_static_scratch_entry_matches_workspace_entry(kind):
    from flydsl_amd import _lib

    handle = _lib.lib()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    assert handle.psg_init() == 0, handle.psg_last_error()
    stream = _lib.stream_handle(None)
    for (M, N, K) in [(80, 2048, 8192), (72, 512, 6144)]:  # both take the split-K plan; the second is smaller
        need = handle.psg_workspace_bytes(M, N, K, _lib.IN_DTYPE[kind])
        assert 0 < need <= handle.psg_static_scratch_bytes()
        d = make_a8w8(M, N, K, kind, seed=M)
        want = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
        got = torch.full((M + 4, N), -8192.0, dtype=torch.bfloat16, device=dev)
        ws = torch.empty(need, dtype=torch.uint8, device=dev)
        a, keep = _args(kind, d, want, M, N, K, dev)
        a.workspace, a.workspace_bytes = ws.data_ptr(), need
        assert handle.psg_gemm_a8w8(ctypes.byref(a), stream) == 0, handle.psg_last_error()
        b, keep2 = _args(kind, d, got, M, N, K, dev)
        print(f"static entry: {kind} M={M} N={N} K={K}", flush=True)
        assert handle.psg_gemm_a8w8_static(ctypes.byref(b), stream) == 0, handle.psg_last_error()
        torch.cuda.synchronize()
        assert np.array_equal(bf16_bits(got[:M]), bf16_bits(want))
        assert (got[M:] == -8192.0).all()
        if kind == "int8":
            ref = C.a8w8(np_bytes(d["a_q"]), np_bytes(d["b_shuf"]), d["sa"].numpy(), d["sb"].numpy(), "int8")
            assert np.array_equal(bf16_bits(want), ref["c_bf16_bits"])


def test_static_scratch_entry_rejects_oversized_plans_and_runs_unsplit_problems():
    from flydsl_amd import _lib

    handle = _lib.lib()
    dev = torch.device("cuda:0")
    # forced 16-way split of a problem whose partial sums exceed the 32 MiB scratch: refused before any launch
    a = _lib.A8W8Args()
    a.a = a.b = a.c = a.scale_a = a.scale_b = 0x1000
    a.M, a.N, a.K, a.in_dtype = 1024, 1024, 4096, 0
    a.force_path, a.tile_m, a.tile_n, a.tile_k = 1, 128, 128, 16
    assert handle.psg_gemm_a8w8_static(ctypes.byref(a), None) == -4  # PSG_E_WORKSPACE
    assert b"static scratch" in handle.psg_last_error()
    # a problem without a split-K plan (small M) goes straight through
    M, N, K = 16, 256, 512
    d = make_a8w8(M, N, K, "int8", seed=9)
    got = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
    b, keep = _args("int8", d, got, M, N, K, dev)
    assert handle.psg_gemm_a8w8_static(ctypes.byref(b), _lib.stream_handle(None)) == 0, handle.psg_last_error()
    torch.cuda.synchronize()
    ref = C.a8w8(np_bytes(d["a_q"]), np_bytes(d["b_shuf"]), d["sa"].numpy(), d["sb"].numpy(), "int8")
    assert np.array_equal(bf16_bits(got), ref["c_bf16_bits"])
