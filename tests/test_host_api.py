"""Host-side tests that need no GPU: the package's quantisers / layouts against the oracle, the validation
rules of the entry points (the cases the reference's own tests hold,
tests/kernels/test_preshuffle_gemm.py:983-1039), and the C ABI (library loads, exports every declared
symbol, struct layouts match the header)."""

import ctypes
import os
import re
import subprocess
import sys
import tempfile

import numpy as np
import pytest
import torch

from flydsl_amd import _lib, layout, quant
from kernels.gemm.mxfp4_preshuffle import launch_gemm
from kernels.gemm.preshuffle_gemm import compile_preshuffle_gemm
from oracle import psg_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "psgemm.h")


# ---- package helpers == oracle --------------------------------------------------------------------
def test_package_layouts_equal_oracle():
    g = torch.Generator().manual_seed(0)
    x = torch.randint(0, 255, (64, 256), generator=g, dtype=torch.uint8)
    assert np.array_equal(layout.shuffle_weight(x).numpy(), O.shuffle_weight(x.numpy()))
    h = torch.randn(64, 256, generator=g).to(torch.bfloat16)
    assert np.array_equal(layout.shuffle_weight(h).view(torch.int16).numpy(), O.shuffle_weight(h.view(torch.int16).numpy()))
    assert np.array_equal(layout.shuffle_weight_w4(x, 16, False, False).numpy(), O.shuffle_weight_w4(x.numpy()))
    s = torch.randint(0, 255, (64, 16), generator=g, dtype=torch.uint8)
    assert np.array_equal(layout.shuffle_scale_w4(s, 1, False).numpy(), O.shuffle_scale_w4(s.numpy()))
    assert getattr(layout.shuffle_weight(x), "is_shuffled", False)
    with pytest.raises(AssertionError):
        layout.shuffle_weight(torch.zeros(20, 64, dtype=torch.int8))
    with pytest.raises(AssertionError):
        layout.shuffle_weight(torch.zeros(32, 48, dtype=torch.int8))
    # leading batch dimension, as the reference's view(-1, ...) allows
    xb = torch.randint(0, 255, (3, 32, 64), generator=g, dtype=torch.uint8)
    got = layout.shuffle_weight(xb)
    for i in range(3):
        assert np.array_equal(got[i].numpy(), O.shuffle_weight(xb[i].numpy()))


def test_package_quantisers_equal_oracle():
    g = torch.Generator().manual_seed(1)
    w = torch.randn(64, 512, generator=g) * torch.logspace(-3, 3, 64).view(-1, 1)
    w[7] = 0
    for qd, kind in ((torch.int8, "int8"), (torch.float8_e4m3fn, "fp8")):
        y, sc = quant.pertoken_quant(w, quant_dtype=qd)
        yo, so = O.pertoken_quant(w.numpy(), kind)
        assert sc.shape == (64, 1) and sc.dtype == torch.float32
        assert np.array_equal(y.view(torch.uint8).numpy(), yo.view(np.uint8))
        assert np.array_equal(sc.numpy(), so)
    p, sc, _ = quant.per_1x32_f4_quant(w)
    po, so = O.per_1x32_f4_quant(w.numpy())
    assert np.array_equal(p.view(torch.uint8).numpy(), po) and np.array_equal(sc.view(torch.uint8).numpy(), so)
    assert np.array_equal(quant.mxfp4_to_f32(p).numpy(), O.mxfp4_to_f32(po))
    b = torch.arange(256, dtype=torch.uint8)
    got, want = quant.e8m0_to_f32(b).numpy(), O.e8m0_to_f32(b.numpy())
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    v = torch.cat([torch.linspace(-8, 8, 20001), torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, -0.0, 6.0, 1e-9])])
    assert np.array_equal(quant.f32_to_e2m1_codes(v).numpy(), O.f32_to_e2m1(v.numpy()))
    e = torch.tensor([1.0, 1.5, 2.0**-127, 0.0, float("nan"), 3e38, 1.4999999])
    assert np.array_equal(quant.f32_to_e8m0(e).view(torch.uint8).numpy(), O.f32_to_e8m0(e.numpy()))


# ---- validation rules of compile_preshuffle_gemm ---------------------------------------------------
@pytest.mark.parametrize("tile_m", [48, 80, 112, 144])
def test_rejects_partial_a_tile(tile_m):
    with pytest.raises(ValueError, match=r"must be a multiple of"):
        compile_preshuffle_gemm(N=1024, K=2048, tile_m=tile_m, tile_n=256, tile_k=64, in_dtype="bf16", out_dtype="bf16")


@pytest.mark.parametrize("tile_m", [64, 96, 128, 160])
def test_accepts_whole_a_tile(tile_m):
    compile_preshuffle_gemm(N=1024, K=2048, tile_m=tile_m, tile_n=256, tile_k=64, in_dtype="bf16", out_dtype="bf16")
    compile_preshuffle_gemm(N=1024, K=2048, tile_m=tile_m, tile_n=256, tile_k=128, in_dtype="int8", out_dtype="bf16")


@pytest.mark.parametrize("bad", [(1,), (1, 2, 3), (-1, 0), (0, -1), 4])
def test_preload_validation(bad):
    with pytest.raises((ValueError, TypeError)):
        compile_preshuffle_gemm(N=1024, K=2048, tile_m=128, tile_n=256, tile_k=64, in_dtype="bf16", out_dtype="bf16", preload=bad)


def test_other_validation_errors():
    ok = dict(N=1024, K=2048, tile_m=128, tile_n=256, tile_k=128)
    with pytest.raises(ValueError, match="in_dtype"):
        compile_preshuffle_gemm(**ok, in_dtype="fp4")
    with pytest.raises(ValueError, match="tile_k"):
        compile_preshuffle_gemm(**{**ok, "tile_k": 96})
    with pytest.raises(ValueError, match="tile_k"):
        compile_preshuffle_gemm(**{**ok, "tile_k": 0})
    with pytest.raises(ValueError, match="epilogue"):
        compile_preshuffle_gemm(**ok, epilogue="bias_tanh")
    with pytest.raises(ValueError, match="lds_stage"):
        compile_preshuffle_gemm(**ok, lds_stage=3)
    with pytest.raises(ValueError, match="LDS swizzle"):
        compile_preshuffle_gemm(N=1024, K=768, tile_m=256, tile_n=256, tile_k=384, in_dtype="int8")
    with pytest.raises(ValueError, match="multiple of 16"):
        compile_preshuffle_gemm(**{**ok, "N": 1000})
    with pytest.raises(TypeError):
        compile_preshuffle_gemm(1024, 2048, 128, 256, 128)  # keyword-only, like the reference
    fn = compile_preshuffle_gemm(**ok, in_dtype="fp8", waves_per_eu=2, use_async_copy=True, xcd_swizzle=4, preload=(2, 2))
    assert fn.N == 1024 and fn.K == 2048


def test_mx_entry_validates_before_touching_the_gpu():
    base = [0, 0, 0, 0, 0, 32, 128, None, 128, 256, 32, 128, 256, "fp4", "bf16", "fp4", 1, -1, -1, -1, -1, -1, -1, 0]
    for idx, val in ((13, "fp5"), (15, "fp6"), (16, 0), (16, 70000), (12, 64), (11, 64), (14, "fp32"), (6, 256)):
        args = list(base)
        args[idx] = val
        with pytest.raises(ValueError):
            launch_gemm(*args)


def test_mx_c_abi_validation_codes():
    handle = _lib.lib()
    m = _lib.MxArgs()
    m.c = m.a = m.b = m.scale_a = m.scale_b = 0x1000
    m.M, m.N, m.K = 32, 128, 256
    for field, val, code, word in (("a_dtype", 3, -3, b"a_dtype"), ("b_dtype", 1, -3, b"b_dtype"), ("batch", 70000, -2, b"batch"),
                                   ("a_row_stride", 100, -2, b"a_row_stride"), ("a_row_stride", 120, -2, b"a_row_stride"),
                                   ("c_row_stride", 64, -2, b"c_row_stride"), ("c_row_stride", 130, -2, b"c_row_stride"),
                                   ("scale_a_chunk_stride", 128, -2, b"scale_a_chunk_stride"), ("a_batch_stride", 8, -6, b"batch strides"),
                                   ("force_path", 4, -2, b"force_path"), ("pad0", 1, -2, b"pad0")):
        old = getattr(m, field)
        setattr(m, field, val)
        assert handle.psg_gemm_mxfp4(ctypes.byref(m), None) == code, field
        assert word in handle.psg_last_error(), (field, handle.psg_last_error())
        setattr(m, field, old)
    # the fp4-only paths refuse other formats, batches and strides
    m.force_path, m.a_dtype = 1, 2
    assert handle.psg_gemm_mxfp4(ctypes.byref(m), None) == -2 and b"fp4 x fp4" in handle.psg_last_error()
    m.a_dtype, m.batch = 0, 2
    assert handle.psg_gemm_mxfp4(ctypes.byref(m), None) == -2


def test_moe_c_abi_validation_codes():
    handle = _lib.lib()
    m = _lib.MoeArgs()
    assert handle.psg_moe_gemm(ctypes.byref(m), None) == -1
    for f in ("out", "x", "w", "scale_x", "scale_w", "sorted_token_ids", "sorted_expert_ids", "sorted_weights", "num_valid_ids"):
        setattr(m, f, 0x1000)
    m.tokens, m.topk, m.experts, m.model_dim, m.inter_dim = 8, 2, 4, 256, 128
    m.sorted_size, m.blocks, m.block_m, m.in_dtype, m.out_dtype, m.stage = 76, 5, 16, 1, 0, 1
    for field, val, code, word in (("stage", 3, -2, b"stage"), ("in_dtype", 2, -3, b"in_dtype"), ("in_dtype", 5, -3, b"in_dtype"), ("out_dtype", 2, -3, b"fp32 output"),
                                   ("block_m", 48, -2, b"block_m"), ("model_dim", 192, -2, b"K=192"), ("inter_dim", 24, -2, b"output width"),
                                   ("tokens", 1 << 24, -2, b"tokens"), ("blocks", 0, -2, b"blocks"), ("x", 0x1004, -6, b"aligned"), ("x_slot_major", 2, -2, b"x_slot_major"), ("no_pairing", 2, -2, b"no_pairing"),
                                   ("pad0", 1, -2, b"pad0")):
        old = getattr(m, field)
        setattr(m, field, val)
        assert handle.psg_moe_gemm(ctypes.byref(m), None) == code, field
        assert word in handle.psg_last_error(), (field, handle.psg_last_error())
        setattr(m, field, old)
    assert handle.psg_moe_reduce(None, None, 1, 1, 4, 0, None) == -1
    assert handle.psg_moe_reduce(0x1000, 0x1000, 4, 2, 6, 0, None) == -2
    assert handle.psg_moe_reduce(0x1000, 0x1000, 4, 2, 8, 3, None) == -3
    assert handle.psg_moe_reduce(0x1008, 0x1000, 4, 2, 8, 2, None) == -6  # fp32 rows are moved 16 bytes at a time


def test_sorter_refuses_more_slots_than_experts():
    """tokens*topk + experts*block_m - topk rows only bound the padded total while a token cannot repeat an expert: experts=2,
    topk=4, block_m=2 with ids [0, 0, 0, 1] pads to 6 rows against a bound of 4."""
    handle = _lib.lib()
    a = _lib.MoeSortArgs()
    for f in ("topk_ids", "topk_weights", "sorted_ids", "sorted_weights", "sorted_expert_ids", "num_valid_ids"):
        setattr(a, f, 0x1000)
    a.tokens, a.topk, a.experts, a.block_m, a.sorted_size, a.blocks = 1, 4, 2, 2, 4, 2
    assert handle.psg_moe_sorting(ctypes.byref(a), None) == -2
    assert b"topk=4 exceeds experts=2" in handle.psg_last_error()


def test_sorter_workspace_comes_from_the_pool_of_the_launch_stream(monkeypatch):
    """A workspace the caller does not bring must outlive the queued launches on whatever stream they run: it is taken from the
    never-released pool keyed by (device, stream), not from the caching allocator, and is refused during graph capture."""
    from flydsl_amd.kernels.moe import moe_sorting as S

    class Fake:
        def __init__(self, numel, dtype, esize=4):
            self._n, self.dtype, self._e, self.is_cuda, self.device = numel, dtype, esize, True, "cuda:0"

        def numel(self):
            return self._n

        def element_size(self):
            return self._e

        def is_contiguous(self):
            return True

        def data_ptr(self):
            return 0x10000

    made = []
    capturing = [False]
    pool = _lib.WorkspacePool(alloc=lambda n, dev: made.append(Fake(n, torch.uint8, 1)) or made[-1], capturing=lambda: capturing[0])
    monkeypatch.setattr(_lib, "_pool", pool)
    monkeypatch.setattr(_lib, "workspace", lambda device, nbytes, stream=0, owner="shared": pool.get(owner, 0, int(stream), int(nbytes)))
    tokens, topk, E, B = 5000, 8, 64, 32
    want = S.moe_sorting_get_workspace_size(tokens, E, topk, B)
    assert want > 0
    rows, blocks = S.sorted_sizes(tokens, topk, E, B)
    outs = (Fake(rows, torch.int32), Fake(rows, torch.float32), Fake(blocks, torch.int32), Fake(2, torch.int32))
    routing = (Fake(tokens * topk, torch.int32), Fake(tokens * topk, torch.float32))
    args, ws = S._sort_args(tokens, topk, *outs, None, E, B, None, None, "cuda:0", routing=routing, stream_h=0x77)
    assert ws is made[0] and ws.numel() >= want and args.workspace_bytes == ws.numel()
    assert pool._live[("moe_sort", 0, 0x77)] is ws  # parked under the launch stream, never dropped
    _, ws2 = S._sort_args(tokens, topk, *outs, None, E, B, None, None, "cuda:0", routing=routing, stream_h=0x77)
    assert ws2 is ws and len(made) == 1
    _, ws3 = S._sort_args(tokens, topk, *outs, None, E, B, None, None, "cuda:0", routing=routing, stream_h=0x88)
    assert ws3 is not ws  # another stream never shares
    capturing[0] = True
    pool2 = _lib.WorkspacePool(alloc=lambda n, dev: made.append(Fake(n, torch.uint8, 1)) or made[-1], capturing=lambda: True)
    monkeypatch.setattr(_lib, "workspace", lambda device, nbytes, stream=0, owner="shared": pool2.get(owner, 0, int(stream), int(nbytes)))
    with pytest.raises(RuntimeError, match="graph capture"):
        S._sort_args(tokens, topk, *outs, None, E, B, None, None, "cuda:0", routing=routing, stream_h=0x99)


def test_mx_quantisers_match_the_oracle_byte_for_byte():
    from flydsl_amd import quant
    from oracle import psg_oracle as O

    rng = np.random.default_rng(5)
    x = (rng.standard_normal((64, 256)) * rng.choice([1e-3, 1.0, 50.0], size=(64, 1))).astype(np.float32)
    x[3, :32] = 0
    a_pad, sc, codes = O.per_1x32_f6_quant(x)
    tp, ts, tc = quant.per_1x32_f6_quant(torch.from_numpy(x))
    assert np.array_equal(tp.numpy(), a_pad) and np.array_equal(ts.numpy(), sc) and np.array_equal(tc.numpy(), codes)
    q, s8 = O.per_1x32_f8_quant(x)
    tq, ts8 = quant.per_1x32_f8_quant(torch.from_numpy(x))
    assert np.array_equal(tq.view(torch.uint8).numpy(), q) and np.array_equal(ts8.numpy(), s8)
    # every midpoint between adjacent e2m3 magnitudes, and both neighbours of each
    mags = O.e2m3_to_f32(np.arange(32, dtype=np.uint8))
    mids = (mags[:-1] + mags[1:]) / 2
    v = np.concatenate([mags, mids, np.nextafter(mids, np.float32(9)), np.nextafter(mids, np.float32(-9)), [7.75, 8.0, 1e3]]).astype(np.float32)
    v = np.concatenate([v, -v])
    assert np.array_equal(quant.f32_to_e2m3_codes(torch.from_numpy(v)).numpy(), O.f32_to_e2m3(v))
    assert np.array_equal(quant.fp6_e2m3_to_f32(torch.arange(64, dtype=torch.uint8)).numpy(), O.e2m3_to_f32(np.arange(64, dtype=np.uint8)))
    c = torch.from_numpy(rng.integers(0, 64, (4, 64), dtype=np.uint8))
    assert np.array_equal(quant.pack_fp6_e2m3(c).numpy(), O.pack_fp6(c.numpy()))


def test_fp4_4wave_call_shape_keeps_the_reference_asserts():
    from kernels.gemm.fp4_gemm_4wave import compile_fp4_gemm_4w

    assert compile_fp4_gemm_4w(K=2048).K == 2048 and compile_fp4_gemm_4w(K=512, MN=(256, 256)).MN == (256, 256)
    for bad in (300, 1280 + 256 * 0 + 128, 256 * 5, 256 * 7):  # not a multiple of 256; odd K-step counts
        with pytest.raises(AssertionError):
            compile_fp4_gemm_4w(K=bad)
    with pytest.raises(TypeError):
        compile_fp4_gemm_4w(2048)  # keyword-only like the reference


# ---- the C ABI -------------------------------------------------------------------------------------
def _declared_functions():
    text = open(HEADER).read()
    return sorted(set(re.findall(r"^\s*(?:int|void|uint64_t|const char \*)\s*\**\s*(psg_\w+)\s*\(", text, flags=re.M)))


def test_library_exports_every_declared_symbol():
    names = _declared_functions()
    assert set(names) == set(_lib.EXPORTS), names
    handle = _lib.lib()
    for n in names:
        assert getattr(handle, n) is not None
    assert handle.psg_abi_version() == _lib.ABI_VERSION
    assert handle.psg_workspace_bytes(16, 6144, 4096, 1) == 0


def test_tile_order_equals_the_oracle_remap_on_every_id():
    """The function the tiled kernel uses to turn a workgroup id into a tile (evaluated on the host through the C ABI)
    against the oracle's xcd_remap_bx_by, id by id, incl. ragged grids: tiles % 8 != 0, tiles_m % group_m != 0."""
    from oracle import psg_oracle as O

    handle = _lib.lib()
    tm, tn = ctypes.c_int32(), ctypes.c_int32()
    for tiles_m, tiles_n, group_m in [(32, 16, 8), (3, 4, 2), (7, 5, 3), (1, 13, 8), (13, 1, 4), (17, 9, 16), (64, 112, 8),
                                      (5, 5, 1), (2, 3, 8), (9, 7, 4)]:
        seen = set()
        for bx in range(tiles_m):
            for by in range(tiles_n):
                lin = bx * tiles_n + by
                handle.psg_tile_coords(lin, tiles_m, tiles_n, group_m, ctypes.byref(tm), ctypes.byref(tn))
                want = O.xcd_remap_bx_by(bx, by, tiles_m * 16, tile_m=16, tile_n=64, n=tiles_n * 64, xcd_swizzle=group_m)
                assert (tm.value, tn.value) == want, (tiles_m, tiles_n, group_m, bx, by)
                seen.add(want)
        assert len(seen) == tiles_m * tiles_n  # a bijection onto the tile grid


def test_workspace_pool_never_releases_a_buffer_it_handed_out():
    class Buf:
        def __init__(self, n, dev):
            self.n, self.dev = n, dev

        def numel(self):
            return self.n

    made = []

    def alloc(n, dev):
        made.append(Buf(n, dev))
        return made[-1]

    capturing = [False]
    pool = _lib.WorkspacePool(alloc=alloc, capturing=lambda: capturing[0])
    a = pool.get("L1", 0, 0x10, 1000)
    assert pool.get("L1", 0, 0x10, 500) is a and pool.get("L1", 0, 0x10, 1000) is a  # reuse while it is large enough
    b = pool.get("L1", 0, 0x20, 1000)
    assert b is not a  # another stream never shares
    c = pool.get("L1", 1, 0x10, 1000)
    assert c is not a and c.dev == 1  # nor another device
    e = pool.get("L2", 0, 0x10, 1000)
    assert e is not a  # nor another launcher
    d = pool.get("L1", 0, 0x10, 4000)  # growth: a new buffer, the old one is parked, not dropped
    assert d is not a and a in pool._parked and len(made) == 5
    assert pool.get("L1", 0, 0x10, 0) is None
    capturing[0] = True
    assert pool.get("L1", 0, 0x10, 4000) is d  # an existing buffer may be used during capture
    assert pool.get("L1", 0, 0x30, 4000) is d  # a capture stream borrows the launcher's warm-up buffer on that device
    with pytest.raises(RuntimeError, match="graph capture"):
        pool.get("L1", 0, 0x10, 8000)  # growth during capture is refused
    with pytest.raises(RuntimeError, match="graph capture"):
        pool.get("L3", 0, 0x30, 10)  # and so is a first allocation
    with pytest.raises(RuntimeError, match="graph capture"):
        pool.get("L1", 1, 0x30, 2000)  # another device's buffer is never borrowed
    assert len(made) == 5


def test_launchers_refuse_operands_that_would_send_a_kernel_out_of_bounds():
    """Host-side checks before any launch (no GPU needed: every case fails on the first check it reaches)."""
    fn = compile_preshuffle_gemm(N=64, K=128, tile_m=32, tile_n=64, tile_k=128, in_dtype="int8")
    cpu = dict(c=torch.zeros(4, 64, dtype=torch.bfloat16), a=torch.zeros(4, 128, dtype=torch.int8),
               b=torch.zeros(64, 128, dtype=torch.int8), sa=torch.zeros(4), sb=torch.zeros(64))
    with pytest.raises(ValueError, match="device"):
        fn(cpu["c"], cpu["a"], cpu["b"], cpu["sa"], cpu["sb"], None, 4, 64, 0)
    with pytest.raises(ValueError, match="N=32 differs"):
        fn(cpu["c"], cpu["a"], cpu["b"], cpu["sa"], cpu["sb"], None, 4, 32, 0)
    with pytest.raises(ValueError, match="outside"):
        fn(cpu["c"], cpu["a"], cpu["b"], cpu["sa"], cpu["sb"], None, 0, 64, 0)

    class Fake:  # stands in for a device tensor
        def __init__(self, numel, esize, contiguous=True, device="cuda:0"):
            self._n, self._e, self._c, self.device, self.is_cuda, self.dtype = numel, esize, contiguous, device, True, "fake"

        def numel(self):
            return self._n

        def element_size(self):
            return self._e

        def is_contiguous(self):
            return self._c

        def data_ptr(self):
            return 0xDEAD0000  # read for the launcher's lookup key only: every case below is refused before any launch

    good = dict(C=Fake(4 * 64, 2), A=Fake(4 * 128, 1), B=Fake(64 * 128, 1), sa=Fake(4, 4), sb=Fake(64, 4))
    for key, bad, msg in [("C", Fake(4 * 64 - 1, 2), "at least"), ("C", Fake(4 * 64, 4), "2"), ("A", Fake(3 * 128, 1), "at least"),
                          ("A", Fake(4 * 128, 1, contiguous=False), "contiguous"), ("B", Fake(64 * 128 + 16, 1), "exactly"),
                          ("sa", Fake(3, 4), "at least"), ("sb", Fake(64, 2), "4"), ("A", Fake(4 * 128, 1, device="cuda:1"), "is on")]:
        ops = dict(good)
        ops[key] = bad
        with pytest.raises(ValueError, match=msg):
            fn(ops["C"], ops["A"], ops["B"], ops["sa"], ops["sb"], None, 4, 64, 0)
    fnb = compile_preshuffle_gemm(N=64, K=128, tile_m=32, tile_n=64, tile_k=128, in_dtype="int8", epilogue="bias")
    with pytest.raises(ValueError, match="bias"):
        fnb(good["C"], good["A"], good["B"], good["sa"], good["sb"], None, 4, 64, 0)
    with pytest.raises(ValueError, match="at least"):
        fnb(good["C"], good["A"], good["B"], good["sa"], good["sb"], Fake(63, 2), 4, 64, 0)
    # the C ABI refuses a misaligned workspace
    handle = _lib.lib()
    args = _lib.A8W8Args()
    args.a = args.b = args.c = args.scale_a = args.scale_b = 0x1000
    args.M, args.N, args.K, args.in_dtype = 64, 64, 128, 0
    args.workspace, args.workspace_bytes = 0x2004, 1 << 20
    assert handle.psg_gemm_a8w8(ctypes.byref(args), None) == -6
    assert b"workspace" in handle.psg_last_error()
    assert handle.psg_static_scratch_bytes() == 32 << 20


def test_rowscale_fp8_entry_points_keep_the_reference_assertions():
    from kernels.gemm.fp8_gemm_4wave import compile_fp8_gemm_4w
    from kernels.gemm.fp8_gemm_8wave import compile_fp8_gemm_8w
    from kernels.gemm.fp8_gemm_utils import preshuffle_b

    with pytest.raises(AssertionError):
        compile_fp8_gemm_8w(K=4096, BLOCK_M=64, BLOCK_N=256)   # 8w needs BLOCK_M >= 128
    with pytest.raises(AssertionError):
        compile_fp8_gemm_8w(K=4096 + 64)                       # K % 128
    with pytest.raises(AssertionError):
        compile_fp8_gemm_4w(K=4096, BLOCK_M=96, BLOCK_N=64)    # BLOCK_M % 64
    fn = compile_fp8_gemm_4w(K=256, BLOCK_M=64, BLOCK_N=64, use_xcd_remap=False, b_preshuffled=True)
    with pytest.raises(ValueError, match="device"):
        fn(torch.zeros(4, 256, dtype=torch.int8), torch.zeros(32, 256, dtype=torch.int8), torch.zeros(4, 32, dtype=torch.bfloat16),
           torch.zeros(4), torch.zeros(32), 4, 32, 0)
    # preshuffle_b is the byte map of shuffle_weight for 1-byte elements
    w = torch.arange(64 * 256, dtype=torch.int32).remainder(251).to(torch.uint8).reshape(64, 256)
    assert torch.equal(preshuffle_b(w).reshape(64, 256), layout.shuffle_weight(w).reshape(64, 256))


def test_int4_packing_against_a_scalar_loop():
    # byte j of every group of 8 values v0..v7 is (v_j & 15) | (v_{j+4} << 4)
    g = torch.Generator().manual_seed(4)
    v = torch.randint(-8, 8, (6, 16), generator=g, dtype=torch.int8)
    got = layout.pack_shuffled_int8_to_int4(v).view(torch.uint8).tolist()
    flat = v.view(-1).tolist()
    want = []
    for base in range(0, len(flat), 8):
        for j in range(4):
            want.append((flat[base + j] & 15) | ((flat[base + j + 4] & 15) << 4))
    assert got == want
    # and back: low nibbles are v0..v3, high nibbles v4..v7, two's complement
    back = []
    for base in range(0, len(got), 4):
        for shift in (0, 4):
            for j in range(4):
                n = (got[base + j] >> shift) & 15
                back.append(n - 16 if n >= 8 else n)
    assert back == flat
    with pytest.raises(ValueError):
        layout.pack_shuffled_int8_to_int4(torch.full((8,), 9, dtype=torch.int8))
    with pytest.raises(ValueError):
        layout.pack_shuffled_int8_to_int4(torch.zeros(12, dtype=torch.int8))


def test_struct_layouts_match_header():
    src = r'''
    #include <stdio.h>
    #include <stddef.h>
    #include "psgemm.h"
    int main(void) {
        printf("%zu %zu %zu %zu %zu %zu %zu\n", sizeof(psg_a8w8_args), offsetof(psg_a8w8_args, workspace_bytes),
               offsetof(psg_a8w8_args, M), offsetof(psg_a8w8_args, epilogue), offsetof(psg_a8w8_args, force_path),
               offsetof(psg_a8w8_args, bias), offsetof(psg_a8w8_args, b_layout));
        printf("%zu %zu %zu %zu %zu %zu %zu %zu\n", sizeof(psg_mxfp4_args), offsetof(psg_mxfp4_args, M), offsetof(psg_mxfp4_args, out_dtype),
               offsetof(psg_mxfp4_args, force_path), offsetof(psg_mxfp4_args, a_dtype), offsetof(psg_mxfp4_args, batch),
               offsetof(psg_mxfp4_args, a_row_stride), offsetof(psg_mxfp4_args, scale_a_batch_stride));
        printf("%zu %zu %zu %zu\n", sizeof(psg_moe_args), offsetof(psg_moe_args, num_valid_ids), offsetof(psg_moe_args, tokens),
               offsetof(psg_moe_args, accumulate));
        printf("%zu %zu %zu %zu\n", sizeof(psg_moe_sort_args), offsetof(psg_moe_sort_args, workspace_bytes), offsetof(psg_moe_sort_args, tokens),
               offsetof(psg_moe_sort_args, blocks));
        printf("%zu %zu %zu %zu\n", sizeof(psg_moe_gating_args), offsetof(psg_moe_gating_args, token_expert_indices),
               offsetof(psg_moe_gating_args, tokens), offsetof(psg_moe_gating_args, renormalize));
        printf("%zu %zu %zu %zu\n", sizeof(psg_moe_mx_args), offsetof(psg_moe_mx_args, num_valid_ids), offsetof(psg_moe_mx_args, tokens),
               offsetof(psg_moe_mx_args, atomic));
        return 0;
    }'''
    with tempfile.TemporaryDirectory() as d:
        c = os.path.join(d, "t.c")
        open(c, "w").write(src)
        exe = os.path.join(d, "t")
        subprocess.run(["gcc", "-std=c99", "-I", os.path.join(ROOT, "include"), c, "-o", exe], check=True)
        out = subprocess.run([exe], check=True, capture_output=True, text=True).stdout.split()
    a, m = _lib.A8W8Args, _lib.MxArgs
    want = [ctypes.sizeof(a), a.workspace_bytes.offset, a.M.offset, a.epilogue.offset, a.force_path.offset, a.bias.offset,
            a.b_layout.offset, ctypes.sizeof(m), m.M.offset, m.out_dtype.offset, m.force_path.offset,
            m.a_dtype.offset, m.batch.offset, m.a_row_stride.offset, m.scale_a_batch_stride.offset]
    e = _lib.MoeArgs
    want += [ctypes.sizeof(e), e.num_valid_ids.offset, e.tokens.offset, e.accumulate.offset]
    so = _lib.MoeSortArgs
    want += [ctypes.sizeof(so), so.workspace_bytes.offset, so.tokens.offset, so.blocks.offset]
    ga = _lib.MoeGatingArgs
    want += [ctypes.sizeof(ga), ga.token_expert_indices.offset, ga.tokens.offset, ga.renormalize.offset]
    mx = _lib.MoeMxArgs
    want += [ctypes.sizeof(mx), mx.num_valid_ids.offset, mx.tokens.offset, mx.atomic.offset]
    assert [int(v) for v in out] == want


def test_mx_moe_validation_errors_without_a_gpu():
    handle = _lib.lib()
    assert handle.psg_moe_mx_gemm(None, None) == -1

    def args(**kw):
        a = _lib.MoeMxArgs()
        for f in ("out", "out_scale", "a", "a_scale", "w", "w_scale", "sorted_token_ids", "sorted_expert_ids", "sorted_weights", "num_valid_ids"):
            setattr(a, f, 0x10000)
        a.tokens, a.experts, a.model_dim, a.inter_dim, a.sorted_size, a.blocks, a.block_m = 8, 2, 512, 256, 128, 4, 32
        a.a_dtype, a.out_dtype, a.stage, a.atomic, a.pad0 = 0, 0, 1, 0, 0
        for k, v in kw.items():
            setattr(a, k, v)
        return a

    bad = [dict(stage=3), dict(block_m=16), dict(block_m=24), dict(block_m=32, a_dtype=3), dict(stage=2, a_dtype=3, block_m=16), dict(model_dim=384), dict(inter_dim=128), dict(a_dtype=1), dict(stage=2, a_dtype=2), dict(stage=2, out_dtype=2),
           dict(blocks=5), dict(blocks=0), dict(tokens=0), dict(experts=0), dict(pad0=1), dict(out_scale=None), dict(stage=2, atomic=1, sorted_weights=None),
           dict(a=0x10008), dict(w=None), dict(sorted_size=16)]
    for kw in bad:
        a = args(**kw)
        assert handle.psg_moe_mx_gemm(ctypes.byref(a), None) != 0, kw
        assert handle.psg_last_error()


def test_mx_scale_sort_validation_errors_without_a_gpu():
    handle = _lib.lib()
    ok = dict(scale=0x1000, ids=0x1000, nv=0x1000, out=0x1000, tokens=4, topk=1, cols=16, rows=64)
    for kw in (dict(scale=None), dict(ids=None), dict(nv=None), dict(out=None), dict(tokens=0), dict(topk=0), dict(topk=256), dict(cols=12), dict(cols=0),
               dict(rows=0), dict(out=0x1002)):
        a = {**ok, **kw}
        assert handle.psg_moe_mx_scale_sort(a["scale"], a["ids"], a["nv"], a["out"], a["tokens"], a["topk"], a["cols"], a["rows"], None) < 0, kw
        assert handle.psg_last_error()


def test_gating_validation_errors_without_a_gpu():
    handle = _lib.lib()
    assert handle.psg_moe_topk_gating(None, None) == -1
    g = _lib.MoeGatingArgs()
    assert handle.psg_moe_topk_gating(ctypes.byref(g), None) == -1 and b"gating" in handle.psg_last_error()
    g.gating = g.weights = g.indices = 0x1000
    g.tokens, g.experts, g.topk, g.dtype, g.renormalize = 4, 128, 6, 1, 1
    for field, val, code, word in (("dtype", 3, -3, b"dtype"), ("tokens", 0, -2, b"tokens"), ("experts", 1025, -2, b"experts"),
                                   ("topk", 33, -2, b"topk"), ("topk", 0, -2, b"topk"), ("renormalize", 2, -2, b"renormalize"),
                                   ("weights", 0x1002, -6, b"aligned"), ("gating", 0x1001, -6, b"aligned"), ("indices", 0, -1, b"indices")):
        old = getattr(g, field)
        setattr(g, field, val)
        assert handle.psg_moe_topk_gating(ctypes.byref(g), None) == code, field
        assert word in handle.psg_last_error(), (field, handle.psg_last_error())
        setattr(g, field, old)
    g.experts, g.topk = 4, 5  # more winners than experts
    assert handle.psg_moe_topk_gating(ctypes.byref(g), None) == -2
    g.experts, g.topk = 128, 6
    # the pair: shapes must agree; beyond the fused range the sorter must read the gating's outputs
    assert handle.psg_moe_softmax_sorting_fused(16, 8, 256) == 1 and handle.psg_moe_softmax_sorting_fused(32, 32, 64) == 1
    assert handle.psg_moe_softmax_sorting_fused(33, 8, 256) == 0 and handle.psg_moe_softmax_sorting_fused(16, 8, 2048) == 0
    assert handle.psg_moe_softmax_sorting_fused(0, 8, 256) == 0
    s = _lib.MoeSortArgs()
    for f in ("sorted_ids", "sorted_weights", "sorted_expert_ids", "num_valid_ids"):
        setattr(s, f, 0x2000)
    s.tokens, s.topk, s.experts, s.block_m = 4, 6, 64, 32
    s.sorted_size, s.blocks = 4 * 6 + 128 * 32, (4 * 6 + 128 * 32 + 31) // 32
    assert handle.psg_moe_softmax_sorting(ctypes.byref(g), None, None) == -1
    assert handle.psg_moe_softmax_sorting(ctypes.byref(g), ctypes.byref(s), None) == -2 and b"disagree" in handle.psg_last_error()
    s.experts = 128
    g.tokens = s.tokens = 100  # two steps: topk_ids / topk_weights missing
    s.sorted_size, s.blocks = 100 * 6 + 128 * 32, (100 * 6 + 128 * 32 + 31) // 32
    assert handle.psg_moe_softmax_sorting(ctypes.byref(g), ctypes.byref(s), None) == -1
    s.topk_ids, s.topk_weights = 0x3000, 0x1000  # ids are not the gating's indices
    assert handle.psg_moe_softmax_sorting(ctypes.byref(g), ctypes.byref(s), None) == -1 and b"indices" in handle.psg_last_error()


def test_validation_errors_come_back_as_codes_without_a_gpu():
    handle = _lib.lib()
    args = _lib.A8W8Args()
    assert handle.psg_gemm_a8w8(ctypes.byref(args), None) == -1  # PSG_E_NULL
    assert b"non-NULL" in handle.psg_last_error()
    args.a = args.b = args.c = args.scale_a = args.scale_b = 0x1000
    args.M, args.N, args.K = 4, 30, 64
    assert handle.psg_gemm_a8w8(ctypes.byref(args), None) == -2  # PSG_E_SHAPE
    args.N, args.K = 32, 100
    assert handle.psg_gemm_a8w8(ctypes.byref(args), None) == -2
    args.K, args.M = 64, 0
    assert handle.psg_gemm_a8w8(ctypes.byref(args), None) == -2
    args.M, args.in_dtype = 4, 7
    assert handle.psg_gemm_a8w8(ctypes.byref(args), None) == -3  # PSG_E_DTYPE
    args.in_dtype, args.a = 1, 0x1001
    assert handle.psg_gemm_a8w8(ctypes.byref(args), None) == -6  # PSG_E_ALIGN
    args.a, args.in_dtype, args.K = 0x1000, 3, 48
    assert handle.psg_gemm_a8w8(ctypes.byref(args), None) == -2  # bf16: K*2 must be a multiple of 64
    with pytest.raises(ValueError):
        _lib.check(-2, "x")
    with pytest.raises(RuntimeError):
        _lib.check(1, "x")


def test_stream_argument_forms():
    assert _lib.stream_handle(0) == 0 and _lib.stream_handle(1234) == 1234

    class S:
        cuda_stream = 77

    assert _lib.stream_handle(S()) == 77
    from flydsl_amd import compiler as flyc
    from flydsl_amd import expr as fx

    assert _lib.stream_handle(fx.Stream(5)) == 5
    p = flyc.from_c_void_p(fx.Uint8, 0xABC0)
    assert p.value == 0xABC0 and int(p) == 0xABC0
    with pytest.raises(TypeError):
        _lib.stream_handle("stream")
    calls = []
    cf = flyc.compile(lambda *a: calls.append(a), 1, 2)
    cf(3, 4)
    assert calls == [(1, 2), (3, 4)]


def test_product_code_does_not_touch_the_oracle():
    bad = []
    for base in ("flydsl_amd", "kernels"):
        for dirpath, _, files in os.walk(os.path.join(ROOT, base)):
            for f in files:
                if f.endswith((".py", ".hip", ".h", ".cpp")):
                    text = open(os.path.join(dirpath, f)).read()
                    if re.search(r"^\s*(from|import)\s+oracle\b", text, flags=re.M) or "psg_oracle" in text:
                        bad.append(os.path.join(dirpath, f))
    assert not bad, bad


def test_compat_aliases_install_and_do_not_shadow():
    import flydsl_amd.compat as compat

    added = compat.install()
    try:
        import flydsl.compiler as flyc
        from tests.kernels.utils import gemm_common_utils
        from tests.test_common import verify_output
        from tests.utils import pertoken_quant, shuffle_weight

        assert flyc.compile is __import__("flydsl_amd.compiler", fromlist=["compile"]).compile
        assert pertoken_quant is quant.pertoken_quant and shuffle_weight is layout.shuffle_weight
        assert gemm_common_utils.shuffle_scale_w4 is layout.shuffle_scale_w4
        ref = torch.ones(10, 100)
        out = ref.clone()
        out[0, :40] += 1.0
        assert verify_output(out, ref, atol=0.1, rtol=0.1)
        out[0:2] += 1.0
        assert not verify_output(out, ref, atol=0.1, rtol=0.1)
        assert compat.install() == []  # second call adds nothing
    finally:
        for name in added:
            sys.modules.pop(name, None)
