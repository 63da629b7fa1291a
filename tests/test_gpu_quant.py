"""GPU parity of the on-device activation quantisers against the CPU oracle: byte-for-byte (integer / bit-pattern
work), including rows with NaN / Inf / all zeros, long rows, 16-bit inputs, ragged M for the MX scale padding, and
an end-to-end quantise -> GEMM run on the device."""

import numpy as np
import pytest
import torch

from oracle import psg_oracle as O

pytestmark = pytest.mark.gpu


def _x(m, k, seed, spread=True):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(m, k, generator=g)
    if spread:
        x = x * torch.logspace(-4, 4, m).view(-1, 1)
    return x


@pytest.mark.parametrize("qd,kind", [(torch.int8, "int8"), (torch.float8_e4m3fn, "fp8")])
@pytest.mark.parametrize("m,k", [(1, 64), (16, 4096), (33, 8192), (5, 24576), (300, 1032)])
def test_pertoken_quant_device_bit_exact(qd, kind, m, k):
    from flydsl_amd import quant_device

    x = _x(m, k, seed=m + k)
    if m > 3:
        x[1] = 0.0
        x[2, 5] = float("nan")
        x[3, 7] = float("inf")
        x[3, 9] = float("-inf")
    y, s = quant_device.pertoken_quant(x.cuda(), quant_dtype=qd)
    torch.cuda.synchronize()
    want_y, want_s = O.pertoken_quant(x.numpy(), kind)
    assert s.shape == (m, 1)
    assert np.array_equal(s.cpu().numpy(), want_s)
    assert np.array_equal(y.view(torch.uint8).cpu().numpy(), want_y.view(np.uint8))


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16])
def test_pertoken_quant_device_16bit_inputs(dt):
    from flydsl_amd import quant_device

    x = _x(40, 2048, seed=3, spread=False).to(dt)
    for qd, kind in ((torch.int8, "int8"), (torch.float8_e4m3fn, "fp8")):
        y, s = quant_device.pertoken_quant(x.cuda(), quant_dtype=qd)
        want_y, want_s = O.pertoken_quant(x.float().numpy(), kind)
        assert np.array_equal(s.cpu().numpy(), want_s)
        assert np.array_equal(y.view(torch.uint8).cpu().numpy(), want_y.view(np.uint8))


def test_fp8_encoder_on_every_midpoint():
    # rows built so that after division by the row scale (row max = 448 -> scale exactly 1) the values sit on
    # every e4m3 code, every midpoint between adjacent codes and their neighbours
    from flydsl_amd import quant_device

    table = O.e4m3fn_to_f32(np.arange(0x7F, dtype=np.uint8)).astype(np.float64)
    mids = (table[:-1] + table[1:]) / 2
    pts = np.concatenate([table, mids, np.nextafter(mids.astype(np.float32), np.float32(np.inf)),
                          np.nextafter(mids.astype(np.float32), np.float32(-np.inf))]).astype(np.float32)
    pts = np.concatenate([pts, -pts])
    k = (len(pts) + 1 + 7) // 8 * 8
    row = np.zeros(k, np.float32)
    row[: len(pts)] = pts
    row[-1] = 448.0
    x = torch.from_numpy(row).view(1, -1)
    y, s = quant_device.pertoken_quant(x.cuda(), quant_dtype=torch.float8_e4m3fn)
    assert s.item() == 1.0
    assert np.array_equal(y.view(torch.uint8).cpu().numpy()[0], O.f32_to_e4m3fn(row))


@pytest.mark.parametrize("m,k", [(1, 256), (32, 2048), (45, 512), (4096, 2048)])
@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
def test_mxfp4_quant_device_bit_exact(m, k, dt):
    from flydsl_amd import quant_device

    x = (_x(m, k, seed=7, spread=m <= 64) if m <= 64 else _x(m, k, seed=7, spread=False)).to(dt)
    if m > 2:
        x[2, 32:64] = 0.0
    r = (m + 31) // 32 * 32
    xp = np.zeros((r, k), np.float32)
    xp[:m] = x.float().numpy()
    want_p, want_s = O.per_1x32_f4_quant(xp)
    p, s = quant_device.per_1x32_f4_quant(x.cuda(), shuffle=False)
    assert np.array_equal(p.view(torch.uint8).cpu().numpy(), want_p[:m])
    assert np.array_equal(s.view(torch.uint8).cpu().numpy(), want_s)
    p2, s2 = quant_device.per_1x32_f4_quant(x.cuda(), shuffle=True)
    assert np.array_equal(p2.view(torch.uint8).cpu().numpy(), want_p[:m])
    assert np.array_equal(s2.view(torch.uint8).cpu().numpy(), O.shuffle_scale_w4(want_s))


def test_e2m1_encoder_on_every_midpoint():
    from flydsl_amd import quant_device

    # a block whose maximum is 4 gets scale byte 127 (amax/4 = 1.0), so codes are taken of the values themselves
    vals = np.array([0.0, 0.25, 0.5, 0.75, 1.0, 1.25, 1.5, 1.75, 2.0, 2.5, 3.0, 3.5, 4.0, 0.2499, 0.2501, 0.7499, 0.7501,
                     1.2499, 1.2501, 1.7499, 1.7501, 2.4999, 2.5001, 3.4999, 3.5001, -0.25, -0.75, -1.25, -2.5, -3.5, -4.0, -0.0],
                    np.float32)
    x = torch.from_numpy(np.tile(vals, 8)).view(1, 256)
    p, s = quant_device.per_1x32_f4_quant(x.cuda(), shuffle=False)
    want_p, want_s = O.per_1x32_f4_quant(np.vstack([x.numpy(), np.zeros((31, 256), np.float32)]))
    assert (s.view(torch.uint8).cpu().numpy()[0] == 127).all()
    assert np.array_equal(p.view(torch.uint8).cpu().numpy(), want_p[:1])


def test_quantise_then_gemm_on_device():
    from flydsl_amd import layout, quant, quant_device
    from kernels.gemm.preshuffle_gemm import compile_preshuffle_gemm

    M, N, K = 48, 512, 1024
    x = _x(M, K, seed=11, spread=False)
    g = torch.Generator().manual_seed(12)
    w = torch.randn(N, K, generator=g) * 0.02
    b_q, sb = quant.pertoken_quant(w, quant_dtype=torch.float8_e4m3fn)
    dev = torch.device("cuda")
    a_q, sa = quant_device.pertoken_quant(x.to(dev), quant_dtype=torch.float8_e4m3fn)
    fn = compile_preshuffle_gemm(N=N, K=K, tile_m=64, tile_n=256, tile_k=128, in_dtype="fp8")
    c = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
    fn(c, a_q, layout.shuffle_weight(b_q).to(dev), sa.view(-1), sb.view(-1).to(dev), torch.empty(0, dtype=torch.bfloat16, device=dev),
       M, N, torch.cuda.current_stream())
    torch.cuda.synchronize()
    aq_h, sa_h = O.pertoken_quant(x.numpy(), "fp8")
    ref = O.run_torch(aq_h, b_q.view(torch.uint8).numpy(), sa_h, sb.numpy(), "fp8")
    ok, ratio = O.within_north_star_tolerance(c.float().cpu().numpy(), ref)
    assert ok, ratio


def test_quantiser_argument_errors():
    from flydsl_amd import quant_device

    with pytest.raises(ValueError):
        quant_device.pertoken_quant(torch.zeros(4, 12, device="cuda"))  # K % 8
    with pytest.raises(ValueError):
        quant_device.per_1x32_f4_quant(torch.zeros(4, 48, device="cuda"), shuffle=False)  # K % 32
    with pytest.raises(ValueError):
        quant_device.per_1x32_f4_quant(torch.zeros(4, 64, device="cuda"), shuffle=True)  # K % 256 for the shuffled layout
    with pytest.raises(TypeError):
        quant_device.pertoken_quant(torch.zeros(4, 64, device="cuda", dtype=torch.float64))


def test_quantisers_with_caller_owned_outputs():
    from flydsl_amd import quant_device

    x = _x(64, 512, seed=9, spread=False).cuda()
    y = torch.empty(64, 512, dtype=torch.uint8, device="cuda")
    s = torch.empty(64, dtype=torch.float32, device="cuda")
    y2, s2 = quant_device.pertoken_quant(x, quant_dtype=torch.float8_e4m3fn, out=(y, s))
    ref_y, ref_s = quant_device.pertoken_quant(x, quant_dtype=torch.float8_e4m3fn)
    assert y2.data_ptr() == y.data_ptr() and torch.equal(y2.view(torch.uint8), ref_y.view(torch.uint8)) and torch.equal(s.view(-1, 1), ref_s)
    p = torch.empty(64, 256, dtype=torch.uint8, device="cuda")
    sc = torch.empty(64, 16, dtype=torch.uint8, device="cuda")
    quant_device.per_1x32_f4_quant(x, shuffle=False, out=(p, sc))
    rp, rs = quant_device.per_1x32_f4_quant(x, shuffle=False)
    assert torch.equal(p, rp.view(torch.uint8)) and torch.equal(sc, rs.view(torch.uint8))
    with pytest.raises(ValueError):
        quant_device.pertoken_quant(x, out=(y[:10], s))


@pytest.mark.parametrize("qd,kind", [(torch.int8, "int8"), (torch.float8_e4m3fn, "fp8")])
def test_pertoken_quant_division_is_exact_over_many_values(qd, kind):
    # 33 M quotients with row scales from 2^-80 to 2^80 (both the fast per-row-reciprocal path and the plain
    # division for extreme rows), compared byte for byte with the oracle's IEEE division
    from flydsl_amd import quant_device

    g = torch.Generator().manual_seed(77)
    m, k = 4096, 8192
    x = torch.randn(m, k, generator=g) * torch.pow(2.0, torch.linspace(-80, 80, m)).view(-1, 1)
    x[:, 0] = x.abs().amax(dim=1)  # make sure the row maximum is hit exactly once more
    y, s = quant_device.pertoken_quant(x.cuda(), quant_dtype=qd)
    want_y, want_s = O.pertoken_quant(x.numpy(), kind)
    assert np.array_equal(s.cpu().numpy(), want_s)
    got = y.view(torch.uint8).cpu().numpy()
    bad = np.argwhere(got != want_y.view(np.uint8))
    assert len(bad) == 0, (len(bad), bad[:5].tolist())
