"""Pins of the oracle's quantisers and GEMM routines: closed-form invariants, float64 / pure-integer
cross-checks on small inputs, and library routines for the activations."""

import numpy as np
import torch
import torch.nn.functional as F

from oracle import psg_oracle as O


def _data(m=12, n=40, k=96, seed=0):
    rng = np.random.default_rng(seed)
    return rng.standard_normal((m, k)).astype(np.float32), (rng.standard_normal((n, k)) * 0.02).astype(np.float32)


def test_pertoken_quant_int8_invariants():
    x, _ = _data()
    x[3] = 0.0  # all-zero row
    x[5, 7] = np.nan
    x[6, 2] = np.inf
    q, s = O.pertoken_quant(x, "int8")
    assert q.dtype == np.int8 and s.shape == (x.shape[0], 1) and s.dtype == np.float32
    assert s[3, 0] == 1.0 and not q[3].any()
    assert q[5, 7] == 0  # NaN -> 0
    assert q[6, 2] == 127 and s[6, 0] == 1.0  # +Inf clamped to dtypeMax -> amax = 127 -> scale 1
    clean = np.nan_to_num(x, nan=0.0, posinf=127.0, neginf=-127.0)
    for r in range(x.shape[0]):
        if r == 3:
            continue
        assert np.abs(q[r]).max() in (126, 127)  # the row maximum maps to +-127 up to one fp32 rounding
        # truncation toward zero: |x| - |q*s| in [0, s)
        err = np.abs(clean[r]) - np.abs(q[r].astype(np.float32) * s[r, 0])
        assert (err > -1e-6 * s[r, 0] * 127).all() and (err < s[r, 0] * (1 + 1e-5)).all()
    assert np.trunc(np.float32(1.5)) == 1 and O.pertoken_quant(np.array([[1.5, -1.5, 127.0]], np.float32), "int8")[0].tolist() == [[1, -1, 127]]


def test_pertoken_quant_matches_library_ops():
    x, w = _data(seed=4)
    for kind, qd in (("int8", torch.int8), ("fp8", torch.float8_e4m3fn)):
        for arr in (x, w):
            t = torch.from_numpy(arr)
            amax = torch.maximum(t.amax(-1, keepdim=True), -t.amin(-1, keepdim=True))
            sc = amax / (127.0 if kind == "int8" else 448.0)
            want_q = (t / sc).to(qd).view(torch.uint8).numpy()
            q, s = O.pertoken_quant(arr, kind)
            assert np.array_equal(s, sc.numpy())
            assert np.array_equal(q.view(np.uint8), want_q)


def test_pertoken_quant_fp8_error_bound():
    x, _ = _data(seed=5)
    q, s = O.pertoken_quant(x, "fp8")
    deq = O.e4m3fn_to_f32(q) * s
    # half an ulp of e4m3 is 2^-4 relative for normals; subnormal spacing 2^-9 in scaled units
    assert (np.abs(deq - x) <= np.maximum(np.abs(x) * 2.0**-4, s * 2.0**-10) * (1 + 1e-5)).all()
    assert np.abs(O.e4m3fn_to_f32(q)).max() == 448.0


def test_int32_accumulators_against_integer_loops():
    rng = np.random.default_rng(6)
    a = rng.integers(-127, 128, (5, 70), dtype=np.int8)
    b = rng.integers(-127, 128, (9, 70), dtype=np.int8)
    want = np.zeros((5, 9), dtype=np.int64)
    for i in range(5):
        for j in range(9):
            for t in range(70):
                want[i, j] += int(a[i, t]) * int(b[j, t])
    assert np.array_equal(O.int32_accumulators(a, b), want.astype(np.int32))
    # extreme: K large enough that a float32 accumulation would lose bits
    a = np.full((1, 40000), 127, np.int8)
    b = np.full((1, 40000), -127, np.int8)
    assert O.int32_accumulators(a, b)[0, 0] == -127 * 127 * 40000


def test_run_torch_against_float64():
    x, w = _data(seed=7)
    for kind in ("int8", "fp8"):
        aq, sa = O.pertoken_quant(x, kind)
        bq, sb = O.pertoken_quant(w, kind)
        a64 = (aq.astype(np.float64) if kind == "int8" else O.e4m3fn_to_f32(aq).astype(np.float64)) * sa.astype(np.float64)
        b64 = (bq.astype(np.float64) if kind == "int8" else O.e4m3fn_to_f32(bq).astype(np.float64)) * sb.astype(np.float64)
        want = a64 @ b64.T
        got = O.run_torch(aq, bq, sa, sb, kind)
        assert np.allclose(got, want, rtol=1e-5, atol=1e-6)
        # transposed operands or a dropped scale would not survive this
        assert not np.allclose(got, (a64 / sa) @ b64.T, rtol=1e-3)
        bias = np.linspace(-1, 1, w.shape[0]).astype(np.float32)
        assert np.allclose(O.run_torch(aq, bq, sa, sb, kind, bias=bias), want + bias, rtol=1e-5, atol=1e-6)


def test_per_1x32_f4_quant_invariants():
    rng = np.random.default_rng(8)
    x = (rng.standard_normal((8, 256)) * rng.choice([1e-4, 1.0, 50.0], (8, 1))).astype(np.float32)
    x[2, 32:64] = 0.0  # an all-zero block
    packed, sc = O.per_1x32_f4_quant(x)
    assert packed.shape == (8, 128) and sc.shape == (8, 8) and packed.dtype == np.uint8
    assert sc[2, 1] == 0 and not packed[2, 16:32].any()
    deq = O.mxfp4_to_f32(packed) * np.repeat(O.e8m0_to_f32(sc), 32, axis=1)
    scale = np.repeat(O.e8m0_to_f32(sc), 32, axis=1).astype(np.float64)
    y = np.abs(x.astype(np.float64)) / scale
    # the scale puts the block maximum in (2, 6]: amax/4 rounded to a power of two within [2/3, 4/3) of it... so
    blk_max = np.abs(x).reshape(8, 8, 32).max(-1)
    ratio = blk_max[sc > 0] / O.e8m0_to_f32(sc)[sc > 0]
    assert (ratio > 2.0 * (1 - 1e-6)).all() and (ratio <= 6.0 * (1 + 1e-6)).all()
    # nearest-value rounding: error at most half the local e2m1 step (0.25 below 2, 0.5 in [2,4), 1 in [4,6])
    half_step = np.where(y < 2, 0.25, np.where(y < 4, 0.5, 1.0))
    assert (np.abs(np.abs(deq.astype(np.float64)) / scale - y) <= half_step + 1e-9).all()
    assert (np.sign(deq) * np.sign(x) >= 0).all()


def test_run_torch_w4_against_float64():
    rng = np.random.default_rng(9)
    x = rng.standard_normal((6, 128)).astype(np.float32)
    w = (rng.standard_normal((10, 128)) * 0.02).astype(np.float32)
    ap, sa = O.per_1x32_f4_quant(x)
    bp, sb = O.per_1x32_f4_quant(w)
    lut = [0, .5, 1, 1.5, 2, 3, 4, 6, -0.0, -.5, -1, -1.5, -2, -3, -4, -6]
    want = np.zeros((6, 10))
    for i in range(6):
        for j in range(10):
            for t in range(128):
                av = lut[(ap[i, t // 2] >> (4 * (t % 2))) & 15] * 2.0 ** (int(sa[i, t // 32]) - 127)
                bv = lut[(bp[j, t // 2] >> (4 * (t % 2))) & 15] * 2.0 ** (int(sb[j, t // 32]) - 127)
                want[i, j] += av * bv
    assert np.allclose(O.run_torch_w4(ap, bp, sa, sb), want, rtol=1e-5, atol=1e-7)


def test_per_1x32_f6_quant_invariants():
    rng = np.random.default_rng(18)
    x = (rng.standard_normal((8, 256)) * rng.choice([1e-4, 1.0, 50.0], (8, 1))).astype(np.float32)
    x[2, 32:64] = 0.0
    a_pad, sc, codes = O.per_1x32_f6_quant(x)
    assert a_pad.shape == (8, 256) and sc.shape == (8, 8) and codes.shape == (8, 256)
    assert not a_pad.reshape(8, 8, 32)[:, :, 24:].any()  # the 8 padding bytes are zero
    assert np.array_equal(O.unpack_fp6_padded(a_pad), codes)
    assert sc[2, 1] == 0 and not codes[2, 32:64].any()
    scale = np.repeat(O.e8m0_to_f32(sc), 32, axis=1).astype(np.float64)
    y = np.abs(x.astype(np.float64)) / scale
    blk_max = np.abs(x).reshape(8, 8, 32).max(-1)
    ratio = blk_max[sc > 0] / O.e8m0_to_f32(sc)[sc > 0]
    assert (ratio > 2.0 * (1 - 1e-6)).all() and (ratio <= 6.0 * (1 + 1e-6)).all()  # same scale rule as fp4 (amax / 4)
    deq = np.abs(O.e2m3_to_f32(codes).astype(np.float64))
    half_step = np.where(y < 2, 0.0625, np.where(y < 4, 0.125, 0.25))
    assert (np.abs(deq - y) <= half_step + 1e-9).all()  # never saturates: the block maximum is <= 6 < 7.5
    assert (np.sign(O.e2m3_to_f32(codes)) * np.sign(x) >= 0).all()


def test_per_1x32_f8_quant_invariants():
    rng = np.random.default_rng(19)
    x = (rng.standard_normal((8, 256)) * rng.choice([1e-4, 1.0, 50.0], (8, 1))).astype(np.float32)
    x[2, 32:64] = 0.0
    q, sc = O.per_1x32_f8_quant(x)
    assert q.shape == (8, 256) and q.dtype == np.uint8 and sc.shape == (8, 8)
    assert not (q[2, 32:64] & 0x7F).any()
    # amax / 448 rounded to a power of two: the scaled block maximum lies in (448 * 2/3, 448 * 4/3]; what exceeds 448
    # is clamped, so no code is NaN and every magnitude is at most 448
    assert ((q & 0x7F) != 0x7F).all()
    dec = O.e4m3fn_to_f32(q)
    assert np.abs(dec).max() <= 448.0
    sf = np.repeat(O.e8m0_to_f32(sc), 32, axis=1).astype(np.float64)
    y = x.astype(np.float64) / sf
    inside = (np.abs(y) <= 448) & (np.abs(y) >= 2.0**-6)
    assert (np.abs(dec[inside] - y[inside]) <= np.abs(y[inside]) * 2.0**-4 + 1e-12).all()  # half an e4m3 step
    clamped = np.abs(y) > 448
    assert (np.abs(dec[clamped]) == 448).all()
    # scale bytes by hand for two blocks: amax = 448 -> 2^0 (byte 127); amax = 3 -> 3/448 = 1.714 * 2^-8 -> rounds up to 2^-7
    t = np.zeros((1, 64), dtype=np.float32)
    t[0, 0], t[0, 32] = 448.0, 3.0
    q2, s2 = O.per_1x32_f8_quant(t)
    assert s2.tolist() == [[127, 120]] and q2[0, 0] == 0x7E and O.e4m3fn_to_f32(q2[:, 32])[0] == 384.0


def test_run_torch_mx_against_float64():
    rng = np.random.default_rng(20)
    x = rng.standard_normal((5, 64)).astype(np.float32)
    w = (rng.standard_normal((7, 64)) * 0.02).astype(np.float32)
    a6, sa6, c6 = O.per_1x32_f6_quant(x)
    a8, sa8 = O.per_1x32_f8_quant(x)
    b4, sb4 = O.per_1x32_f4_quant(w)
    b8, sb8 = O.per_1x32_f8_quant(w)
    e2m3 = np.concatenate([[(m / 8.0) if e == 0 else (2.0 ** (e - 1)) * (1 + m / 8.0) for e in range(4) for m in range(8)]] * 2)
    e2m3[32:] *= -1
    e2m1 = np.array([0, .5, 1, 1.5, 2, 3, 4, 6, -0.0, -.5, -1, -1.5, -2, -3, -4, -6])
    e4m3 = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).double().numpy()

    def val(q, s, fmt, i, t):
        if fmt == "fp4":
            v = e2m1[(q[i, t // 2] >> (4 * (t % 2))) & 15]
        elif fmt == "fp6":  # bits [6j, 6j+6) of the 24-byte group
            grp = int.from_bytes(q[i, 32 * (t // 32): 32 * (t // 32) + 24].tobytes(), "little")
            v = e2m3[(grp >> (6 * (t % 32))) & 63]
        else:
            v = e4m3[q[i, t]]
        return v * 2.0 ** (int(s[i, t // 32]) - 127)

    for (aq, sa, af), (bq, sb, bf) in [((a6, sa6, "fp6"), (b4, sb4, "fp4")), ((a8, sa8, "fp8"), (b8, sb8, "fp8")),
                                       ((a8, sa8, "fp8"), (b4, sb4, "fp4")), ((a6, sa6, "fp6"), (b8, sb8, "fp8"))]:
        want = np.array([[sum(val(aq, sa, af, i, t) * val(bq, sb, bf, j, t) for t in range(64)) for j in range(7)] for i in range(5)])
        assert np.allclose(O.run_torch_mx(aq, bq, sa, sb, af, bf), want, rtol=1e-5, atol=1e-7)
    a4, sa4 = O.per_1x32_f4_quant(x)
    assert np.array_equal(O.run_torch_mx(a4, b4, sa4, sb4), O.run_torch_w4(a4, b4, sa4, sb4))


def test_activations_against_library():
    v = np.linspace(-12, 12, 4001).astype(np.float32).reshape(1, -1)
    t = torch.from_numpy(v)
    assert np.array_equal(O.apply_bias_act(v, None, "relu"), F.relu(t).numpy())
    assert np.allclose(O.apply_bias_act(v, None, "silu"), F.silu(t).numpy(), rtol=1e-5, atol=1e-6)
    assert np.allclose(O.apply_bias_act(v, None, "gelu"), F.gelu(t, approximate="tanh").numpy(), rtol=1e-5, atol=2e-6)
    big = np.array([[-1e4, 1e4, -90.0, 90.0]], np.float32)  # overflow-safe forms stay finite
    assert np.isfinite(O.apply_bias_act(big, None, "gelu")).all() and np.isfinite(O.apply_bias_act(big, None, "silu")).all()
    bias = np.full(v.shape[1], 0.5, np.float32)
    assert np.array_equal(O.apply_bias_act(v, bias, "none"), v + 0.5)


def test_epilogue_order_is_acc_times_sa_then_sb():
    acc = np.array([[3, -7]], np.int32)
    sa = np.array([0.1], np.float32)
    sb = np.array([3.0, 1e-3], np.float32)
    want = (np.float32(acc) * sa[:, None]).astype(np.float32) * sb[None, :]
    assert np.array_equal(O.epilogue_a8w8(acc, sa, sb), want.astype(np.float32))


def test_verify_output_rule():
    ref = np.ones((10, 100), np.float32)
    out = ref.copy()
    out[0, :40] += 1.0  # 4 % of elements off by a lot: passes the 5 % rule
    assert O.verify_output(out, ref, atol=0.1, rtol=0.1)
    out[0:2, :] += 1.0  # 20 % off and a large cosine-style distance: fails
    assert not O.verify_output(out, ref, atol=0.1, rtol=0.1)
    assert O.logits_diff(ref, ref) == 0.0 and O.logits_diff(np.zeros(3), np.zeros(3)) == 0.0
    ok, ratio = O.within_north_star_tolerance(ref * 1.005, ref)
    assert ok and 0.2 < ratio < 0.3
    assert not O.within_north_star_tolerance(ref * 1.03, ref)[0]
