"""Pins of the oracle's codecs.  The reference holds no golden vectors for this path, so each codec is
checked against something independent of its own formula: a library cast, an exhaustive table, or a
brute-force nearest-value search."""

import numpy as np
import torch

from oracle import psg_oracle as O


def test_e4m3fn_decode_matches_library_cast_on_all_codes():
    codes = torch.arange(256, dtype=torch.uint8)
    want = codes.view(torch.float8_e4m3fn).to(torch.float32).numpy()
    got = O.e4m3fn_to_f32(codes.numpy())
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert np.array_equal(got[~np.isnan(got)], want[~np.isnan(want)])
    assert np.isnan(got[0x7F]) and np.isnan(got[0xFF]) and got[0x7E] == 448.0


def _e4m3_sweep():
    table = O.e4m3fn_to_f32(np.arange(0x7F, dtype=np.uint8)).astype(np.float64)  # positive finite codes, ascending
    mids = (table[:-1] + table[1:]) / 2
    eps = np.concatenate([np.nextafter(mids.astype(np.float32), np.float32(np.inf)),
                          np.nextafter(mids.astype(np.float32), np.float32(-np.inf))])
    rng = np.random.default_rng(1)
    rand = (rng.standard_normal(20000) * rng.choice([1e-3, 0.1, 1, 30, 200], 20000)).astype(np.float32)
    pos = np.concatenate([table, mids, eps, [0.0, 448.0, 463.9, 464.0]]).astype(np.float32)
    return np.concatenate([pos, -pos, rand]).astype(np.float32)


def test_f32_to_e4m3fn_matches_library_cast_including_every_midpoint():
    x = _e4m3_sweep()
    want = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = O.f32_to_e4m3fn(x)
    nan_w = (want & 0x7F) == 0x7F
    nan_g = (got & 0x7F) == 0x7F
    assert np.array_equal(nan_w, nan_g)
    assert np.array_equal(got[~nan_g], want[~nan_w])


def test_e8m0_decode_all_bytes():
    b = np.arange(256, dtype=np.uint8)
    got = O.e8m0_to_f32(b)
    for i in range(1, 255):
        assert got[i] == np.ldexp(np.float32(1.0), i - 127)
    assert got.view(np.uint32)[0] == 0x00400000 and got[0] == np.float32(2.0) ** -127
    assert np.isnan(got[255])


def test_f32_to_e8m0_known_answers():
    # (value, expected byte): exponent of the value, +1 when the mantissa is >= 1.5
    cases = [(1.0, 127), (1.25, 127), (np.nextafter(np.float32(1.5), np.float32(0)), 127), (1.5, 128), (1.75, 128),
             (2.0, 128), (3.0, 129), (0.5, 126), (0.75, 127), (2.0**-126, 1), (1.5 * 2.0**-126, 2), (2.0**127, 254),
             (0.0, 0), (2.0**-127, 0), (2.0**-127 + 2.0**-128, 1), (2.0**-127 + 2.0**-149, 1), (2.0**-128, 0)]
    x = np.array([c[0] for c in cases], dtype=np.float32)
    want = np.array([c[1] for c in cases], dtype=np.uint8)
    assert np.array_equal(O.f32_to_e8m0(x), want)
    assert O.f32_to_e8m0(np.array([np.nan, np.inf], dtype=np.float32)).tolist() == [255, 255]
    # the increment wraps in 8 bits like the reference's uint8 arithmetic
    assert O.f32_to_e8m0(np.array([1.5 * 2.0**127], dtype=np.float32))[0] == 255


def _nearest_e2m1_bruteforce(x):
    """Independent statement of e2m1 rounding: nearest of the 8 magnitudes, ties to the even mantissa bit
    (codes 0,2,4,6 have mantissa 0), saturating; sign kept."""
    mags = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0])
    out = np.zeros(x.shape, dtype=np.uint8)
    for i, v in enumerate(x.astype(np.float64)):
        a = abs(v)
        d = np.abs(mags - a)
        best = np.flatnonzero(d == d.min())
        code = best[0] if len(best) == 1 else [c for c in best if c % 2 == 0][0]
        if a >= 6.0:
            code = 7
        out[i] = code | (8 if np.signbit(np.float32(v)) else 0)
    return out


def test_f32_to_e2m1_matches_bruteforce_nearest_even():
    mags = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0], dtype=np.float32)
    mids = (mags[:-1] + mags[1:]) / 2
    near = np.concatenate([np.nextafter(mids, np.float32(np.inf)), np.nextafter(mids, np.float32(-np.inf))])
    rng = np.random.default_rng(2)
    x = np.concatenate([mags, mids, near, [6.0, 6.5, 100.0, 1e-8, 0.2499, 5.9999], rng.uniform(0, 7, 4000)]).astype(np.float32)
    x = np.concatenate([x, -x])
    assert np.array_equal(O.f32_to_e2m1(x), _nearest_e2m1_bruteforce(x))
    # every midpoint, spelled out: 0.25->0, 0.75->1, 1.25->1, 1.75->2, 2.5->2, 3.5->4, 5->4
    got = O.E2M1_LUT[O.f32_to_e2m1(mids)]
    assert got.tolist() == [0.0, 1.0, 1.0, 2.0, 2.0, 4.0, 4.0]


def test_pack_and_decode_nibble_order():
    codes = np.array([[0x3, 0xA]], dtype=np.uint8)  # element 0 = 1.5, element 1 = -1.0
    packed = O.pack_uint4(codes)
    assert packed.tolist() == [[0xA3]]  # even index in the low nibble
    assert O.mxfp4_to_f32(packed).tolist() == [[1.5, -1.0]]
    allcodes = O.pack_uint4(np.arange(16, dtype=np.uint8).reshape(1, 16))
    assert O.mxfp4_to_f32(allcodes).tolist() == [[0, .5, 1, 1.5, 2, 3, 4, 6, -0.0, -.5, -1, -1.5, -2, -3, -4, -6]]


def test_bf16_rounding_matches_library_cast():
    rng = np.random.default_rng(3)
    x = (rng.standard_normal(50000) * rng.choice([1e-20, 1e-3, 1, 1e5, 1e30], 50000)).astype(np.float32)
    ties = (np.arange(1, 2000, dtype=np.uint32) << 16 | 0x8000).view(np.float32)  # exact halfway cases
    x = np.concatenate([x, ties, -ties, [0.0, -0.0, np.inf, -np.inf]]).astype(np.float32)
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(O.f32_to_bf16_bits(x), want)
    assert np.array_equal(O.bf16_bits_to_f32(want), torch.from_numpy(x).to(torch.bfloat16).float().numpy())


def _e2m3_magnitudes():
    """The format's definition, stated with Fractions-free float64 arithmetic: exponent field 0 is subnormal (m/8),
    otherwise 2^(e-1) * (1 + m/8)."""
    return np.array([(m / 8.0) if e == 0 else (2.0 ** (e - 1)) * (1 + m / 8.0) for e in range(4) for m in range(8)])


def test_e2m3_decode_all_codes():
    mags = _e2m3_magnitudes()
    assert mags[0] == 0 and mags[1] == 0.125 and mags[8] == 1.0 and mags[31] == 7.5 and (np.diff(mags) > 0).all()
    want = np.concatenate([mags, -mags]).astype(np.float32)
    got = O.e2m3_to_f32(np.arange(64, dtype=np.uint8))
    assert np.array_equal(got, want) and np.signbit(got[32])
    assert np.array_equal(O.e2m3_to_f32(np.arange(64, 256, dtype=np.uint8)), O.e2m3_to_f32(np.arange(64, 256, dtype=np.uint8) & 0x3F))


def test_f32_to_e2m3_matches_bruteforce_nearest_even():
    mags = _e2m3_magnitudes()
    mids = ((mags[:-1] + mags[1:]) / 2).astype(np.float32)
    near = np.concatenate([np.nextafter(mids, np.float32(np.inf)), np.nextafter(mids, np.float32(-np.inf))])
    rng = np.random.default_rng(12)
    x = np.concatenate([mags, mids, near, [7.5, 7.75, 8.0, 100.0, 1e-8, 0.0624, 0.0626], rng.uniform(0, 8, 6000)]).astype(np.float32)
    x = np.concatenate([x, -x])
    want = np.zeros(x.shape, dtype=np.uint8)
    for i, v in enumerate(x.astype(np.float64)):
        a = abs(v)
        d = np.abs(mags - a)
        best = np.flatnonzero(d == d.min())
        code = best[0] if len(best) == 1 else [c for c in best if c % 2 == 0][0]  # tie -> even mantissa
        if a >= 7.5:
            code = 31
        want[i] = code | (32 if np.signbit(np.float32(v)) else 0)
    assert np.array_equal(O.f32_to_e2m3(x), want)
    # the generic encoder with (2, 1) is the e2m1 encoder pinned above
    assert np.array_equal(O.f32_to_floatx(x, 2, 1), O.f32_to_e2m1(x))


def test_pack_fp6_against_bit_string():
    rng = np.random.default_rng(13)
    codes = rng.integers(0, 64, (3, 64), dtype=np.uint8)
    packed = O.pack_fp6(codes)
    assert packed.shape == (3, 48)
    for r in range(3):
        big = 0
        for j, c in enumerate(codes[r].tolist()):
            big |= c << (6 * j)  # element j at bits [6j, 6j+6) of one long little-endian integer
        assert packed[r].tobytes() == big.to_bytes(48, "little")
    # the spelled-out example of the reference's docstring: b0 = e1[1:0]<<6 | e0, b1 = e2[3:0]<<4 | e1>>2, b2 = e3<<2 | e2>>4
    e = [0b101011, 0b110110, 0b011101, 0b100001]
    assert O.pack_fp6(np.array([e], dtype=np.uint8)).tolist() == [[((e[1] & 3) << 6) | e[0], ((e[2] & 15) << 4) | (e[1] >> 2), (e[3] << 2) | (e[2] >> 4)]]
    # padded layout round trip (24 packed + 8 padding bytes per 32 elements)
    pad = np.zeros((3, 2, 32), dtype=np.uint8)
    pad[:, :, :24] = packed.reshape(3, 2, 24)
    pad[:, :, 24:] = 0xEE  # padding is never read
    assert np.array_equal(O.unpack_fp6_padded(pad.reshape(3, 64)), codes)
