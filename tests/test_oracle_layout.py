"""Pins of the oracle's wire formats: explicit loops over the closed-form byte offsets, bijectivity, and
agreement of the two oracles (numpy on un-shuffled operands vs C on the wire format)."""

import numpy as np

from oracle import c_oracle as C
from oracle import psg_oracle as O


def test_shuffle_weight_1byte_closed_form():
    n, k = 32, 128
    w = np.arange(n * k, dtype=np.uint32).astype(np.uint8).reshape(n, k) ^ np.arange(n, dtype=np.uint8)[:, None]
    w = (np.arange(n * k) % 251).astype(np.uint8).reshape(n, k)
    flat = O.shuffle_weight(w).reshape(-1)
    seen = np.zeros(n * k, dtype=bool)
    for r in range(n):
        for c in range(k):
            off = (r // 16) * 16 * k + (c // 64) * 1024 + ((c % 64) // 16) * 256 + (r % 16) * 16 + c % 16
            assert flat[off] == w[r, c]
            seen[off] = True
    assert seen.all()
    # the same map written the way the host utility states it: (k/32)*512 + ((k%32)/16)*256
    for r, c in [(0, 0), (5, 17), (17, 33), (31, 127)]:
        off2 = (r // 16) * 16 * k + (c // 32) * 512 + ((c % 32) // 16) * 256 + (r % 16) * 16 + c % 16
        assert flat[off2] == w[r, c]


def test_shuffle_weight_2byte_closed_form():
    n, k = 32, 64
    w = np.arange(n * k, dtype=np.uint16).reshape(n, k)
    flat = O.shuffle_weight(w).reshape(-1)
    for r in range(n):
        for c in range(k):
            off = (r // 16) * 16 * k + (c // 32) * 512 + ((c % 32) // 8) * 128 + (r % 16) * 8 + c % 8
            assert flat[off] == w[r, c]


def test_shuffle_weight_w4_is_the_same_map_on_packed_bytes():
    n, kpk = 32, 128
    p = (np.arange(n * kpk) % 253).astype(np.uint8).reshape(n, kpk)
    assert np.array_equal(O.shuffle_weight_w4(p), O.shuffle_weight(p))
    # one lane's 16 bytes = 32 consecutive fp4 of one row = exactly one scale block
    flat = O.shuffle_weight_w4(p).reshape(-1)
    lane = 37  # nlane 5, klane 2
    chunk = flat[1024 * 1 + lane * 16: 1024 * 1 + lane * 16 + 16]  # block (n/16 = 0, kbyte/64 = 1)
    assert np.array_equal(chunk, p[5, 64 + 2 * 16: 64 + 3 * 16])


def test_shuffle_scale_w4_closed_form():
    r, kb = 64, 16
    s = (np.arange(r * kb) % 241).astype(np.uint8).reshape(r, kb)
    flat = O.shuffle_scale_w4(s).reshape(-1)
    seen = np.zeros(r * kb, dtype=bool)
    for i in range(r):
        for j in range(kb):
            off = (i // 32) * 32 * kb + (j // 8) * 256 + (j % 4) * 64 + (i % 16) * 4 + ((j % 8) // 4) * 2 + (i % 32) // 16
            assert flat[off] == s[i, j]
            seen[off] = True
    assert seen.all()
    # dword view: lane = (kb%4)*16 + r%16, byte = 2*(128-K half) + (16-row half)
    dw = flat.reshape(-1, 4)
    i, j = 21, 13  # chunk 0, row half 1, r%16 = 5; k chunk 1, half 1, kb%4 = 1
    assert dw[(0 * (kb // 8) + 1) * 64 + 1 * 16 + 5, 1 * 2 + 1] == s[i, j]


def test_two_oracles_agree_a8w8():
    rng = np.random.default_rng(0)
    m, n, k = 9, 48, 192
    x = rng.standard_normal((m, k)).astype(np.float32)
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    for kind in ("int8", "fp8"):
        aq, sa = O.pertoken_quant(x, kind)
        bq, sb = O.pertoken_quant(w, kind)
        r = C.a8w8(aq, O.shuffle_weight(bq.view(np.uint8)), sa, sb, kind, want_acc_i32=(kind == "int8"))
        ref = O.run_torch(aq, bq, sa, sb, kind)
        out = O.bf16_bits_to_f32(r["c_bf16_bits"])
        assert np.allclose(out, ref, rtol=2 ** -7, atol=1e-6)
        if kind == "int8":
            assert np.array_equal(r["acc_i32"], O.int32_accumulators(aq, bq))
            # same arithmetic order -> same bits
            want = O.f32_to_bf16_bits(O.epilogue_a8w8(r["acc_i32"], sa, sb))
            assert np.array_equal(r["c_bf16_bits"], want)


def test_two_oracles_agree_mxfp4():
    rng = np.random.default_rng(1)
    m, n, k = 32, 64, 512
    x = rng.standard_normal((m, k)).astype(np.float32)
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    ap, sa = O.per_1x32_f4_quant(x)
    bp, sb = O.per_1x32_f4_quant(w)
    ref = O.run_torch_w4(ap, bp, sa, sb)
    r = C.mxfp4(ap, O.shuffle_weight_w4(bp), O.shuffle_scale_w4(sa), O.shuffle_scale_w4(sb), m, n, k)
    assert np.allclose(r["out_f32"], ref, rtol=1e-5, atol=1e-6 * np.abs(ref).max())


def test_xcd_remap_is_a_bijection():
    for (m, n, tm, tn, sw) in [(8192, 4096, 256, 256, 4), (4096, 28672, 256, 256, 4), (300, 1056, 64, 128, 3),
                               (33, 1024, 32, 64, 1), (5133, 5120, 64, 256, 8)]:
        gx, gy = n // tn, (m + tm - 1) // tm
        seen = set()
        for bx in range(gy):
            for by in range(gx):
                nb = O.xcd_remap_bx_by(bx, by, m, tile_m=tm, tile_n=tn, n=n, xcd_swizzle=sw)
                assert 0 <= nb[0] < gy and 0 <= nb[1] < gx
                seen.add(nb)
        assert len(seen) == gx * gy
    assert O.xcd_remap_bx_by(3, 5, 100, tile_m=16, tile_n=64, n=1024, xcd_swizzle=0) == (3, 5)


def test_xcd_remap_known_answers():
    """Worked by hand from the reference's formula (kernels/common/mma/mfma_preshuffle_pipeline.py:685-729) for
    M=768, N=1024, 256x256 tiles (gy=3 M-tiles, gx=4 N-tiles, 12 workgroups: q=1, r=4) and xcd_swizzle=2:
      (bx,by) -> linear -> (xcd, in_xcd) -> wgid -> group / in_group -> (bx', by')
      (0,0) -> 0  -> (0,0) -> 0        -> 0 / 0  -> (0,0)
      (0,1) -> 1  -> (1,0) -> 1+1=2    -> 0 / 2  -> (0,1)
      (1,1) -> 5  -> (5,0) -> 5+4=9    -> 1 / 1, last group holds 1 M-tile -> (2,1)
      (2,1) -> 9  -> (1,1) -> 1+1+1=3  -> 0 / 3  -> (1,1)
      (2,3) -> 11 -> (3,1) -> 3+3+1=7  -> 0 / 7  -> (1,3)
      (1,3) -> 7  -> (7,0) -> 7+4=11   -> 1 / 3  -> (2,3)
    A transposed (bx,by), a dropped remainder term or a row-major walk inside the group each break one of these."""
    kw = dict(tile_m=256, tile_n=256, n=1024, xcd_swizzle=2)
    for (bx, by), want in {(0, 0): (0, 0), (0, 1): (0, 1), (1, 1): (2, 1), (2, 1): (1, 1), (2, 3): (1, 3), (1, 3): (2, 3)}.items():
        assert O.xcd_remap_bx_by(bx, by, 768, **kw) == want, (bx, by)
