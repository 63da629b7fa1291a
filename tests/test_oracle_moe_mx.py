"""Pins of the oracle's fused MX-FP4 MoE restatement (CPU only) and of the product's host-side scale layout helpers against it.

The reference holds no golden vectors for these functions; each is pinned by independent means: explicit loops over the
closed-form byte offsets, the defining inequality of the power-of-two round-up, and a token-major recomputation of the
grouped stages with ``run_torch_mx`` (a different index order from the sorted-block loop of the oracle)."""

import numpy as np
import torch

from flydsl_amd import layout
from oracle import psg_oracle as O


def test_e8m0_shuffle_matches_closed_form_offsets_and_the_gemm_scale_layout():
    rng = np.random.default_rng(0)
    for r, c in ((64, 8), (300, 12), (256, 16)):
        sc = rng.integers(1, 255, size=(r, c), dtype=np.uint8)
        out = O.e8m0_shuffle(sc)
        rp, cp = (r + 255) // 256 * 256, (c + 7) // 8 * 8
        assert out.shape == (rp, cp)
        flat = out.reshape(-1)
        want = np.zeros(rp * cp, dtype=np.uint8)
        for i in range(r):
            for j in range(c):
                want[((i // 32 * (cp // 8) + j // 8) * 4 + j % 4) * 64 + (i % 16) * 4 + ((j % 8) // 4) * 2 + (i % 32) // 16] = sc[i, j]
        assert np.array_equal(flat, want)
        assert np.array_equal(O.e8m0_unshuffle(out, rp, cp)[:r, :c], sc)
        assert np.array_equal(layout.e8m0_shuffle(torch.from_numpy(sc)).numpy(), out)
    sc = rng.integers(0, 255, size=(256, 16), dtype=np.uint8)
    assert np.array_equal(O.e8m0_shuffle(sc), O.shuffle_scale_w4(sc))


def test_moe_mxfp4_sort_matches_explicit_loops():
    rng = np.random.default_rng(1)
    tokens, topk, c = 11, 3, 16
    ids = np.concatenate([rng.integers(0, tokens, size=40), np.full(8, tokens), rng.integers(0, tokens, size=10)]).astype(np.int64)
    ids = (ids | (rng.integers(0, topk, size=ids.size) << 24)).astype(np.int32)
    num_valid = 48
    for sc in (rng.integers(1, 255, size=(tokens, c), dtype=np.uint8), rng.integers(1, 255, size=(tokens, topk, c), dtype=np.uint8)):
        out = O.moe_mxfp4_sort(sc, ids, num_valid, tokens)
        rows = (ids.size + 31) // 32 * 32
        assert out.shape == (rows, c)
        u32 = out.reshape(rows // 32, c // 8, 4, 16, 4)  # [row chunk][column chunk][column % 4][row % 16][byte]
        for i in range(rows):
            tok, slot = (int(ids[i]) & 0xFFFFFF, int(ids[i]) >> 24) if i < ids.size else (tokens, 0)
            for j in range(c):
                got = u32[i // 32, j // 8, j % 4, i % 16, ((i % 32) // 16) + 2 * ((j % 8) // 4)]
                if i < num_valid and tok < tokens:
                    assert got == (sc[tok, j] if sc.ndim == 2 else sc[tok, slot, j])
                else:
                    assert got == 0
        t = layout.moe_mxfp4_sort(torch.from_numpy(sc), torch.from_numpy(ids), torch.tensor([num_valid, tokens], dtype=torch.int32), tokens)
        assert np.array_equal(t.numpy(), out)


def test_e8m0_roundup_is_the_smallest_power_of_two_not_below_amax_over_six():
    rng = np.random.default_rng(2)
    amax = np.concatenate([np.exp(rng.uniform(-40, 40, size=4000)), 6.0 * np.ldexp(1.0, np.arange(-60, 60)), [0.0, 6.0, 5.9999995, 6.000001, 3.0, 12.0]]).astype(np.float32)
    b = O.e8m0_roundup(amax).astype(np.int64)
    v = (amax * np.float32(1.0 / 6.0)).astype(np.float32).astype(np.float64)
    nz = amax > 0
    assert np.all(b[~nz] == 0)
    hi, lo = np.ldexp(1.0, b[nz] - 127), np.ldexp(1.0, b[nz] - 128)
    assert np.all(v[nz] <= hi) and np.all(v[nz] > lo)
    assert O.e8m0_roundup(np.array([3.4e38], dtype=np.float32))[0] <= 254


def test_requant_error_is_below_half_a_code_step_and_never_saturates():
    rng = np.random.default_rng(3)
    y = (rng.standard_normal((16, 128)) * np.exp(rng.uniform(-6, 6, size=(16, 1)))).astype(np.float32)
    y[3, 32:64] = 0.0
    packed, sc = O.mxfp4_requant_roundup(y)
    deq = O.mxfp4_to_f32(packed) * np.repeat(np.ldexp(1.0, sc.astype(np.int32) - 127), 32, axis=1)
    step = np.repeat(np.ldexp(1.0, sc.astype(np.int32) - 127), 32, axis=1)
    assert np.all(np.abs(deq - y) <= 1.0 * step * (1 + 1e-6))  # the widest e2m1 gap (4..6) is two scale units
    assert np.all(np.abs(deq) <= 6.0 * step) and np.all(np.abs(y) <= 6.0 * step * (1 + 1e-6))
    assert sc[3, 1] == 0 and not packed[3, 16:32].any()


def _problem(tokens, model_dim, inter, experts, topk, bm, a_fmt, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((tokens, model_dim)).astype(np.float32)
    w1 = (rng.standard_normal((experts * 2 * inter, model_dim)) / np.sqrt(model_dim)).astype(np.float32)
    w2 = (rng.standard_normal((experts * model_dim, inter)) / np.sqrt(inter)).astype(np.float32)
    a_q, a_s = O.per_1x32_f4_quant(x) if a_fmt == "fp4" else O.per_1x32_f8_quant(x)
    w1_q, w1_s = O.per_1x32_f4_quant(w1)
    w2_q, w2_s = O.per_1x32_f4_quant(w2)
    ids = np.stack([rng.permutation(experts)[:topk] for _ in range(tokens)]).astype(np.int32)
    wts = rng.uniform(0.1, 1.0, size=(tokens, topk)).astype(np.float32)
    return dict(a_q=a_q, a_s=a_s[:tokens], w1_q=w1_q, w1_s=w1_s, w2_q=w2_q, w2_s=w2_s, ids=ids, wts=wts, sort=O.moe_sorting(ids, wts, experts, bm))


def test_sorted_block_stages_agree_with_a_token_major_recomputation():
    tokens, model_dim, inter, experts, topk, bm = 9, 256, 256, 4, 2, 32
    for a_fmt in ("fp4", "fp8"):
        p = _problem(tokens, model_dim, inter, experts, topk, bm, a_fmt, seed=5)
        sid, sw, se, npp = p["sort"]
        y, packed, sc = O.moe_mx_gemm1(p["a_q"], p["a_s"], p["w1_q"], p["w1_s"], sid, se, int(npp[0]), tokens, inter, bm, a_fmt)
        flat, out = O.moe_mx_gemm2(packed, sc, p["w2_q"], p["w2_s"], sid, sw, se, int(npp[0]), tokens, model_dim, bm)
        want_out = np.zeros((tokens, model_dim), dtype=np.float64)
        seen = 0
        for i in range(int(npp[0])):
            t, s = int(sid[i]) & 0xFFFFFF, int(sid[i]) >> 24
            if t >= tokens:
                assert not y[i].any() and not packed[i].any() and not sc[i].any()
                continue
            e = int(p["ids"][t, s])
            assert e == int(se[i // bm])
            gu = O.run_torch_mx(p["a_q"][t : t + 1], p["w1_q"][e * 2 * inter : (e + 1) * 2 * inter], p["a_s"][t : t + 1],
                                p["w1_s"][e * 2 * inter : (e + 1) * 2 * inter], a_fmt, "fp4")[0]
            g, u = gu[:inter].astype(np.float64), gu[inter:].astype(np.float64)
            np.testing.assert_allclose(y[i], g / (1 + np.exp(-g)) * u, rtol=2e-5, atol=1e-6)
            q, s2 = O.mxfp4_requant_roundup(y[i : i + 1])
            assert np.array_equal(q[0], packed[i]) and np.array_equal(s2[0], sc[i])
            d = O.run_torch_mx(q, p["w2_q"][e * model_dim : (e + 1) * model_dim], s2, p["w2_s"][e * model_dim : (e + 1) * model_dim])[0]
            np.testing.assert_allclose(flat[i], d, rtol=2e-5, atol=1e-6)
            want_out[t] += float(p["wts"][t, s]) * d
            seen += 1
        assert seen == tokens * topk
        np.testing.assert_allclose(out, want_out, rtol=1e-4, atol=1e-5)
