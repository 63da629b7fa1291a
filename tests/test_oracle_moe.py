"""Pins of the MoE oracle functions: sorting by invariants and a hand-worked example, the two stage references by scalar
float64 loops on tiny inputs, and the product's vectorised sorter against the oracle's loop."""

import math

import numpy as np
import torch

from oracle import psg_oracle as O


def _routing(tokens, experts, topk, seed):
    g = torch.Generator().manual_seed(seed)
    score = torch.rand(tokens, experts, generator=g)
    vals, ids = torch.topk(score, k=topk, dim=1)
    return ids.numpy().astype(np.int32), torch.softmax(vals, dim=1).numpy().astype(np.float32)


def test_moe_sorting_hand_worked_example():
    # 3 tokens, top-2, 3 experts, blocks of 4: expert 0 <- (t0,s0),(t2,s1); expert 1 <- (t0,s1),(t1,s0),(t2,s0); expert 2 <- (t1,s1)
    ids = np.array([[0, 1], [1, 2], [1, 0]], dtype=np.int32)
    w = np.array([[.6, .4], [.7, .3], [.8, .2]], dtype=np.float32)
    sid, sw, se, npp = O.moe_sorting(ids, w, 3, 4)
    pad = (2 << 24) | 3
    assert sid.tolist() == [0, (1 << 24) | 2, pad, pad, (1 << 24) | 0, 1, 2, pad, (1 << 24) | 1, pad, pad, pad, pad, pad, pad, pad]
    assert se.tolist() == [0, 1, 2, -1]
    assert npp.tolist() == [12, 3]
    assert np.allclose(sw[[0, 1, 4, 5, 6, 8]], [.6, .2, .4, .7, .8, .3])
    assert len(sid) == 3 * 2 + 3 * 4 - 2


def test_moe_sorting_hand_worked_example_with_expert_mask():
    # same routing, expert 1 switched off: its three pairs vanish, expert 2 becomes local expert 1
    ids = np.array([[0, 1], [1, 2], [1, 0]], dtype=np.int32)
    w = np.array([[.6, .4], [.7, .3], [.8, .2]], dtype=np.float32)
    sid, sw, se, npp = O.moe_sorting(ids, w, 3, 4, expert_mask=np.array([1, 0, 1], dtype=np.int32))
    pad = (2 << 24) | 3
    assert sid.tolist() == [0, (1 << 24) | 2, pad, pad, (1 << 24) | 1] + [pad] * 11
    assert se.tolist() == [0, 1, -1, -1]
    assert npp.tolist() == [8, 3]
    assert np.allclose(sw[[0, 1, 4]], [.6, .2, .3]) and (sw[[2, 3, 5, 6, 7]] == 0).all()
    # an all-ones mask changes nothing
    for a, b in zip(O.moe_sorting(ids, w, 3, 4, expert_mask=np.ones(3, dtype=np.int32)), O.moe_sorting(ids, w, 3, 4)):
        assert np.array_equal(a, b)


def test_moe_sorting_invariants_and_product_sorter():
    from flydsl_amd.kernels.moe.moe_sorting import moe_sorting

    for tokens, experts, topk, bm, seed in [(8, 4, 2, 16, 0), (129, 8, 2, 32, 1), (33, 8, 2, 64, 2), (1, 8, 1, 16, 3), (333, 17, 9, 64, 4), (7, 8, 2, 128, 5)]:
        ids, w = _routing(tokens, experts, topk, seed)
        sid, sw, se, npp = O.moe_sorting(ids, w, experts, bm)
        valid = int(npp[0])
        assert valid % bm == 0 and npp[1] == tokens
        blocks = valid // bm
        assert (se[:blocks] >= 0).all() and (np.diff(se[:blocks]) >= 0).all() and (se[blocks:] == -1).all()
        seen = set()
        for i in range(valid):
            t, s = int(sid[i]) & 0xFFFFFF, int(sid[i]) >> 24
            if t >= tokens:
                assert (t, s) == (tokens, topk)
                continue
            assert ids[t, s] == se[i // bm] and sw[i] == w[t, s] and (t, s) not in seen
            seen.add((t, s))
        assert len(seen) == tokens * topk
        assert (sid[valid:] == ((topk << 24) | tokens)).all()
        got = moe_sorting(torch.from_numpy(ids), torch.from_numpy(w), num_experts=experts, block_size=bm)
        for a, b in zip(got, (sid, sw, se, npp)):
            assert np.array_equal(a.numpy(), b)


def test_moe_gemm1_slot_major_rows_against_a_scalar_loop():
    # the int8smooth layout: one row of x and one scale per (slot, token) at slot*tokens + token
    rng = np.random.default_rng(9)
    tokens, experts, topk, model_dim, inter = 4, 3, 2, 16, 8
    ids, w = _routing(tokens, experts, topk, 4)
    xq = rng.integers(-127, 128, (topk * tokens, model_dim)).astype(np.int8)
    w1q = rng.integers(-127, 128, (experts * 2 * inter, model_dim)).astype(np.int8)
    sx = rng.uniform(0.01, 0.02, topk * tokens).astype(np.float32)
    sw1 = rng.uniform(0.001, 0.002, experts * 2 * inter).astype(np.float32)
    want = np.zeros((tokens, topk, inter))
    for t in range(tokens):
        for s in range(topk):
            e, r = int(ids[t, s]), s * tokens + t
            for n in range(inter):
                g = sum(float(xq[r, k]) * sx[r] * float(w1q[e * 2 * inter + n, k]) * sw1[e * 2 * inter + n] for k in range(model_dim))
                u = sum(float(xq[r, k]) * sx[r] * float(w1q[e * 2 * inter + inter + n, k]) * sw1[e * 2 * inter + inter + n] for k in range(model_dim))
                want[t, s, n] = g / (1 + math.exp(-g)) * u
    got = O.moe_gemm1(xq.view(np.uint8), w1q.view(np.uint8), sx, sw1, ids, w, inter, False, "int8", x_slot_major=True)
    assert np.allclose(got, want, rtol=2e-5, atol=1e-6 * np.abs(want).max())
    # rows that repeat the token's row in every slot give the token-major result
    rep_x = np.tile(xq[:tokens], (topk, 1))
    rep_s = np.tile(sx[:tokens], topk)
    a = O.moe_gemm1(rep_x.view(np.uint8), w1q.view(np.uint8), rep_s, sw1, ids, w, inter, False, "int8", x_slot_major=True)
    b = O.moe_gemm1(xq[:tokens].view(np.uint8), w1q.view(np.uint8), sx[:tokens], sw1, ids, w, inter, False, "int8")
    assert np.array_equal(a, b)


def test_moe_reduce_with_and_without_mask_against_a_scalar_loop():
    rng = np.random.default_rng(5)
    tokens, topk, dim, experts = 6, 3, 8, 5
    x = rng.standard_normal((tokens, topk, dim)).astype(np.float32)
    ids = rng.integers(0, experts, (tokens, topk)).astype(np.int32)
    mask = np.array([1, 0, 1, 1, 0], dtype=np.int32)
    xp = x.copy()
    xp[mask[ids] == 0] = np.nan  # what stage 2 never wrote must not reach the sum
    got = O.moe_reduce(xp, ids, mask)
    for t in range(tokens):
        for d in range(dim):
            acc = np.float32(0)
            for k in range(topk):
                if mask[ids[t, k]]:
                    acc = np.float32(acc + x[t, k, d])
            assert got[t, d] == acc
    assert np.array_equal(O.moe_reduce(x), x[:, 0] + x[:, 1] + x[:, 2])
    assert np.array_equal(O.moe_reduce(x, ids, np.ones(experts, dtype=np.int32)), O.moe_reduce(x))
    assert not np.isnan(got).any() and (O.moe_reduce(x, ids, np.zeros(experts, dtype=np.int32)) == 0).all()


def test_moe_stage_references_against_scalar_loops():
    rng = np.random.default_rng(3)
    tokens, experts, topk, model_dim, inter = 5, 3, 2, 32, 16
    ids, w = _routing(tokens, experts, topk, 7)
    for kind in ("int8", "fp8"):
        if kind == "int8":
            xq = rng.integers(-127, 128, (tokens, model_dim)).astype(np.int8)
            w1q = rng.integers(-127, 128, (experts * 2 * inter, model_dim)).astype(np.int8)
            w2q = rng.integers(-127, 128, (experts * model_dim, inter)).astype(np.int8)
            a2q = rng.integers(-127, 128, (tokens, topk, inter)).astype(np.int8)
            dec = lambda q: q.astype(np.float64)  # noqa: E731
        else:
            codes = np.array([c for c in range(256) if (c & 0x7F) != 0x7F], dtype=np.uint8)
            xq, w1q = rng.choice(codes, (tokens, model_dim)), rng.choice(codes, (experts * 2 * inter, model_dim))
            w2q, a2q = rng.choice(codes, (experts * model_dim, inter)), rng.choice(codes, (tokens, topk, inter))
            dec = lambda q: O.e4m3fn_to_f32(q).astype(np.float64)  # noqa: E731
        sx = rng.uniform(0.01, 0.02, tokens).astype(np.float32)
        sw1 = rng.uniform(0.001, 0.002, experts * 2 * inter).astype(np.float32)
        sa2 = rng.uniform(0.01, 0.02, tokens * topk).astype(np.float32)
        sw2 = rng.uniform(0.001, 0.002, experts * model_dim).astype(np.float32)
        for dow in (False, True):
            want1 = np.zeros((tokens, topk, inter))
            want2 = np.zeros((tokens, model_dim))
            for t in range(tokens):
                for s in range(topk):
                    e = int(ids[t, s])
                    for n in range(inter):
                        g = sum(dec(xq)[t, k] * sx[t] * dec(w1q)[e * 2 * inter + n, k] * sw1[e * 2 * inter + n] for k in range(model_dim))
                        u = sum(dec(xq)[t, k] * sx[t] * dec(w1q)[e * 2 * inter + inter + n, k] * sw1[e * 2 * inter + inter + n] for k in range(model_dim))
                        want1[t, s, n] = g / (1 + math.exp(-g)) * u * (w[t, s] if dow else 1.0)
                    for n in range(model_dim):
                        y = sum(dec(a2q)[t, s, k] * sa2[t * topk + s] * dec(w2q)[e * model_dim + n, k] * sw2[e * model_dim + n] for k in range(inter))
                        want2[t, n] += y * (w[t, s] if dow else 1.0)
            got1 = O.moe_gemm1(xq, w1q, sx, sw1, ids, w, inter, dow, kind)
            got2 = O.moe_gemm2(a2q, w2q, sa2, sw2, ids, w, model_dim, dow, kind)
            assert np.allclose(got1, want1, rtol=2e-5, atol=1e-6 * np.abs(want1).max())
            assert np.allclose(got2, want2, rtol=2e-5, atol=1e-6 * np.abs(want2).max())
            per_slot = O.moe_gemm2(a2q, w2q, sa2, sw2, ids, w, model_dim, dow, kind, reduce_slots=False)
            assert np.allclose(per_slot.sum(1), got2, rtol=1e-6, atol=1e-7)


def test_topk_gating_softmax_against_scipy_and_closed_forms():
    import scipy.special

    rng = np.random.default_rng(3)
    for tokens, experts, topk in ((37, 128, 6), (5, 8, 2), (16, 96, 9), (3, 7, 7)):
        x = rng.uniform(-2, 2, (tokens, experts)).astype(np.float32)
        p = scipy.special.softmax(x.astype(np.float64), axis=1)
        order = np.argsort(-p, axis=1, kind="stable")[:, :topk]  # an independent top-k: stable sort = lower index first
        want_w = np.take_along_axis(p, order, axis=1)
        for renorm in (False, True):
            w, idx, tei = O.topk_gating_softmax(x, topk, renorm)
            assert np.array_equal(idx, order.astype(np.int32))
            ref = want_w / want_w.sum(1, keepdims=True) if renorm else want_w
            assert np.allclose(w, ref, rtol=2e-6, atol=0)
            assert w.dtype == np.float32 and idx.dtype == np.int32 and tei.dtype == np.int32
            assert all(tei[t, k] == k * tokens + t for t in range(tokens) for k in range(topk))
            if renorm:
                assert np.allclose(w.sum(1), 1.0, atol=1e-6)
        # a shift of the logits changes nothing (max subtraction)
        w1, i1, _ = O.topk_gating_softmax(x + np.float32(8.0), topk, True)
        w0, i0, _ = O.topk_gating_softmax(x, topk, True)
        assert np.array_equal(i0, i1) and np.allclose(w0, w1, rtol=1e-5)
    # uniform logits: every probability 1/E, ties go to the lowest indices in order; renormalised 1/k
    w, idx, _ = O.topk_gating_softmax(np.full((2, 16), 0.25, np.float32), 4, False)
    assert np.array_equal(idx, np.tile(np.arange(4, dtype=np.int32), (2, 1))) and np.allclose(w, 1 / 16)
    w, _, _ = O.topk_gating_softmax(np.full((2, 16), 0.25, np.float32), 4, True)
    assert np.allclose(w, 0.25)
    # one dominant logit: weight ~1 first; equal runners-up in index order
    x = np.zeros((1, 8), np.float32)
    x[0, 5] = 40.0
    w, idx, _ = O.topk_gating_softmax(x, 3, False)
    assert idx.tolist() == [[5, 0, 1]] and abs(w[0, 0] - 1.0) < 1e-6 and w[0, 1] == w[0, 2] < 1e-15
    # ties between distinct positions inside a row
    x = np.array([[1.0, 3.0, 3.0, 0.0, 3.0, 2.0]], np.float32)
    assert O.topk_gating_softmax(x, 4, True)[1].tolist() == [[1, 2, 4, 5]]
