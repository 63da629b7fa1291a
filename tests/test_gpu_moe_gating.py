"""GPU parity of the router gating (``psg_moe_topk_gating``) and of gating + sorting (``psg_moe_softmax_sorting``) against the
oracle, through the reference's call shapes (kernels/moe/topk_gating_softmax_kernel.py:392-686 ``build_topk_gating_softmax_module``,
kernels/moe/moe_sorting_kernel.py:2250 ``moe_softmax_sort_flydsl``).  Shapes and checks follow the reference's
tests/kernels/test_topk_gating_softmax.py (its four configurations, logits quantised to the input dtype first, the
``k * num_tokens + row`` rule, renormalised sums) plus expert counts its layout rejects, unaligned rows, exact ties and
both sides of the fused / two-step border.

Indices are compared exactly on every row whose oracle probabilities around the cut are either equal (a tie: lower index
wins on both sides) or more than a few fp32 ulps apart; rows with closer probabilities could legitimately order differently
(the GPU's exp2 and numpy's differ in the last bit) and are checked the way the reference's test does: every chosen expert
reaches the k-th largest probability.  Weights: rtol 2e-5 (fp32 arithmetic on both sides, different summation order)."""

import numpy as np
import pytest
import torch

from oracle import psg_oracle as O
from kernels.moe.topk_gating_softmax_kernel import build_topk_gating_softmax_module
from kernels.moe.moe_sorting_kernel import moe_softmax_sort_flydsl
from flydsl_amd.kernels.moe.moe_sorting import sorted_sizes

pytestmark = pytest.mark.gpu
TDT = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}


def _logits(tokens, experts, dtype_str, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.rand((tokens, experts), generator=g) * 4.0 - 2.0  # the reference test's distribution
    return x.to(TDT[dtype_str]).contiguous()


def _gate(x, topk, dtype_str, renorm=True, tei=True):
    dev = torch.device("cuda")
    tokens, experts = x.shape
    launch = build_topk_gating_softmax_module(num_experts=experts, topk=topk, dtype_str=dtype_str, renormalize=renorm)
    w = torch.full((tokens, topk), float("nan"), dtype=torch.float32, device=dev)
    idx = torch.full((tokens, topk), -7, dtype=torch.int32, device=dev)
    te = torch.full((tokens, topk), -7, dtype=torch.int32, device=dev) if tei else None
    launch(x.to(dev), w, idx, te, tokens, stream=torch.cuda.current_stream())
    torch.cuda.synchronize()
    return w.cpu().numpy(), idx.cpu().numpy(), None if te is None else te.cpu().numpy()


def _check(x, topk, got, renorm):
    w, idx, tei = got
    xf = x.float().numpy()
    rw, ridx, rtei = O.topk_gating_softmax(xf, topk, renorm)
    tokens, experts = xf.shape
    if tei is not None:
        assert np.array_equal(tei, rtei)
    # probabilities in float64 for the separation test
    p = np.exp(xf.astype(np.float64) - xf.max(1, keepdims=True))
    p /= p.sum(1, keepdims=True)
    srt = -np.sort(-p, axis=1)[:, : min(topk + 1, experts)]
    gap = np.abs(np.diff(srt, axis=1)) / srt[:, :-1]
    clear = np.all((gap == 0) | (gap > 2e-6), axis=1)
    assert clear.mean() > 0.97
    assert np.array_equal(idx[clear], ridx[clear])
    assert np.allclose(w[clear], rw[clear], rtol=2e-5, atol=0)
    for t in np.nonzero(~clear)[0]:
        assert len(set(idx[t].tolist())) == topk and all(p[t, j] >= srt[t, topk - 1] * (1 - 1e-5) for j in idx[t])
        assert np.allclose(np.sort(w[t]), np.sort(rw[t]), rtol=1e-4)
    assert idx.min() >= 0 and idx.max() < experts
    if renorm:
        assert np.allclose(w.sum(1), 1.0, atol=1e-5)
    assert np.all(np.diff(w, axis=1) <= 0)  # found in descending order


@pytest.mark.parametrize("tokens,experts,topk,dtype_str", [
    (1024, 128, 6, "bf16"), (512, 64, 2, "bf16"), (256, 8, 2, "f32"), (128, 128, 6, "f16"),  # the reference's configurations
    (4096, 256, 8, "bf16"), (1, 256, 8, "bf16"), (33, 96, 9, "f16"), (17, 7, 7, "f32"), (5, 1024, 32, "f32"), (64, 20, 3, "bf16"),
    (300, 384, 10, "f32"), (9, 16, 1, "f16"), (2, 1, 1, "f32"), (77, 160, 4, "bf16"),
])
@pytest.mark.parametrize("renorm", [True, False])
def test_gating_matches_oracle(tokens, experts, topk, dtype_str, renorm):
    x = _logits(tokens, experts, dtype_str, seed=tokens + experts + topk)
    _check(x, topk, _gate(x, topk, dtype_str, renorm), renorm)


def test_rows_that_are_not_vector_aligned_and_no_tei():
    # a view that starts 2 bytes into an allocation: the lanes' column groups cannot be fetched as aligned vectors
    dev = torch.device("cuda")
    tokens, experts, topk = 50, 128, 6
    x = _logits(tokens, experts, "bf16", 5)
    pad = torch.zeros(tokens * experts + 1, dtype=torch.bfloat16, device=dev)
    pad[1:] = x.to(dev).view(-1)
    view = pad[1:].view(tokens, experts)
    launch = build_topk_gating_softmax_module(num_experts=experts, topk=topk, dtype_str="bf16")
    w = torch.empty((tokens, topk), dtype=torch.float32, device=dev)
    idx = torch.empty((tokens, topk), dtype=torch.float32, device=dev)  # an fp32 view over int32 storage, as the reference's callers pass
    launch(view, w, idx, None, tokens, stream=None)
    torch.cuda.synchronize()
    _check(x, topk, (w.cpu().numpy(), idx.view(torch.int32).cpu().numpy(), None), True)


def test_ties_go_to_the_lower_expert_and_uniform_rows():
    x = torch.zeros((3, 64), dtype=torch.float32)
    x[1, [9, 40, 41]] = 2.0
    x[2, 63] = 30.0
    w, idx, _ = _gate(x, 4, "f32", renorm=False)
    assert idx[0].tolist() == [0, 1, 2, 3] and np.allclose(w[0], 1 / 64, rtol=1e-6)
    assert idx[1].tolist() == [9, 40, 41, 0]
    assert idx[2].tolist() == [63, 0, 1, 2] and abs(w[2, 0] - 1.0) < 1e-6


def test_graph_replays_equal_eager():
    dev = torch.device("cuda")
    tokens, experts, topk = 200, 256, 8
    xs = [_logits(tokens, experts, "bf16", s).to(dev) for s in range(3)]
    launch = build_topk_gating_softmax_module(num_experts=experts, topk=topk, dtype_str="bf16")
    x = torch.empty_like(xs[0])
    w = torch.empty((tokens, topk), dtype=torch.float32, device=dev)
    idx = torch.empty((tokens, topk), dtype=torch.int32, device=dev)
    tei = torch.empty((tokens, topk), dtype=torch.int32, device=dev)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    x.copy_(xs[0])
    with torch.cuda.stream(side):
        launch(x, w, idx, tei, tokens, stream=side)
    side.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        launch(x, w, idx, tei, tokens, stream=torch.cuda.current_stream())
    for src in xs:
        x.copy_(src)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        got = (w.cpu().numpy().copy(), idx.cpu().numpy().copy())
        w.fill_(0)
        launch(x, w, idx, tei, tokens, stream=None)
        torch.cuda.synchronize()
        assert np.array_equal(got[0], w.cpu().numpy()) and np.array_equal(got[1], idx.cpu().numpy())


@pytest.mark.parametrize("tokens,experts,topk,unit,dtype_str", [
    (1, 256, 8, 32, "bf16"), (4, 8, 2, 16, "f32"), (16, 128, 6, 32, "bf16"), (16, 256, 8, 32, "f16"), (32, 64, 32, 16, "bf16"),  # one launch
    (17, 256, 8, 32, "bf16"), (33, 128, 8, 32, "bf16"), (200, 128, 6, 64, "f16"), (1500, 32, 4, 32, "f32"),                                                 # two steps
])
@pytest.mark.parametrize("masked", [False, True])
def test_gating_plus_sorting_equals_the_two_steps(tokens, experts, topk, unit, dtype_str, masked):
    # the routing the stand-alone gating kernel finds (checked against the oracle above), sorted by the oracle, is what
    # the combined call must produce bit for bit, whichever way it runs
    dev = torch.device("cuda")
    x = _logits(tokens, experts, dtype_str, seed=tokens * 3 + experts)
    w, idx, _ = _gate(x, topk, dtype_str, True, tei=False)
    mask = None
    if masked:
        mask = (np.random.default_rng(tokens).random(experts) < 0.7).astype(np.int32)
        mask[int(idx[0, 0])] = 1
    want = O.moe_sorting(idx, w, experts, unit, expert_mask=mask)
    rows, blocks = sorted_sizes(tokens, topk, experts, unit)
    s_ids = torch.full((rows,), -7, dtype=torch.int32, device=dev)
    s_w = torch.full((rows,), float("nan"), dtype=torch.float32, device=dev)
    s_e = torch.full((blocks,), -7, dtype=torch.int32, device=dev)
    nv = torch.full((2,), -7, dtype=torch.int32, device=dev)
    buf = torch.full((tokens, 64), 3.0, dtype=torch.bfloat16, device=dev)
    ids_out = torch.full((tokens, topk), -7, dtype=torch.int32, device=dev)
    w_out = torch.full((tokens, topk), float("nan"), dtype=torch.float32, device=dev)
    m = None if mask is None else torch.from_numpy(mask).to(dev)
    moe_softmax_sort_flydsl(x.to(dev), s_ids, s_w, s_e, nv, buf, experts, topk, dtype_str, unit, m, True, None, topk_ids=ids_out, topk_weights=w_out)
    torch.cuda.synchronize()
    for name, a, b in zip(("sorted_ids", "sorted_weights", "sorted_expert_ids", "num_valid_ids"), (s_ids, s_w, s_e, nv), want):
        assert np.array_equal(a.cpu().numpy(), b), name
    assert float(buf.float().abs().max()) == 0.0
    assert np.array_equal(ids_out.cpu().numpy(), idx) and np.array_equal(w_out.cpu().numpy(), w)  # the routing is handed out too
    # without the optional routing outputs
    s_ids.fill_(-7)
    moe_softmax_sort_flydsl(x.to(dev), s_ids, s_w, s_e, nv, None, experts, topk, dtype_str, unit, m)
    torch.cuda.synchronize()
    assert np.array_equal(s_ids.cpu().numpy(), want[0])


def test_argument_errors():
    with pytest.raises(ValueError):
        build_topk_gating_softmax_module(num_experts=2048, topk=8)
    with pytest.raises(ValueError):
        build_topk_gating_softmax_module(num_experts=8, topk=9)
    with pytest.raises(ValueError):
        build_topk_gating_softmax_module(num_experts=8, topk=2, dtype_str="f64")
    launch = build_topk_gating_softmax_module(num_experts=8, topk=2, dtype_str="bf16")
    dev = torch.device("cuda")
    w = torch.empty((4, 2), dtype=torch.float32, device=dev)
    idx = torch.empty((4, 2), dtype=torch.int32, device=dev)
    with pytest.raises(ValueError):  # dtype of the logits
        launch(torch.zeros((4, 8), dtype=torch.float32, device=dev), w, idx, None, 4)
    with pytest.raises(ValueError):  # more tokens than the tensors hold
        launch(torch.zeros((4, 8), dtype=torch.bfloat16, device=dev), w, idx, None, 5)
    with pytest.raises(ValueError):  # host tensor
        launch(torch.zeros((4, 8), dtype=torch.bfloat16), w, idx, None, 4)
