"""GPU parity of the device-side expert sorter (``psg_moe_sorting``) against the oracle, bit for bit, through the
reference's call shape ``moe_sorting_flydsl`` (kernels/moe/moe_sorting_kernel.py:2070-2083).  The shapes follow the
reference's tests/kernels/test_moe_sorting.py (token counts from 1 to thousands, 8 to 256 experts, expert masks, the
cleared ``moe_buf``) plus cases its generator avoids: an expert nobody routes to, every token on one expert, an expert
id repeated inside a token, ids outside the expert range."""

import numpy as np
import pytest
import torch

from oracle import psg_oracle as O
from kernels.moe.moe_sorting_kernel import UNIT_SIZE, moe_sorting_flydsl, moe_sorting_get_workspace_size
from flydsl_amd.kernels.moe.moe_sorting import moe_sorting, sorted_sizes

pytestmark = pytest.mark.gpu


def _routing(tokens, experts, topk, seed):
    g = torch.Generator().manual_seed(seed)
    score = torch.randn(tokens, experts, generator=g)
    vals, ids = torch.topk(score, k=topk, dim=1)
    return ids.to(torch.int32), torch.softmax(vals, dim=1).to(torch.float32)


def _run(ids, w, experts, unit, mask=None, model_dim=256, poison=True, workspace=None):
    dev = torch.device("cuda")
    tokens, topk = ids.shape
    rows, blocks = sorted_sizes(tokens, topk, experts, unit)
    fill = -7 if poison else 0
    s_ids = torch.full((rows,), fill, dtype=torch.int32, device=dev)
    s_w = torch.full((rows,), float("nan"), dtype=torch.float32, device=dev)
    s_e = torch.full((blocks,), fill, dtype=torch.int32, device=dev)
    nv = torch.full((2,), fill, dtype=torch.int32, device=dev)
    buf = torch.full((tokens, model_dim), 3.0, dtype=torch.bfloat16, device=dev)
    m = None if mask is None else torch.from_numpy(mask).to(dev)
    moe_sorting_flydsl(ids.to(dev), w.to(dev), s_ids, s_w, s_e, nv, buf, experts, unit, m, None, workspace)
    torch.cuda.synchronize()
    return s_ids.cpu().numpy(), s_w.cpu().numpy(), s_e.cpu().numpy(), nv.cpu().numpy(), buf


def _check(got, ids, w, experts, unit, mask=None):
    want = O.moe_sorting(ids.numpy(), w.numpy(), experts, unit, expert_mask=mask)
    for name, a, b in zip(("sorted_ids", "sorted_weights", "sorted_expert_ids", "num_valid_ids"), got, want):
        assert np.array_equal(a, b), name
    assert float(got[4].float().abs().max()) == 0.0  # moe_buf cleared by the same launch


@pytest.mark.parametrize("tokens,experts,topk,unit", [
    (1, 8, 1, 16), (1, 256, 8, 32), (8, 4, 2, 16), (33, 8, 2, 64), (64, 32, 8, 16), (129, 8, 2, 32), (333, 17, 9, 64),
    (7, 8, 2, 128), (512, 64, 6, 32), (2048, 128, 8, 32), (4096, 256, 8, 32), (5000, 32, 4, 128), (300, 200, 3, 1),
])
@pytest.mark.parametrize("workspace", [None, False], ids=["planned", "one_launch"])
def test_sorter_matches_oracle(tokens, experts, topk, unit, workspace):
    ids, w = _routing(tokens, experts, topk, seed=tokens + experts)
    _check(_run(ids, w, experts, unit, workspace=workspace), ids, w, experts, unit)


def test_workspace_sizes_and_a_workspace_that_is_too_small():
    assert moe_sorting_get_workspace_size(64, 32, 8) == 0           # decode-sized routings sort in one launch
    big = moe_sorting_get_workspace_size(4096, 256, 8)
    assert big > 0 and big % 4 == 0
    ids, w = _routing(4096, 256, 8, 9)
    small = torch.empty(big - 4, dtype=torch.uint8, device="cuda")  # refused as a workspace: the single launch runs instead
    _check(_run(ids, w, 256, 32, workspace=small), ids, w, 256, 32)
    exact = torch.full((big,), 0xA5, dtype=torch.uint8, device="cuda")  # contents need no initialisation
    _check(_run(ids, w, 256, 32, workspace=exact), ids, w, 256, 32)


def test_default_unit_size_is_the_references():
    assert UNIT_SIZE == 32


@pytest.mark.parametrize("tokens,experts,topk,unit,seed", [(64, 32, 8, 32, 0), (1000, 64, 6, 32, 1), (17, 16, 4, 16, 2), (3000, 96, 8, 64, 3)])
def test_expert_mask_drops_and_renumbers(tokens, experts, topk, unit, seed):
    ids, w = _routing(tokens, experts, topk, seed)
    rng = np.random.default_rng(seed)
    mask = (rng.random(experts) < 0.6).astype(np.int32)
    mask[0], mask[-1] = 0, 1
    _check(_run(ids, w, experts, unit, mask), ids, w, experts, unit, mask)
    zero = np.zeros(experts, dtype=np.int32)  # everything masked: no rows in use
    got = _run(ids, w, experts, unit, zero)
    _check(got, ids, w, experts, unit, zero)
    assert got[3].tolist() == [0, tokens]


def test_degenerate_routings():
    # every token on one expert; experts nobody routes to; one expert twice inside a token
    for tokens in (200, 5000):  # one launch / three launches
        experts, topk, unit = 16, 2, 32
        ids = torch.full((tokens, topk), 5, dtype=torch.int32)
        w = torch.rand(tokens, topk)
        _check(_run(ids, w, experts, unit), ids, w, experts, unit)
    ids2 = torch.tensor([[3, 3], [0, 15], [15, 15]], dtype=torch.int32)
    w2 = torch.rand(3, 2)
    _check(_run(ids2, w2, experts, 16), ids2, w2, experts, 16)


def test_ids_outside_the_expert_range_are_dropped():
    tokens, experts, topk, unit = 40, 8, 2, 16
    ids, w = _routing(tokens, experts, topk, 3)
    ids[5, 0], ids[9, 1], ids[11, 0] = -1, experts, 1 << 20
    got = _run(ids, w, experts, unit)
    want = O.moe_sorting(ids.numpy(), w.numpy(), experts, unit)  # the oracle only looks for ids in range(experts)
    for a, b in zip(got[:4], want):
        assert np.array_equal(a, b)


def test_results_do_not_depend_on_earlier_contents_or_timing():
    ids, w = _routing(777, 64, 8, 11)  # 6216 pairs: three launches
    a = _run(ids, w, 64, 32, poison=True)
    b = _run(ids, w, 64, 32, poison=False, workspace=False)
    for x, y in zip(a[:4], b[:4]):
        assert np.array_equal(x, y)


def test_device_path_of_the_convenience_sorter_and_graph_replay():
    dev = torch.device("cuda")
    ids, w = _routing(300, 32, 4, 5)
    got = moe_sorting(ids.to(dev), w.to(dev), num_experts=32, block_size=64)
    want = O.moe_sorting(ids.numpy(), w.numpy(), 32, 64)
    for a, b in zip(got, want):
        assert np.array_equal(a.cpu().numpy(), b)
    # recorded once, replayed with new routings in the same buffers
    T = 2000  # 8000 pairs: the three-launch plan, workspace owned by the caller as a capture needs it
    ids, w = _routing(T, 32, 4, 5)
    rows, blocks = sorted_sizes(T, 4, 32, 64)
    ws = torch.empty(moe_sorting_get_workspace_size(T, 32, 4), dtype=torch.uint8, device=dev)
    d_ids, d_w = ids.to(dev), w.to(dev)
    out = (torch.empty(rows, dtype=torch.int32, device=dev), torch.empty(rows, dtype=torch.float32, device=dev),
           torch.empty(blocks, dtype=torch.int32, device=dev), torch.empty(2, dtype=torch.int32, device=dev))
    buf = torch.ones(T, 64, dtype=torch.bfloat16, device=dev)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        moe_sorting_flydsl(d_ids, d_w, *out, buf, 32, 64, None, None, ws)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        moe_sorting_flydsl(d_ids, d_w, *out, buf, 32, 64, None, None, ws)
    for seed in (6, 7, 8):
        ids2, w2 = _routing(T, 32, 4, seed)
        d_ids.copy_(ids2.to(dev))
        d_w.copy_(w2.to(dev))
        buf.fill_(1.0)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        want = O.moe_sorting(ids2.numpy(), w2.numpy(), 32, 64)
        for a, b in zip(out, want):
            assert np.array_equal(a.cpu().numpy(), b)
        assert float(buf.float().abs().max()) == 0.0


def test_bad_arguments_are_refused_before_launch():
    dev = torch.device("cuda")
    ids, w = _routing(16, 8, 2, 0)
    rows, blocks = sorted_sizes(16, 2, 8, 32)
    ok = lambda n=rows, b=blocks: (torch.empty(n, dtype=torch.int32, device=dev), torch.empty(n, dtype=torch.float32, device=dev),
                                   torch.empty(b, dtype=torch.int32, device=dev), torch.empty(2, dtype=torch.int32, device=dev))
    with pytest.raises(ValueError):
        moe_sorting_flydsl(ids.to(dev), w.to(dev), *ok(rows - 1), None, 8, 32)
    with pytest.raises(ValueError):
        moe_sorting_flydsl(ids.to(dev).long(), w.to(dev), *ok(), None, 8, 32)
    with pytest.raises(ValueError):
        moe_sorting_flydsl(ids, w, *ok(), None, 8, 32)  # host tensors
    with pytest.raises(ValueError):
        moe_sorting_flydsl(ids.to(dev), w.to(dev), *ok(), None, 8, 32, None, 0)  # num_local_tokens outside [1, tokens]
    with pytest.raises(ValueError):
        moe_sorting_flydsl(ids.to(dev), w.to(dev), *ok(), None, 5000, 32)  # more experts than the kernel's histogram holds


@pytest.mark.parametrize("local", [40, torch.tensor([7], dtype=torch.int32)])
def test_num_local_tokens_sorts_only_the_first_rows(local):
    # the reference's expert-parallel token count (moe_sorting_kernel.py:2100-2104): the routing behaves as if it had that many tokens
    dev = torch.device("cuda")
    tokens, experts, topk, unit = 64, 16, 4, 16
    ids, w = _routing(tokens, experts, topk, 11)
    m = int(local.item()) if isinstance(local, torch.Tensor) else local
    rows, blocks = sorted_sizes(tokens, topk, experts, unit)
    s_ids = torch.full((rows,), -7, dtype=torch.int32, device=dev)
    s_w = torch.full((rows,), float("nan"), dtype=torch.float32, device=dev)
    s_e = torch.full((blocks,), -7, dtype=torch.int32, device=dev)
    nv = torch.full((2,), -7, dtype=torch.int32, device=dev)
    moe_sorting_flydsl(ids.to(dev), w.to(dev), s_ids, s_w, s_e, nv, None, experts, unit, None, local.to(dev) if isinstance(local, torch.Tensor) else local)
    torch.cuda.synchronize()
    want = O.moe_sorting(ids[:m].numpy(), w[:m].numpy(), experts, unit)
    n = want[0].size  # the oracle sizes its outputs for m tokens; the caller's are larger and padded the same way
    assert np.array_equal(s_ids.cpu().numpy()[:n], want[0]) and np.all(s_ids.cpu().numpy()[n:] == ((topk << 24) | m))
    assert np.array_equal(s_w.cpu().numpy()[:n], want[1]) and np.array_equal(nv.cpu().numpy(), want[3])
    nb = want[2].size
    assert np.array_equal(s_e.cpu().numpy()[:nb], want[2]) and np.all(s_e.cpu().numpy()[nb:] == -1)
    with pytest.raises(ValueError):
        moe_sorting_flydsl(ids.to(dev), w.to(dev), s_ids, s_w, s_e, nv, None, experts, unit, None, tokens + 1)


def test_random_routings_both_plans():
    # 40 random shapes around the borders of the kernels: 4096 pairs (one launch / three), 1024-pair slices, 64-pair chunks,
    # expert counts that are not powers of two, masks, ids outside the range
    rng = np.random.default_rng(2024)
    for case in range(40):
        experts = int(rng.choice([3, 8, 17, 32, 96, 129, 256, 1000]))
        topk = int(rng.integers(1, min(experts, 9) + 1))
        pairs = int(rng.choice([1, 63, 64, 65, 1023, 1025, 4095, 4097, 6000, 9000, 20000]))
        tokens = max(1, pairs // topk)
        unit = int(rng.choice([1, 16, 32, 64, 128]))
        ids = torch.from_numpy(rng.integers(0, experts, (tokens, topk)).astype(np.int32))
        if case % 5 == 0:
            ids[rng.integers(0, tokens), rng.integers(0, topk)] = experts + 3  # dropped by the kernel, as by the oracle
        w = torch.from_numpy(rng.random((tokens, topk), dtype=np.float32))
        mask = None
        if case % 3 == 0:
            mask = (rng.random(experts) < 0.7).astype(np.int32)
        valid = ids.clone()
        for workspace in (None, False):
            got = _run(valid, w, experts, unit, mask, workspace=workspace)
            want = O.moe_sorting(np.where(valid.numpy() < experts, valid.numpy(), -1), w.numpy(), experts, unit, expert_mask=mask)
            for name, a, b in zip(("sorted_ids", "sorted_weights", "sorted_expert_ids", "num_valid_ids"), got, want):
                assert np.array_equal(a, b), (case, name, tokens, experts, topk, unit, workspace)
