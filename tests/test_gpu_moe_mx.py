"""GPU parity of the fused MX-FP4 MoE stages against the CPU oracle, through the reference's call shapes
(kernels/moe/mxfp_moe/host.py; the reference's end-to-end check is tests/kernels/test_moe_gemm.py:540-818).

Stage 1 ends in a quantiser, so it is compared in three ways: the scale bytes (equal but for blocks whose maximum sits on a
power-of-two boundary, where the fp32 summation order decides: at most 0.5 % of the blocks, off by one), the codes (equal for
at least 99 % of the elements) and the dequantised values against the oracle's unquantised fp32 result (within one scale unit,
the widest half-step of e2m1, plus 1e-3 relative).  Stage 2 is checked on the DEVICE's stage-1 output, so its own error is
what is measured: |out-ref| <= 1e-2*|ref| + 1e-2*max|ref| for one row per sorted position, 3e-2*max|ref| for the atomic
epilogue (its 16-bit additions round in arrival order)."""

import numpy as np
import pytest
import torch

from flydsl_amd import layout
from kernels.moe.mxfp_moe import flydsl_mxfp4_gemm1, flydsl_mxfp4_gemm2
from oracle import psg_oracle as O

pytestmark = pytest.mark.gpu


def _problem(tokens, model_dim, inter, experts, topk, bm, a_fmt, seed, hot_expert=False):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((tokens, model_dim)).astype(np.float32)
    w1 = (rng.standard_normal((experts * 2 * inter, model_dim)) / np.sqrt(model_dim)).astype(np.float32)
    w2 = (rng.standard_normal((experts * model_dim, inter)) / np.sqrt(inter)).astype(np.float32)
    a_q, a_s = O.per_1x32_f4_quant(x) if a_fmt == "fp4" else O.per_1x32_f8_quant(x)
    w1_q, w1_s = O.per_1x32_f4_quant(w1)
    w2_q, w2_s = O.per_1x32_f4_quant(w2)
    ids = np.stack([rng.permutation(experts)[:topk] for _ in range(tokens)]).astype(np.int32)
    if hot_expert:
        ids[:, 0] = 1  # every token also goes to expert 1: several blocks of one expert
        ids[:, 1:] = np.where(ids[:, 1:] == 1, 0, ids[:, 1:])
    wts = rng.uniform(0.1, 1.0, size=(tokens, topk)).astype(np.float32)
    return dict(a_q=a_q, a_s=a_s[:tokens], w1_q=w1_q, w1_s=w1_s, w2_q=w2_q, w2_s=w2_s, ids=ids, wts=wts, sort=O.moe_sorting(ids, wts, experts, bm))


def _device_inputs(p, tokens, bm, dev):
    sid, sw, se, npp = p["sort"]
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    d = dict(a=t(p["a_q"]), w1=t(O.shuffle_weight_w4(p["w1_q"])), w2=t(O.shuffle_weight_w4(p["w2_q"])),
             w1_s=layout.e8m0_shuffle(t(p["w1_s"])), w2_s=layout.e8m0_shuffle(t(p["w2_s"])),
             sid=t(sid), sw=t(sw), se=t(se), cumsum=t(npp[:1].astype(np.int32)))
    d["a_s"] = layout.moe_mxfp4_sort(t(p["a_s"]).view(tokens, 1, -1), d["sid"], d["cumsum"], tokens, block_size=bm)
    return d


def _stage1(p, d, tokens, model_dim, inter, experts, topk, bm, a_fmt, dev):
    rows = int(d["sid"].numel())
    codes = torch.full((rows, inter // 2), 0x77, dtype=torch.uint8, device=dev)
    scales = torch.full(((rows + 255) // 256 * 256 * (inter // 32),), 0x77, dtype=torch.uint8, device=dev)
    flydsl_mxfp4_gemm1(a_quant=d["a"], a_scale_sorted_shuffled=d["a_s"], w1_u8=d["w1"], w1_scale_u8=d["w1_s"], sorted_expert_ids=d["se"],
                       cumsum_tensor=d["cumsum"], m_indices=d["sid"], inter_sorted_quant=codes, inter_sorted_shuffled_scale=scales,
                       hidden_states=None, n_tokens=tokens, BM=bm, use_nt=bm == 32, inline_quant=False, NE=experts, D_HIDDEN=model_dim,
                       D_INTER=inter, topk=topk, a_dtype=a_fmt)
    torch.cuda.synchronize()
    return codes, scales


def _check_stage1(p, codes, scales, tokens, inter, bm, a_fmt):
    sid, sw, se, npp = p["sort"]
    nv = int(npp[0])
    y, want_q, want_s = O.moe_mx_gemm1(p["a_q"], p["a_s"], p["w1_q"], p["w1_s"], sid, se, nv, tokens, inter, bm, a_fmt)
    got_q = codes.cpu().numpy()
    rows32 = (sid.size + 31) // 32 * 32
    got_s = O.e8m0_unshuffle(scales.cpu().numpy(), rows32, inter // 32)
    assert np.all(got_q[nv:] == 0x77), "rows past num_valid must stay untouched"
    live = (sid[:nv] & 0xFFFFFF) < tokens
    assert not got_q[:nv][~live].any() and not got_s[:nv][~live].any(), "padding rows hold zero codes and zero scales"
    ds = got_s[:nv][live].astype(np.int32) - want_s[:nv][live].astype(np.int32)
    if ds.size:  # small problems: one block on a boundary, a handful of elements on a rounding tie
        assert np.abs(ds).max() <= 1 and np.count_nonzero(ds) <= max(5e-3 * ds.size, 1), (np.abs(ds).max(), np.mean(ds != 0))
        assert np.count_nonzero(got_q[:nv][live] != want_q[:nv][live]) <= max(0.01 * got_q[:nv][live].size, 4)
    unit = np.repeat(np.ldexp(1.0, got_s[:nv].astype(np.int32) - 127), 32, axis=1) * (got_s[:nv] != 0).repeat(32, axis=1)
    deq = O.mxfp4_to_f32(got_q[:nv]) * unit
    assert np.all(np.abs(deq - y[:nv]) <= unit * 1.0 + 1e-3 * np.abs(y[:nv]) + 1e-30)
    return got_q, got_s


@pytest.mark.parametrize("a_fmt", ["fp4", "fp8"])
@pytest.mark.parametrize("bm", [32, 64, 128])
def test_fused_stages_match_the_oracle(bm, a_fmt):
    tokens, model_dim, inter, experts, topk = 70, 512, 256, 5, 2
    dev = torch.device("cuda")
    p = _problem(tokens, model_dim, inter, experts, topk, bm, a_fmt, seed=bm + len(a_fmt), hot_expert=True)
    d = _device_inputs(p, tokens, bm, dev)
    codes, scales = _stage1(p, d, tokens, model_dim, inter, experts, topk, bm, a_fmt, dev)
    got_q, got_s = _check_stage1(p, codes, scales, tokens, inter, bm, a_fmt)
    sid, sw, se, npp = p["sort"]
    nv, rows = int(npp[0]), sid.size
    clean_q, clean_s = got_q.copy(), got_s.copy()
    clean_q[nv:], clean_s[nv:] = 0, 0
    flat_ref, out_ref = O.moe_mx_gemm2(clean_q, clean_s[:rows], p["w2_q"], p["w2_s"], sid, sw, se, nv, tokens, model_dim, bm)
    common = dict(inter_sorted_quant=codes, inter_sorted_shuffled_scale=scales, w2_u8=d["w2"], w2_scale_u8=d["w2_s"], sorted_expert_ids=d["se"],
                  cumsum_tensor=d["cumsum"], sorted_token_ids=d["sid"], sorted_weights=d["sw"], M_logical=tokens, max_sorted=rows, BM=bm,
                  NE=experts, D_HIDDEN=model_dim, D_INTER=inter, topk=topk)
    for dt in (torch.bfloat16, torch.float16):
        flat = torch.full((rows, model_dim), 7.0, dtype=dt, device=dev)
        flydsl_mxfp4_gemm2(flat_out=flat, use_nt=False, epilog="nonatomic", **common)
        out = torch.zeros(tokens, model_dim, dtype=dt, device=dev)
        flydsl_mxfp4_gemm2(flat_out=out, use_nt=True, epilog="atomic", **common)
        torch.cuda.synchronize()
        f = flat.float().cpu().numpy()
        assert np.all(f[nv:] == 7.0)
        live = (sid[:nv] & 0xFFFFFF) < tokens
        tol = 1e-2 * np.abs(flat_ref[:nv][live]) + 1e-2 * np.abs(flat_ref).max()
        assert np.all(np.abs(f[:nv][live] - flat_ref[:nv][live]) <= tol)
        o = out.float().cpu().numpy()
        assert np.abs(o - out_ref).max() <= 3e-2 * np.abs(out_ref).max(), np.abs(o - out_ref).max() / np.abs(out_ref).max()


def test_blocks_of_masked_experts_are_skipped_and_longer_dims_work():
    tokens, model_dim, inter, experts, topk, bm = 33, 1024, 512, 4, 2, 32
    dev = torch.device("cuda")
    p = _problem(tokens, model_dim, inter, experts, topk, bm, "fp4", seed=9)
    sid, sw, se, npp = p["sort"]
    se = se.copy()
    masked = int(se[0])
    se[se == masked] = -1  # expert parallelism: blocks of experts that live elsewhere carry -1
    p["sort"] = (sid, sw, se, npp)
    d = _device_inputs(p, tokens, bm, dev)
    codes, scales = _stage1(p, d, tokens, model_dim, inter, experts, topk, bm, "fp4", dev)
    got_q = codes.cpu().numpy()
    nv = int(npp[0])
    skipped = np.repeat(se[: nv // bm] < 0, bm)
    assert np.all(got_q[:nv][skipped] == 0x77), "blocks of a masked expert are not written"
    y, want_q, want_s = O.moe_mx_gemm1(p["a_q"], p["a_s"], p["w1_q"], p["w1_s"], sid, se, nv, tokens, inter, bm, "fp4")
    assert np.mean(got_q[:nv][~skipped] == want_q[:nv][~skipped]) >= 0.99
    out = torch.zeros(tokens, model_dim, dtype=torch.bfloat16, device=dev)
    flydsl_mxfp4_gemm2(inter_sorted_quant=codes, inter_sorted_shuffled_scale=scales, w2_u8=d["w2"], w2_scale_u8=d["w2_s"], sorted_expert_ids=d["se"],
                       cumsum_tensor=d["cumsum"], sorted_token_ids=d["sid"], sorted_weights=d["sw"], flat_out=out, M_logical=tokens,
                       max_sorted=sid.size, BM=bm, use_nt=True, epilog="atomic", NE=experts, D_HIDDEN=model_dim, D_INTER=inter, topk=topk)
    torch.cuda.synchronize()
    got_s = O.e8m0_unshuffle(scales.cpu().numpy(), (sid.size + 31) // 32 * 32, inter // 32)
    q, s = got_q.copy(), got_s.copy()
    q[nv:], s[nv:] = 0, 0
    q[:nv][skipped], s[:nv][skipped] = 0, 0
    _, out_ref = O.moe_mx_gemm2(q, s[: sid.size], p["w2_q"], p["w2_s"], sid, sw, se, nv, tokens, model_dim, bm)
    assert np.abs(out.float().cpu().numpy() - out_ref).max() <= 3e-2 * np.abs(out_ref).max()


@pytest.mark.parametrize("tokens,model_dim", [(5, 512), (70, 512), (21, 7424)])
def test_blocks_of_16_rows_quantise_bf16_activations_in_the_kernel(tokens, model_dim):
    """The reference's inline_quant variant (gemm1.py:324-412; tests/kernels/test_moe_gemm.py:856): stage 1 reads bf16 rows and
    quantises them itself.  The oracle quantises the same bf16 values with the same rule and runs the pre-quantised path.
    One case has long rows (7424 elements: 58 K steps, an odd number of 256-element scale chunks)."""
    inter, experts, topk, bm = 256, 6, 3, 16
    dev = torch.device("cuda")
    p = _problem(tokens, model_dim, inter, experts, topk, bm, "fp4", seed=40 + tokens, hot_expert=tokens > 16)
    g = torch.Generator().manual_seed(tokens)
    hidden = (torch.randn(tokens, model_dim, generator=g) * torch.exp(torch.randn(tokens, 1, generator=g))).to(torch.bfloat16)
    hidden[0, 32:64] = 0
    p["a_q"], p["a_s"] = O.mxfp4_requant_roundup(hidden.float().numpy())
    sid, sw, se, npp = p["sort"]
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    d = dict(w1=t(O.shuffle_weight_w4(p["w1_q"])), w2=t(O.shuffle_weight_w4(p["w2_q"])), w1_s=layout.e8m0_shuffle(t(p["w1_s"])),
             w2_s=layout.e8m0_shuffle(t(p["w2_s"])), sid=t(sid), sw=t(sw), se=t(se), cumsum=t(npp[:1].astype(np.int32)))
    rows = sid.size
    codes = torch.full((rows, inter // 2), 0x77, dtype=torch.uint8, device=dev)
    scales = torch.full(((rows + 255) // 256 * 256 * (inter // 32),), 0x77, dtype=torch.uint8, device=dev)
    dummy = torch.zeros(16, dtype=torch.uint8, device=dev)
    flydsl_mxfp4_gemm1(a_quant=dummy, a_scale_sorted_shuffled=dummy, w1_u8=d["w1"], w1_scale_u8=d["w1_s"], sorted_expert_ids=d["se"],
                       cumsum_tensor=d["cumsum"], m_indices=d["sid"], inter_sorted_quant=codes, inter_sorted_shuffled_scale=scales,
                       hidden_states=hidden.to(dev), n_tokens=tokens, BM=bm, use_nt=True, inline_quant=True, NE=experts, D_HIDDEN=model_dim,
                       D_INTER=inter, topk=topk, a_dtype="fp4")
    torch.cuda.synchronize()
    got_q, got_s = _check_stage1(p, codes, scales, tokens, inter, bm, "fp4")
    nv = int(npp[0])
    q, s = got_q.copy(), got_s.copy()
    q[nv:], s[nv:] = 0, 0
    flat_ref, out_ref = O.moe_mx_gemm2(q, s[:rows], p["w2_q"], p["w2_s"], sid, sw, se, nv, tokens, model_dim, bm)
    common = dict(inter_sorted_quant=codes, inter_sorted_shuffled_scale=scales, w2_u8=d["w2"], w2_scale_u8=d["w2_s"], sorted_expert_ids=d["se"],
                  cumsum_tensor=d["cumsum"], sorted_token_ids=d["sid"], sorted_weights=d["sw"], M_logical=tokens, max_sorted=rows, BM=bm,
                  NE=experts, D_HIDDEN=model_dim, D_INTER=inter, topk=topk)
    flat = torch.full((rows, model_dim), 7.0, dtype=torch.bfloat16, device=dev)
    flydsl_mxfp4_gemm2(flat_out=flat, use_nt=False, epilog="nonatomic", **common)
    out = torch.zeros(tokens, model_dim, dtype=torch.bfloat16, device=dev)
    flydsl_mxfp4_gemm2(flat_out=out, use_nt=True, epilog="atomic", **common)
    torch.cuda.synchronize()
    f = flat.float().cpu().numpy()
    assert np.all(f[nv:] == 7.0)
    live = (sid[:nv] & 0xFFFFFF) < tokens
    tol = 1e-2 * np.abs(flat_ref[:nv][live]) + 1e-2 * np.abs(flat_ref).max()
    assert np.all(np.abs(f[:nv][live] - flat_ref[:nv][live]) <= tol)
    assert np.abs(out.float().cpu().numpy() - out_ref).max() <= 3e-2 * np.abs(out_ref).max()


def test_random_problems_over_every_block_size_and_activation_format():
    """Sixteen seeded problems: token counts from 1 up, experts without tokens, top-k up to the expert count, widths from the
    smallest (256) to several column tiles with tile counts that are and are not multiples of 8, every block size with each of its
    activation formats, both stage-2 epilogues."""
    dev = torch.device("cuda")
    rng = np.random.default_rng(2024)
    variants = [(32, "fp4"), (64, "fp4"), (128, "fp4"), (32, "fp8"), (64, "fp8"), (128, "fp8"), (16, "bf16")]
    for case in range(16):
        bm, a_fmt = variants[case % len(variants)]
        tokens = int(rng.choice([1, 2, 7, 16, 33, 100, 257]))
        experts = int(rng.choice([1, 3, 8, 24]))
        topk = int(rng.integers(1, min(experts, 6) + 1))
        model_dim = 256 * int(rng.choice([1, 2, 3, 5]))
        inter = 256 * int(rng.choice([1, 2, 3, 5]))
        print(f"case {case}: bm={bm} a={a_fmt} tokens={tokens} experts={experts} topk={topk} model_dim={model_dim} inter={inter}", flush=True)
        p = _problem(tokens, model_dim, inter, experts, topk, bm, "fp8" if a_fmt == "fp8" else "fp4", seed=1000 + case)
        sid, sw, se, npp = p["sort"]
        rows, nv = sid.size, int(npp[0])
        if a_fmt == "bf16":
            g = torch.Generator().manual_seed(case)
            hidden = torch.randn(tokens, model_dim, generator=g).to(torch.bfloat16)
            p["a_q"], p["a_s"] = O.mxfp4_requant_roundup(hidden.float().numpy())
        d = _device_inputs(p, tokens, max(bm, 32), dev)
        codes = torch.full((rows, inter // 2), 0x77, dtype=torch.uint8, device=dev)
        scales = torch.full(((rows + 255) // 256 * 256 * (inter // 32),), 0x77, dtype=torch.uint8, device=dev)
        extra = dict(inline_quant=True, hidden_states=hidden.to(dev), a_dtype="fp4") if a_fmt == "bf16" else dict(a_dtype=a_fmt)
        flydsl_mxfp4_gemm1(a_quant=d["a"], a_scale_sorted_shuffled=d["a_s"], w1_u8=d["w1"], w1_scale_u8=d["w1_s"], sorted_expert_ids=d["se"],
                           cumsum_tensor=d["cumsum"], m_indices=d["sid"], inter_sorted_quant=codes, inter_sorted_shuffled_scale=scales,
                           n_tokens=tokens, BM=bm, NE=experts, D_HIDDEN=model_dim, D_INTER=inter, topk=topk, **extra)
        torch.cuda.synchronize()
        got_q, got_s = _check_stage1(p, codes, scales, tokens, inter, bm, "fp8" if a_fmt == "fp8" else "fp4")
        q, s2 = got_q.copy(), got_s.copy()
        q[nv:], s2[nv:] = 0, 0
        flat_ref, out_ref = O.moe_mx_gemm2(q, s2[:rows], p["w2_q"], p["w2_s"], sid, sw, se, nv, tokens, model_dim, bm)
        common = dict(inter_sorted_quant=codes, inter_sorted_shuffled_scale=scales, w2_u8=d["w2"], w2_scale_u8=d["w2_s"], sorted_expert_ids=d["se"],
                      cumsum_tensor=d["cumsum"], sorted_token_ids=d["sid"], sorted_weights=d["sw"], M_logical=tokens, max_sorted=rows, BM=bm,
                      NE=experts, D_HIDDEN=model_dim, D_INTER=inter, topk=topk)
        flat = torch.full((rows, model_dim), 7.0, dtype=torch.bfloat16, device=dev)
        flydsl_mxfp4_gemm2(flat_out=flat, epilog="nonatomic", **common)
        out = torch.zeros(tokens, model_dim, dtype=torch.bfloat16, device=dev)
        flydsl_mxfp4_gemm2(flat_out=out, epilog="atomic", **common)
        torch.cuda.synchronize()
        f = flat.float().cpu().numpy()
        assert np.all(f[nv:] == 7.0)
        live = (sid[:nv] & 0xFFFFFF) < tokens
        scale = max(float(np.abs(flat_ref).max()), 1e-30)
        assert np.all(np.abs(f[:nv][live] - flat_ref[:nv][live]) <= 1e-2 * np.abs(flat_ref[:nv][live]) + 1e-2 * scale), case
        assert np.abs(out.float().cpu().numpy() - out_ref).max() <= 3e-2 * max(float(np.abs(out_ref).max()), 1e-30), case


def test_device_scale_sort_matches_the_oracle_byte_for_byte():
    from kernels.moe.mxfp_moe import moe_mxfp4_sort

    dev = torch.device("cuda")
    rng = np.random.default_rng(77)
    for tokens, topk, cols, n_ids, nv in ((11, 3, 16, 58, 48), (1, 1, 8, 32, 32), (300, 8, 128, 4000, 3968), (40, 2, 24, 100, 100)):
        ids = rng.integers(0, tokens + 3, size=n_ids).astype(np.int64)  # some ids at or past `tokens`: padding
        ids = (ids | (rng.integers(0, topk, size=n_ids) << 24)).astype(np.int32)
        for sc in (rng.integers(1, 255, size=(tokens, cols), dtype=np.uint8), rng.integers(1, 255, size=(tokens, topk, cols), dtype=np.uint8)):
            want = O.moe_mxfp4_sort(sc, ids, nv, tokens)
            out = torch.full((want.shape[0] + 32, cols), 0x5A, dtype=torch.uint8, device=dev)
            got = moe_mxfp4_sort(torch.from_numpy(sc).to(dev), torch.from_numpy(ids).to(dev), torch.tensor([nv, tokens], dtype=torch.int32, device=dev),
                                 tokens, out=out)
            torch.cuda.synchronize()
            g = got.cpu().numpy()
            assert np.array_equal(g.reshape(-1)[: want.size], want.reshape(-1))
            assert np.all(g.reshape(-1)[want.size :] == 0x5A), "nothing past ceil(rows/32)*32 rows is written"


def test_layer_from_bf16_activations_runs_on_the_device_and_replays_in_a_graph():
    """bf16 hidden state -> device MX-FP4 quantiser -> device scale sort -> stage 1 -> stage 2 (atomic), caller-owned buffers only;
    eager once, then captured into a HIP graph and replayed three times with eager work in between.  The oracle quantises the same
    hidden state with the host rule the device quantiser is byte-equal to."""
    from flydsl_amd import quant_device
    from kernels.moe.mxfp_moe import moe_mxfp4_sort

    tokens, model_dim, inter, experts, topk, bm = 45, 768, 512, 7, 3, 32
    dev = torch.device("cuda")
    p = _problem(tokens, model_dim, inter, experts, topk, bm, "fp4", seed=91)
    hidden = torch.randn(tokens, model_dim, generator=torch.Generator().manual_seed(3)).to(torch.bfloat16)
    p["a_q"], a_s = O.per_1x32_f4_quant(hidden.float().numpy())
    p["a_s"] = a_s[:tokens]
    sid, sw, se, npp = p["sort"]
    rows, nv = sid.size, int(npp[0])
    d = _device_inputs(p, tokens, bm, dev)
    hid = hidden.to(dev)
    a_q = torch.empty(tokens, model_dim // 2, dtype=torch.uint8, device=dev)
    a_s_rm = torch.empty((tokens + 31) // 32 * 32, model_dim // 32, dtype=torch.uint8, device=dev)
    a_s_sorted = torch.empty((rows + 31) // 32 * 32, model_dim // 32, dtype=torch.uint8, device=dev)
    codes = torch.full((rows, inter // 2), 0x77, dtype=torch.uint8, device=dev)
    scales = torch.full(((rows + 255) // 256 * 256 * (inter // 32),), 0x77, dtype=torch.uint8, device=dev)
    out = torch.zeros(tokens, model_dim, dtype=torch.bfloat16, device=dev)

    def layer():
        out.zero_()
        quant_device.per_1x32_f4_quant(hid, shuffle=False, out=(a_q, a_s_rm))
        moe_mxfp4_sort(a_s_rm[:tokens], d["sid"], d["cumsum"], tokens, block_size=bm, out=a_s_sorted)
        flydsl_mxfp4_gemm1(a_quant=a_q, a_scale_sorted_shuffled=a_s_sorted, w1_u8=d["w1"], w1_scale_u8=d["w1_s"], sorted_expert_ids=d["se"],
                           cumsum_tensor=d["cumsum"], m_indices=d["sid"], inter_sorted_quant=codes, inter_sorted_shuffled_scale=scales,
                           n_tokens=tokens, BM=bm, NE=experts, D_HIDDEN=model_dim, D_INTER=inter, topk=topk)
        flydsl_mxfp4_gemm2(inter_sorted_quant=codes, inter_sorted_shuffled_scale=scales, w2_u8=d["w2"], w2_scale_u8=d["w2_s"], sorted_expert_ids=d["se"],
                           cumsum_tensor=d["cumsum"], sorted_token_ids=d["sid"], sorted_weights=d["sw"], flat_out=out, M_logical=tokens,
                           max_sorted=rows, BM=bm, epilog="atomic", NE=experts, D_HIDDEN=model_dim, D_INTER=inter, topk=topk)

    layer()
    torch.cuda.synchronize()
    assert np.array_equal(a_q.cpu().numpy(), p["a_q"]) and np.array_equal(a_s_sorted.cpu().numpy(), d["a_s"].cpu().numpy())
    got_q, got_s = _check_stage1(p, codes, scales, tokens, inter, bm, "fp4")
    q, s2 = got_q.copy(), got_s.copy()
    q[nv:], s2[nv:] = 0, 0
    _, out_ref = O.moe_mx_gemm2(q, s2[:rows], p["w2_q"], p["w2_s"], sid, sw, se, nv, tokens, model_dim, bm)
    tol = 3e-2 * float(np.abs(out_ref).max())
    assert np.abs(out.float().cpu().numpy() - out_ref).max() <= tol
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        layer()
        side.synchronize()
        with torch.cuda.graph(g, stream=side):
            layer()
    torch.cuda.synchronize()
    for _ in range(3):
        out.fill_(5.0)
        codes.fill_(0x33)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert np.array_equal(codes.cpu().numpy()[:nv], got_q[:nv])
        assert np.abs(out.float().cpu().numpy() - out_ref).max() <= tol


def test_unbuilt_variants_raise_like_the_reference():
    dev = torch.device("cuda")
    z = torch.zeros(64, dtype=torch.uint8, device=dev)
    base = dict(a_quant=z, a_scale_sorted_shuffled=z, w1_u8=z, w1_scale_u8=z, sorted_expert_ids=z, cumsum_tensor=z, m_indices=z,
                inter_sorted_quant=z, inter_sorted_shuffled_scale=z, hidden_states=z, n_tokens=4, use_nt=False, NE=2, D_HIDDEN=512, D_INTER=256, topk=1)
    with pytest.raises(NotImplementedError):
        flydsl_mxfp4_gemm1(BM=32, inline_quant=True, **base)
    with pytest.raises(NotImplementedError):
        flydsl_mxfp4_gemm1(BM=16, inline_quant=False, **base)
    with pytest.raises(NotImplementedError):
        flydsl_mxfp4_gemm1(BM=16, inline_quant=True, a_dtype="fp8", **base)
    with pytest.raises(NotImplementedError):
        flydsl_mxfp4_gemm1(BM=32, inline_quant=False, interleave=True, **base)
    with pytest.raises(NotImplementedError):
        flydsl_mxfp4_gemm1(BM=32, inline_quant=False, **{**base, "D_HIDDEN": 384})
    g2 = dict(inter_sorted_quant=z, inter_sorted_shuffled_scale=z, w2_u8=z, w2_scale_u8=z, sorted_expert_ids=z, cumsum_tensor=z, sorted_token_ids=z,
              sorted_weights=z, flat_out=z, M_logical=4, max_sorted=32, BM=32, use_nt=False, NE=2, D_HIDDEN=512, D_INTER=256, topk=1)
    with pytest.raises(NotImplementedError):
        flydsl_mxfp4_gemm2(epilog="nonatomic_mxfp4", **g2)
    with pytest.raises(NotImplementedError):
        flydsl_mxfp4_gemm2(epilog="atomic", **{**g2, "D_INTER": 320})
    # a pointer is all the library sees: wrong element types are refused before anything is launched
    i32 = torch.zeros(64, dtype=torch.int32, device=dev)
    ok1 = {**base, "sorted_expert_ids": i32, "cumsum_tensor": i32, "m_indices": i32}
    with pytest.raises(TypeError):
        flydsl_mxfp4_gemm1(BM=32, **{**ok1, "m_indices": i32.long()})
    with pytest.raises(TypeError):
        flydsl_mxfp4_gemm1(BM=32, **{**ok1, "cumsum_tensor": i32.cpu()})
    with pytest.raises(ValueError):
        flydsl_mxfp4_gemm1(BM=32, **ok1)  # 64 bytes of weights
    with pytest.raises(TypeError):
        flydsl_mxfp4_gemm2(epilog="atomic", **{**g2, "sorted_expert_ids": i32, "cumsum_tensor": i32, "sorted_token_ids": i32, "sorted_weights": i32})
