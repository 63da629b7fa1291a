#!/usr/bin/env python3
"""Benchmark of the preshuffle quantized GEMM on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-others] [--no-cpu] [--next-rows [--next-rows-only SECTION]] [--reference-shapes]

A step is one GEMM launch on one set of synthetic operands (seed 0; activations N(0,1), weights
N(0,0.02), quantised and preshuffled on the host, resident in HBM before the timed region).
Steps rotate through enough independent operand sets that the weights cannot be served from the
256 MB Infinity Cache.  The K timed steps are recorded once into a HIP graph; the graph is replayed as often as
it takes to time at least 50 ms of work (a K-step graph of a 7 us kernel is far too short to time once), bracketed
by ``torch.cuda.synchronize()`` on both sides (wall clock -> ``value`` / ``ms_per_step``) and by HIP events
on the launch stream (-> ``roofline.achieved``).  Prints ONE JSON line.
"""

from __future__ import annotations

import argparse
import ctypes
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# name -> (family, dtype label, M, N, K, roofline bound)
WORKLOADS = {
    "fp8_decode_m1": ("a8w8", "fp8", 1, 6144, 4096, "hbm"),
    "fp8_decode_m16": ("a8w8", "fp8", 16, 6144, 4096, "hbm"),
    "fp8_decode_m32": ("a8w8", "fp8", 32, 6144, 4096, "hbm"),
    "fp8_prefill_m8192": ("a8w8", "fp8", 8192, 4096, 4096, "mfma"),
    "int8_ffn_m4096": ("a8w8", "int8", 4096, 28672, 8192, "mfma"),
    "mxfp4_m32": ("mxfp4", "fp4", 32, 7168, 2048, "hbm"),
    "mxfp4_m4096": ("mxfp4", "fp4", 4096, 7168, 2048, "mfma"),
    "int8_plumbing_m128": ("a8w8", "int8", 128, 1024, 1024, "mfma"),
    "bf16_m5120": ("a16w16", "bf16", 5120, 5120, 8320, "mfma"),
}
DEFAULT_WORKLOAD = "fp8_decode_m16"
PEAK = {"hbm": 8000.0, "fp8": 5000.0, "int8": 5000.0, "fp4": 10100.0, "bf16": 2500.0, "fp16": 2500.0}  # GB/s, TFLOP/s (dense, published)
MALL_BYTES = 256 << 20
MIN_TIMED_S = 0.05  # every timed region holds at least this much GPU work


def algorithmic_bytes(family, M, N, K):
    if family == "a8w8":
        return M * K + N * K + 2 * M * N + 4 * (M + N)
    if family == "a16w16":
        return 2 * M * K + 2 * N * K + 2 * M * N
    return M * K // 2 + N * K // 2 + 2 * M * N + (M + N) * (K // 32)


def make_launcher(family, kind, M, N, K):
    import torch

    if family in ("a8w8", "a16w16"):
        from kernels.gemm.preshuffle_gemm import compile_preshuffle_gemm

        fn = compile_preshuffle_gemm(N=N, K=K, tile_m=128, tile_n=256, tile_k=64, in_dtype=kind)
        bias = torch.empty(0, dtype=torch.bfloat16, device="cuda")

        def launch(s):
            fn(s["c"], s["a"], s["b"], s["sa"], s["sb"], bias, M, N, torch.cuda.current_stream())
    else:
        from kernels.gemm.mxfp4_preshuffle import launch_gemm

        def launch(s):
            launch_gemm(s["c"], s["a"], s["b"], s["sa"], s["sb"], M, N, torch.cuda.current_stream(), N, K, 64, 256, 256,
                        "fp4", "bf16", "fp4", 1, -1, -1, -1, -1, -1, -1, 0, 0)
    return launch


def run_workload(name, steps, warmup, check=True):
    import numpy as np
    import torch

    family, kind, M, N, K, bound = WORKLOADS[name]
    dev = torch.device("cuda:0")
    nbytes = algorithmic_bytes(family, M, N, K)
    flops = 2.0 * M * N * K
    # enough operand sets that one pass over them exceeds twice the Infinity Cache
    n_sets = max(2, min(32, math.ceil(2 * MALL_BYTES / nbytes)))
    if nbytes * n_sets > (8 << 30):
        n_sets = max(2, (8 << 30) // nbytes)
    from flydsl_amd.synthetic import make_a8w8, make_a16w16, make_mxfp4

    if family == "a8w8":
        host = make_a8w8(M, N, K, kind, seed=0)
    elif family == "a16w16":
        host = make_a16w16(M, N, K, kind, seed=0, w_std=0.02)
    else:
        host = make_mxfp4(M, N, K, seed=0)
    sets = []
    for i in range(n_sets):
        if family == "a16w16":
            none = torch.empty(0, dtype=torch.float32, device=dev)
            s = {"a": host["a_q"].to(dev), "b": host["b_shuf"].to(dev), "sa": none, "sb": none}
        elif family == "a8w8":
            s = {"a": host["a_q"].to(dev), "b": host["b_shuf"].to(dev), "sa": host["sa"].to(dev), "sb": host["sb"].to(dev)}
        else:
            s = {"a": host["a_q"].to(dev), "b": host["b_shuf"].to(dev), "sa": host["sa_shuf"].to(dev), "sb": host["sb_shuf"].to(dev)}
        s["c"] = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
        sets.append(s)
    launch = make_launcher(family, kind, M, N, K)

    for i in range(warmup):
        launch(sets[i % n_sets])
    torch.cuda.synchronize()

    # record the K timed steps into one graph on a side stream
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        for i in range(steps):
            launch(sets[i % n_sets])
    torch.cuda.synchronize()
    graph.replay()  # untimed: first replay uploads the graph
    torch.cuda.synchronize()

    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    # one timed probe replay sizes the number of replays so that every timed region holds at least MIN_TIMED_S of work
    torch.cuda.synchronize()
    ev0.record()
    graph.replay()
    ev1.record()
    torch.cuda.synchronize()
    replays = max(1, math.ceil(MIN_TIMED_S / max(ev0.elapsed_time(ev1) * 1e-3, 1e-7)))
    best_wall, best_ev = float("inf"), float("inf")
    for _ in range(3):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ev0.record()
        for _r in range(replays):
            graph.replay()
        ev1.record()
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        best_wall = min(best_wall, wall)
        best_ev = min(best_ev, ev0.elapsed_time(ev1) * 1e-3)
    sec_per_step = best_wall / (steps * replays)
    kernel_s = best_ev / (steps * replays)

    # hot-cache figure (one operand set): informative only
    ghot = torch.cuda.CUDAGraph()
    with torch.cuda.graph(ghot, stream=side):
        for i in range(steps):
            launch(sets[0])
    torch.cuda.synchronize()
    ghot.replay()
    torch.cuda.synchronize()
    ev0.record()
    for _r in range(replays):
        ghot.replay()
    ev1.record()
    torch.cuda.synchronize()
    hot_s = ev0.elapsed_time(ev1) * 1e-3 / (steps * replays)

    ok = None
    if check:
        from oracle import psg_oracle as O

        out = sets[(steps - 1) % n_sets]["c"].float().cpu().numpy()
        rows = np.arange(M) if M <= 256 else np.array(sorted({(i * 131 + 7) % M for i in range(64)}))
        if family == "a16w16":
            ref = O.run_torch(host["a_q"].view(torch.int16).numpy().view(np.uint16)[rows],
                              host["b_q"].view(torch.int16).numpy().view(np.uint16), None, None, kind)
        elif family == "a8w8":
            ref = O.run_torch(host["a_q"].view(torch.uint8).numpy()[rows], host["b_q"].view(torch.uint8).numpy(),
                              host["sa"].numpy()[rows], host["sb"].numpy(), kind)
        else:
            ref = O.run_torch_w4(host["a_q"].numpy()[rows], host["b_q"].numpy(), host["sa"].numpy()[:M][rows], host["sb"].numpy())
        bound_abs = 1e-2 * np.abs(ref) + 1e-2 * np.abs(ref).max()
        ok = bool(np.all(np.abs(out[rows] - ref) <= bound_abs))

    if bound == "hbm":
        achieved, peak, unit = nbytes / kernel_s / 1e9, PEAK["hbm"], "GB/s"
    else:
        achieved, peak, unit = flops / kernel_s / 1e12, PEAK[kind], "TFLOP/s"
    res = {
        "workload": name, "dtype": kind, "M": M, "N": N, "K": K,
        "tflops": flops / sec_per_step / 1e12, "gb_per_s": nbytes / sec_per_step / 1e9,
        "us_per_step_wall": sec_per_step * 1e6, "us_per_launch_events": kernel_s * 1e6, "us_per_launch_hot_cache": hot_s * 1e6,
        "operand_sets": n_sets, "graph_replays_per_timing": replays, "parity_ok": ok,
        "roofline": {"bound": bound, "achieved": achieved, "peak": peak, "unit": unit, "frac": achieved / peak,
                     "traffic": None, "algorithmic_bytes": nbytes, "flops": flops},
    }
    del graph, ghot, sets
    torch.cuda.empty_cache()
    return res, host


def run_quant_workload(name, steps=50, warmup=5):
    """The on-device quantisers that feed the GEMM: bf16 activations [M,K] -> fp8 + per-row scales, or -> MXFP4 + shuffled
    e8m0 scales.  HBM-bound; algorithmic bytes = input + outputs, each touched once."""
    import numpy as np
    import torch

    from flydsl_amd import quant_device
    from oracle import psg_oracle as O

    kind, M, K = {"quant_pertoken_fp8_m8192": ("fp8", 8192, 4096), "quant_mxfp4_m4096": ("fp4", 4096, 2048)}[name]
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(0)
    host = torch.randn(M, K, generator=g).to(torch.bfloat16)
    n_sets = max(2, min(32, math.ceil(2 * MALL_BYTES / (M * K * 2))))
    xs = [host.to(dev) for _ in range(n_sets)]
    if kind == "fp8":
        out = (torch.empty(M, K, dtype=torch.uint8, device=dev), torch.empty(M, 1, dtype=torch.float32, device=dev))
        f = lambda x: quant_device.pertoken_quant(x, quant_dtype=torch.float8_e4m3fn, stream=torch.cuda.current_stream(), out=out)  # noqa: E731
        nbytes = M * K * 2 + M * K + M * 4
    else:
        out = (torch.empty(M, K // 2, dtype=torch.uint8, device=dev), torch.empty(M, K // 32, dtype=torch.uint8, device=dev))
        f = lambda x: quant_device.per_1x32_f4_quant(x, shuffle=True, stream=torch.cuda.current_stream(), out=out)  # noqa: E731
        nbytes = M * K * 2 + M * K // 2 + M * K // 32
    for i in range(warmup):
        f(xs[i % n_sets])
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        for i in range(steps):
            f(xs[i % n_sets])
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    ev0.record()
    graph.replay()
    ev1.record()
    torch.cuda.synchronize()
    # one timed probe replay sizes the number of replays so that the timed region holds at least MIN_TIMED_S of work
    replays = max(1, math.ceil(MIN_TIMED_S / max(ev0.elapsed_time(ev1) * 1e-3, 1e-7)))
    ev0.record()
    for _r in range(replays):
        graph.replay()
    ev1.record()
    torch.cuda.synchronize()
    sec = ev0.elapsed_time(ev1) * 1e-3 / (steps * replays)
    if kind == "fp8":
        wy, ws = O.pertoken_quant(host.float().numpy(), "fp8")
        ok = bool(np.array_equal(out[0].view(torch.uint8).cpu().numpy(), wy) and np.array_equal(out[1].cpu().numpy(), ws))
    else:
        wp, ws = O.per_1x32_f4_quant(host.float().numpy())
        ok = bool(np.array_equal(out[0].view(torch.uint8).cpu().numpy(), wp) and
                  np.array_equal(out[1].view(torch.uint8).cpu().numpy(), O.shuffle_scale_w4(ws)))
    achieved = nbytes / sec / 1e9
    return {"workload": name, "dtype": kind, "M": M, "K": K, "gb_per_s": achieved, "us_per_launch_events": sec * 1e6,
            "operand_sets": n_sets, "graph_replays_per_timing": replays, "parity_ok": ok, "timing": "graph replay, caller-owned outputs, HIP events",
            "roofline": {"bound": "hbm", "achieved": achieved, "peak": PEAK["hbm"], "unit": "GB/s", "frac": achieved / PEAK["hbm"],
                         "traffic": load_traffic(name), "algorithmic_bytes": nbytes}}


def run_next_row_workloads(only=None):
    """Timings of the kernels of the rows next to the hot path (``--next-rows``): the general MX kernel on the reference's
    test shapes and the two MoE stages.  HIP events around plain launch loops (every kernel here runs for >= 15 us, so
    launch gaps hide behind the previous kernel); weights sized beyond the Infinity Cache where the shape allows."""
    import math as _m

    import torch

    from flydsl_amd import layout, quant
    from flydsl_amd.kernels.moe.moe_sorting import moe_sorting, moe_sorting_flydsl, moe_sorting_get_workspace_size, sorted_sizes
    from flydsl_amd.synthetic import make_mx
    from kernels.gemm.mxfp4_preshuffle import launch_gemm
    from kernels.moe.moe_gemm_2stage import compile_moe_gemm1, compile_moe_gemm2

    dev = torch.device("cuda:0")

    def timed(f, iters=20):
        for _ in range(3):
            f()
        torch.cuda.synchronize()
        best = float("inf")
        for _ in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(iters):
                f()
            e1.record()
            torch.cuda.synchronize()
            best = min(best, e0.elapsed_time(e1) * 1e-3 / iters)
        return best

    out = []
    want = lambda section: only is None or only == section  # noqa: E731  (--next-rows-only: one section, e.g. under a profiler)
    for af, bf in (("fp8", "fp8"), ("fp6", "fp4"), ("fp8", "fp4")) if want("mx") else ():
        for M in (1024, 64, 32):
            N = K = 8192
            d = make_mx(min(M, 256), 512, K, af, bf, seed=0)
            rep = lambda t, n: t.repeat((n + t.shape[0] - 1) // t.shape[0], 1)[:n].contiguous().to(dev)  # noqa: E731
            a, b = rep(d["a_q"], M), rep(d["b_shuf"].view(512, -1), N)
            sa = d["sa_shuf"].view(-1).repeat((M + 255) // 256 + 1).contiguous().to(dev)
            sb = d["sb_shuf"].view(-1).repeat(N // 512).contiguous().to(dev)
            c = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
            sec = timed(lambda: launch_gemm(c, a, b, sa, sb, M, N, None, N, K, 64, 256, 256, af, "bf16", bf, 1, -1, -1, -1, -1, -1, -1, 0, 0))
            wbytes = N * K // (2 if bf == "fp4" else 1)
            out.append({"workload": f"mx_{af}x{bf}_m{M}_n8192_k8192", "us_per_launch_events": sec * 1e6, "tflops": 2.0 * M * N * K / sec / 1e12,
                        "weight_gb_per_s": wbytes / sec / 1e9})
    for tokens, model_dim, inter_dim, experts, topk, tile_m in ((4096, 4096, 1536, 32, 8, 128), (64, 4096, 1536, 32, 8, 16), (333, 4096, 2048, 17, 9, 64)) if want("moe_fp8") else ():
        g = torch.Generator().manual_seed(0)
        vals, ids = torch.topk(torch.rand(tokens, experts, generator=g), k=topk, dim=1)
        sid, swt, se, npp = moe_sorting(ids.int().to(dev), torch.softmax(vals, 1).to(dev), num_experts=experts, block_size=tile_m)  # device sorter
        qd = torch.float8_e4m3fn
        xq, sx = quant.pertoken_quant(torch.randn(tokens, model_dim, generator=g), quant_dtype=qd)
        w1q = layout.shuffle_weight((torch.randn(experts * 2 * inter_dim, model_dim, generator=g) / _m.sqrt(model_dim) * 40).to(qd))
        w2q = layout.shuffle_weight((torch.randn(experts * model_dim, inter_dim, generator=g) / _m.sqrt(inter_dim) * 40).to(qd))
        a2q, sa2 = quant.pertoken_quant(torch.randn(tokens * topk, inter_dim, generator=g), quant_dtype=qd)
        sw1 = torch.full((experts * 2 * inter_dim,), 0.025, device=dev)
        sw2 = torch.full((experts * model_dim,), 0.025, device=dev)
        xq, w1q, w2q, a2q, sx, sa2 = [t.to(dev).contiguous().view(-1) for t in (xq, w1q, w2q, a2q, sx, sa2)]
        out1 = torch.empty(tokens, topk, inter_dim, dtype=torch.bfloat16, device=dev)
        out2 = torch.zeros(tokens, model_dim, dtype=torch.bfloat16, device=dev)
        nv, blocks = npp[:1].contiguous(), int(se.numel())
        kw = dict(model_dim=model_dim, inter_dim=inter_dim, experts=experts, topk=topk, tile_m=tile_m, tile_n=128, tile_k=128, in_dtype="fp8")
        e1 = compile_moe_gemm1(doweight_stage1=False, out_dtype="bf16", **kw)
        e2 = compile_moe_gemm2(doweight_stage2=True, out_dtype="bf16", accumulate=True, **kw)
        s1 = timed(lambda: e1(out1, xq, w1q, sx, sw1, sid, se, swt, nv, tokens, inter_dim, model_dim, blocks, None))
        s2 = timed(lambda: e2(out2, a2q, w2q, sa2, sw2, sid, se, swt, nv, tokens, model_dim, inter_dim, blocks, None))
        tag = f"tokens{tokens}_e{experts}_top{topk}_model{model_dim}_inter{inter_dim}_block{tile_m}"
        out.append({"workload": f"moe_fp8_stage1_{tag}", "us_per_launch_events": s1 * 1e6, "tflops": 2.0 * tokens * topk * 2 * inter_dim * model_dim / s1 / 1e12,
                    "weight_gb_per_s": experts * 2 * inter_dim * model_dim / s1 / 1e9})
        out.append({"workload": f"moe_fp8_stage2_atomic_{tag}", "us_per_launch_events": s2 * 1e6, "tflops": 2.0 * tokens * topk * model_dim * inter_dim / s2 / 1e12,
                    "weight_gb_per_s": experts * model_dim * inter_dim / s2 / 1e9})
        if tokens == 333:
            continue
        # the same two stages with int8 activations and packed int4 weights (W4A8): half the weight bytes
        x8, sx8 = quant.pertoken_quant(torch.randn(tokens, model_dim, generator=g), quant_dtype=torch.int8)
        a8, sa8 = quant.pertoken_quant(torch.randn(tokens * topk, inter_dim, generator=g), quant_dtype=torch.int8)
        w1p = layout.pack_shuffled_int8_to_int4(layout.shuffle_weight(torch.randint(-8, 8, (experts * 2 * inter_dim, model_dim), generator=g, dtype=torch.int8)))
        w2p = layout.pack_shuffled_int8_to_int4(layout.shuffle_weight(torch.randint(-8, 8, (experts * model_dim, inter_dim), generator=g, dtype=torch.int8)))
        x8, a8, sx8, sa8, w1p, w2p = [t.to(dev).contiguous().view(-1) for t in (x8, a8, sx8, sa8, w1p, w2p)]
        kw["in_dtype"] = "int4"
        f1 = compile_moe_gemm1(doweight_stage1=False, out_dtype="bf16", **kw)
        f2 = compile_moe_gemm2(doweight_stage2=True, out_dtype="bf16", accumulate=True, **kw)
        s1 = timed(lambda: f1(out1, x8, w1p, sx8, sw1, sid, se, swt, nv, tokens, inter_dim, model_dim, blocks, None))
        s2 = timed(lambda: f2(out2, a8, w2p, sa8, sw2, sid, se, swt, nv, tokens, model_dim, inter_dim, blocks, None))
        out.append({"workload": f"moe_w4a8_stage1_{tag}", "us_per_launch_events": s1 * 1e6, "tflops": 2.0 * tokens * topk * 2 * inter_dim * model_dim / s1 / 1e12,
                    "weight_gb_per_s": experts * 2 * inter_dim * model_dim / 2 / s1 / 1e9})
        out.append({"workload": f"moe_w4a8_stage2_atomic_{tag}", "us_per_launch_events": s2 * 1e6, "tflops": 2.0 * tokens * topk * model_dim * inter_dim / s2 / 1e12,
                    "weight_gb_per_s": experts * model_dim * inter_dim / 2 / s2 / 1e9})
    # the fused MX-FP4 stages (fp4 activations and weights, one e8m0 scale per 32 elements; stage 1 quantises its output again and writes
    # it by sorted position, stage 2 adds weight * row into the token's output row); blocks of at least 32 sorted rows
    from kernels.moe.mxfp_moe import flydsl_mxfp4_gemm1, flydsl_mxfp4_gemm2

    for tokens, model_dim, inter_dim, experts, topk, bm in ((4096, 4096, 1536, 32, 8, 128), (64, 4096, 1536, 32, 8, 32)) if want("moe_mxfp4") else ():
        g = torch.Generator().manual_seed(0)
        vals, ids = torch.topk(torch.rand(tokens, experts, generator=g), k=topk, dim=1)
        sid, swt, se, npp = moe_sorting(ids.int().to(dev), torch.softmax(vals, 1).to(dev), num_experts=experts, block_size=bm)
        rows = int(sid.numel())
        rb = lambda *shape: torch.randint(0, 256, shape, dtype=torch.uint8, generator=g).to(dev)  # noqa: E731
        sc = lambda n: torch.randint(120, 130, (n,), dtype=torch.uint8, generator=g).to(dev)  # noqa: E731
        a4, a4s = rb(tokens, model_dim // 2), sc((rows + 31) // 32 * 32 * (model_dim // 32))
        w1m, w1s = rb(experts * 2 * inter_dim, model_dim // 2), sc(experts * 2 * inter_dim * (model_dim // 32))
        w2m, w2s = rb(experts * model_dim, inter_dim // 2), sc(experts * model_dim * (inter_dim // 32))
        iq = torch.zeros(rows, inter_dim // 2, dtype=torch.uint8, device=dev)
        iqs = torch.zeros((rows + 255) // 256 * 256 * (inter_dim // 32), dtype=torch.uint8, device=dev)
        outm = torch.zeros(tokens, model_dim, dtype=torch.bfloat16, device=dev)
        nv = npp[:1].contiguous()
        kw = dict(sorted_expert_ids=se, cumsum_tensor=nv, BM=bm, NE=experts, D_HIDDEN=model_dim, D_INTER=inter_dim, topk=topk)
        s1 = timed(lambda: flydsl_mxfp4_gemm1(a_quant=a4, a_scale_sorted_shuffled=a4s, w1_u8=w1m, w1_scale_u8=w1s, m_indices=sid, inter_sorted_quant=iq,
                                              inter_sorted_shuffled_scale=iqs, n_tokens=tokens, **kw))
        s2 = timed(lambda: flydsl_mxfp4_gemm2(inter_sorted_quant=iq, inter_sorted_shuffled_scale=iqs, w2_u8=w2m, w2_scale_u8=w2s, sorted_token_ids=sid,
                                              sorted_weights=swt, flat_out=outm, M_logical=tokens, max_sorted=rows, epilog="atomic", **kw))
        tag = f"tokens{tokens}_e{experts}_top{topk}_model{model_dim}_inter{inter_dim}_block{bm}"
        out.append({"workload": f"moe_mxfp4_stage1_{tag}", "us_per_launch_events": s1 * 1e6, "tflops": 2.0 * tokens * topk * 2 * inter_dim * model_dim / s1 / 1e12,
                    "weight_gb_per_s": experts * 2 * inter_dim * model_dim / 2 / s1 / 1e9})
        out.append({"workload": f"moe_mxfp4_stage2_atomic_{tag}", "us_per_launch_events": s2 * 1e6, "tflops": 2.0 * tokens * topk * model_dim * inter_dim / s2 / 1e12,
                    "weight_gb_per_s": experts * model_dim * inter_dim / 2 / s2 / 1e9})
        # the launches in front of stage 1 when the activations arrive as bf16: the MX-FP4 quantiser and the scale sort
        from flydsl_amd import quant_device
        from kernels.moe.mxfp_moe import moe_mxfp4_sort

        hid = torch.randn(tokens, model_dim, generator=g).to(torch.bfloat16).to(dev)
        xq_buf = torch.empty(tokens, model_dim // 2, dtype=torch.uint8, device=dev)
        xs_buf = torch.empty((tokens + 31) // 32 * 32, model_dim // 32, dtype=torch.uint8, device=dev)
        xs_sorted = torch.empty((rows + 31) // 32 * 32, model_dim // 32, dtype=torch.uint8, device=dev)

        def front():
            quant_device.per_1x32_f4_quant(hid, shuffle=False, out=(xq_buf, xs_buf))
            moe_mxfp4_sort(xs_buf[:tokens], sid, nv, tokens, block_size=bm, out=xs_sorted)

        sf = timed(front, iters=50)
        out.append({"workload": f"moe_mxfp4_quant_and_scale_sort_tokens{tokens}_model{model_dim}_block{bm}", "us_per_launch_events": sf * 1e6, "tflops": 0.0,
                    "weight_gb_per_s": 0.0})
        if tokens <= 64:
            # the same stage 1 on blocks of 16 rows reading the bf16 rows itself (no launches in front of it)
            sid16, swt16, se16, npp16 = moe_sorting(ids.int().to(dev), torch.softmax(vals, 1).to(dev), num_experts=experts, block_size=16)
            rows16 = int(sid16.numel())
            iq16 = torch.zeros(rows16, inter_dim // 2, dtype=torch.uint8, device=dev)
            iqs16 = torch.zeros((rows16 + 255) // 256 * 256 * (inter_dim // 32), dtype=torch.uint8, device=dev)
            nv16 = npp16[:1].contiguous()
            s16 = timed(lambda: flydsl_mxfp4_gemm1(a_quant=a4, a_scale_sorted_shuffled=a4s, w1_u8=w1m, w1_scale_u8=w1s, m_indices=sid16, inter_sorted_quant=iq16,
                                                   inter_sorted_shuffled_scale=iqs16, n_tokens=tokens, inline_quant=True, hidden_states=hid,
                                                   sorted_expert_ids=se16, cumsum_tensor=nv16, BM=16, NE=experts, D_HIDDEN=model_dim, D_INTER=inter_dim, topk=topk))
            out.append({"workload": f"moe_mxfp4_stage1_inline_quant_tokens{tokens}_e{experts}_top{topk}_model{model_dim}_inter{inter_dim}_block16",
                        "us_per_launch_events": s16 * 1e6, "tflops": 2.0 * tokens * topk * 2 * inter_dim * model_dim / s16 / 1e12,
                        "weight_gb_per_s": experts * 2 * inter_dim * model_dim / 2 / s16 / 1e9})
    # the device-side expert sorter in front of the stages (outputs pre-allocated, accumulate buffer cleared by the same launch)
    for tokens, model_dim, experts, topk, tile_m in ((64, 4096, 32, 8, 16), (4096, 4096, 32, 8, 128), (4096, 4096, 256, 8, 32), (16384, 4096, 256, 8, 32)) if want("moe_sorting") else ():
        g = torch.Generator().manual_seed(0)
        vals, ids = torch.topk(torch.rand(tokens, experts, generator=g), k=topk, dim=1)
        d_ids, d_w = ids.int().to(dev), torch.softmax(vals, 1).to(dev)
        rows, blocks = sorted_sizes(tokens, topk, experts, tile_m)
        bufs = (torch.empty(rows, dtype=torch.int32, device=dev), torch.empty(rows, dtype=torch.float32, device=dev),
                torch.empty(blocks, dtype=torch.int32, device=dev), torch.empty(2, dtype=torch.int32, device=dev))
        acc = torch.empty(tokens, model_dim, dtype=torch.bfloat16, device=dev)
        ws = torch.empty(max(4, moe_sorting_get_workspace_size(tokens, experts, topk)), dtype=torch.uint8, device=dev)
        sec = timed(lambda: moe_sorting_flydsl(d_ids, d_w, *bufs, acc, experts, tile_m, None, None, ws), iters=50)
        out.append({"workload": f"moe_sorting_tokens{tokens}_e{experts}_top{topk}_block{tile_m}_clear{tokens}x{model_dim}bf16",
                    "us_per_launch_events": sec * 1e6, "tflops": 0.0, "weight_gb_per_s": 0.0})
    # the router gating in front of the sorter, alone and as one call with the sorter; 20 launches recorded into a HIP graph
    # (these kernels are shorter than the gap between two eager launches)
    from kernels.moe.moe_sorting_kernel import moe_softmax_sort_flydsl
    from kernels.moe.topk_gating_softmax_kernel import build_topk_gating_softmax_module

    def graph_timed(f, steps=20):
        for _ in range(3):
            f()
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            for _ in range(steps):
                f()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        best = float("inf")
        for _ in range(5):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(10):
                g.replay()
            e1.record()
            torch.cuda.synchronize()
            best = min(best, e0.elapsed_time(e1) / 1e3 / steps / 10)
        return best

    for tokens, experts, topk in ((16, 256, 8), (16, 128, 6), (1024, 128, 6), (16384, 256, 8)) if want("moe_gating") else ():
        g = torch.Generator().manual_seed(0)
        x = (torch.rand(tokens, experts, generator=g) * 4 - 2).to(torch.bfloat16).to(dev)
        w = torch.empty(tokens, topk, dtype=torch.float32, device=dev)
        idx = torch.empty(tokens, topk, dtype=torch.int32, device=dev)
        tei = torch.empty_like(idx)
        launch = build_topk_gating_softmax_module(num_experts=experts, topk=topk, dtype_str="bf16")
        sec = graph_timed(lambda: launch(x, w, idx, tei, tokens, stream=torch.cuda.current_stream()))
        out.append({"workload": f"moe_topk_gating_bf16_tokens{tokens}_e{experts}_top{topk}", "us_per_launch_events": sec * 1e6, "tflops": 0.0,
                    "weight_gb_per_s": (tokens * experts * 2 + tokens * topk * 12) / sec / 1e9})
        rows, blocks = sorted_sizes(tokens, topk, experts, 32)
        bufs = (torch.empty(rows, dtype=torch.int32, device=dev), torch.empty(rows, dtype=torch.float32, device=dev),
                torch.empty(blocks, dtype=torch.int32, device=dev), torch.empty(2, dtype=torch.int32, device=dev))
        acc = torch.empty(tokens, 4096, dtype=torch.bfloat16, device=dev)
        ws = torch.empty(max(4, moe_sorting_get_workspace_size(tokens, experts, topk)), dtype=torch.uint8, device=dev)
        sec = graph_timed(lambda: moe_softmax_sort_flydsl(x, *bufs, acc, experts, topk, "bf16", 32, None, True, None, topk_ids=idx, topk_weights=w,
                                                          workspace=ws, stream=torch.cuda.current_stream()))
        out.append({"workload": f"moe_softmax_sort_bf16_tokens{tokens}_e{experts}_top{topk}_block32_clear{tokens}x4096bf16", "us_per_launch_events": sec * 1e6,
                    "tflops": 0.0, "weight_gb_per_s": 0.0})
    return out


def run_reference_test_shapes():
    """The shapes of the reference's own tests for this path (tests/kernels/test_preshuffle_gemm.py:118-126 for the 8- and
    16-bit GEMM, :346-353 for MXFP4), through the automatic dispatcher (``--reference-shapes``).  Each shape is recorded
    20 times into a HIP graph over rotating operand sets; the graph is replayed until 50 ms are timed."""
    import torch

    from flydsl_amd.synthetic import make_a8w8, make_a16w16, make_mxfp4

    dev = torch.device("cuda:0")
    out = []

    graph_time = _graph_time

    def tile(t, rows, unit):  # rows of a host tensor repeated to `rows` (weights of the large shapes are built from a slab)
        return t.repeat((rows + unit - 1) // unit, *([1] * (t.dim() - 1)))[:rows].contiguous()

    shapes8 = [(16, 5120, 8192), (33, 1024, 2048), (5120, 5120, 8320), (5120, 2048, 8320), (9728, 8192, 8320), (5133, 5120, 8320)]
    for kind in ("fp8", "int8", "bf16"):
        for M, N, K in shapes8:
            mh, nh = min(M, 512), min(N, 512)
            family = "a16w16" if kind == "bf16" else "a8w8"
            host = make_a16w16(mh, nh, K, kind, seed=0, w_std=0.02) if kind == "bf16" else make_a8w8(mh, nh, K, kind, seed=0)
            nbytes = algorithmic_bytes(family, M, N, K)
            n_sets = max(2, min(16, math.ceil(2 * MALL_BYTES / nbytes)))
            sets = []
            for _ in range(n_sets):
                none = torch.empty(0, dtype=torch.float32, device=dev)
                s = {"a": tile(host["a_q"], M, mh).to(dev), "b": tile(host["b_shuf"].view(nh, -1), N, nh).to(dev),
                     "sa": none if kind == "bf16" else tile(host["sa"].view(-1), M, mh).to(dev),
                     "sb": none if kind == "bf16" else tile(host["sb"].view(-1), N, nh).to(dev),
                     "c": torch.zeros(M, N, dtype=torch.bfloat16, device=dev)}
                sets.append(s)
            sec = graph_time(make_launcher(family, kind, M, N, K), sets)
            out.append({"workload": f"{kind}_m{M}_n{N}_k{K}", "us_per_launch_events": sec * 1e6, "tflops": 2.0 * M * N * K / sec / 1e12,
                        "gb_per_s": nbytes / sec / 1e9, "operand_sets": n_sets})
            del sets
            torch.cuda.empty_cache()
    for M, N, K in [(64, 8192, 8192), (32, 8192, 8192), (128, 8192, 8192), (1024, 8192, 8192), (5133, 8192, 8192)]:
        mh, nh = min(M, 512), 512
        host = make_mxfp4(mh, nh, K, seed=0)
        nbytes = algorithmic_bytes("mxfp4", M, N, K)
        n_sets = max(2, min(16, math.ceil(2 * MALL_BYTES / nbytes)))
        sets = []
        for _ in range(n_sets):
            sets.append({"a": tile(host["a_q"], M, mh).to(dev), "b": tile(host["b_shuf"].view(nh, -1), N, nh).to(dev),
                         "sa": host["sa_shuf"].view(-1).repeat((M + mh - 1) // mh + 1).contiguous().to(dev),
                         "sb": host["sb_shuf"].view(-1).repeat(N // nh).contiguous().to(dev),
                         "c": torch.zeros(M, N, dtype=torch.bfloat16, device=dev)})
        sec = graph_time(make_launcher("mxfp4", "fp4", M, N, K), sets)
        out.append({"workload": f"mxfp4_m{M}_n{N}_k{K}", "us_per_launch_events": sec * 1e6, "tflops": 2.0 * M * N * K / sec / 1e12,
                    "gb_per_s": nbytes / sec / 1e9, "operand_sets": n_sets})
        del sets
        torch.cuda.empty_cache()
    return out


# the reference's own benchmark list for this path (scripts/run_benchmark.sh:120-142, GEMM_SHAPES): dtype, M, N, K
REFERENCE_BENCHMARK_SHAPES = [("fp8", 16, 40960, 5120), ("fp8", 16, 77824, 5120), ("fp8", 256, 2112, 7168), ("fp8", 512, 2112, 7168),
                              ("fp8", 5120, 5120, 8320), ("fp8", 9728, 8192, 8320), ("fp8", 8192, 8192, 8192),
                              ("int8", 9728, 8192, 8320), ("bf16", 5120, 5120, 8320)]


def run_reference_benchmark_shapes():
    """The nine shapes the reference benchmarks this path on (its results are not recorded anywhere), through the automatic
    dispatcher, each with the roofline that bounds it: HBM when the algorithmic flops per byte lie below peak flops / peak
    bytes, MFMA otherwise.  Same timing as the main workloads: 20 launches per HIP graph over rotating operand sets (more
    than twice the Infinity Cache per pass), replayed until 50 ms are timed."""
    import torch

    from flydsl_amd.synthetic import make_a8w8, make_a16w16

    dev = torch.device("cuda:0")
    out = []

    def tile(t, rows, unit):
        return t.repeat((rows + unit - 1) // unit, *([1] * (t.dim() - 1)))[:rows].contiguous()

    for kind, M, N, K in REFERENCE_BENCHMARK_SHAPES:
        family = "a16w16" if kind == "bf16" else "a8w8"
        mh, nh = min(M, 512), min(N, 512)
        host = make_a16w16(mh, nh, K, kind, seed=0, w_std=0.02) if kind == "bf16" else make_a8w8(mh, nh, K, kind, seed=0)
        nbytes = algorithmic_bytes(family, M, N, K)
        flops = 2.0 * M * N * K
        n_sets = max(2, min(16, math.ceil(2 * MALL_BYTES / nbytes)))
        none = torch.empty(0, dtype=torch.float32, device=dev)
        sets = [{"a": tile(host["a_q"], M, mh).to(dev), "b": tile(host["b_shuf"].view(nh, -1), N, nh).to(dev),
                 "sa": none if kind == "bf16" else tile(host["sa"].view(-1), M, mh).to(dev),
                 "sb": none if kind == "bf16" else tile(host["sb"].view(-1), N, nh).to(dev),
                 "c": torch.zeros(M, N, dtype=torch.bfloat16, device=dev)} for _ in range(n_sets)]
        sec = _graph_time(make_launcher(family, kind, M, N, K), sets)
        bound = "hbm" if flops / nbytes < PEAK[kind] * 1e12 / (PEAK["hbm"] * 1e9) else "mfma"
        achieved = nbytes / sec / 1e9 if bound == "hbm" else flops / sec / 1e12
        peak = PEAK["hbm"] if bound == "hbm" else PEAK[kind]
        out.append({"workload": f"{kind}_m{M}_n{N}_k{K}", "us_per_launch_events": sec * 1e6, "tflops": flops / sec / 1e12,
                    "gb_per_s": nbytes / sec / 1e9, "operand_sets": n_sets,
                    "roofline": {"bound": bound, "achieved": achieved, "peak": peak, "unit": "GB/s" if bound == "hbm" else "TFLOP/s",
                                 "frac": achieved / peak, "algorithmic_bytes": nbytes, "flops": flops}})
        del sets
        torch.cuda.empty_cache()
    return out


def _graph_time(launch, sets, steps=20):
    """Seconds per launch: `steps` launches recorded into one HIP graph over rotating operand sets, replayed until
    MIN_TIMED_S of work is timed with events on the launch stream."""
    import torch

    for i in range(3):
        launch(sets[i % len(sets)])
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        for i in range(steps):
            launch(sets[i % len(sets)])
    torch.cuda.synchronize()
    g.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    g.replay()
    e1.record()
    torch.cuda.synchronize()
    replays = max(1, math.ceil(MIN_TIMED_S / max(e0.elapsed_time(e1) * 1e-3, 1e-7)))
    best = float("inf")
    for _ in range(2):
        e0.record()
        for _r in range(replays):
            g.replay()
        e1.record()
        torch.cuda.synchronize()
        best = min(best, e0.elapsed_time(e1) * 1e-3 / (steps * replays))
    return best


def host_cost_per_call(name="fp8_decode_m16", calls=2000):
    """Host time of one eager launch (no graph): wall clock of a loop of `calls` launches on one stream divided by the
    calls, for the launcher's default path (operands validated once, then looked up) and for the path that validates every
    call.  The GPU work of the loop is far shorter than the loop, so this is the cost of getting a launch into the queue."""
    import torch

    from flydsl_amd.synthetic import make_a8w8
    from kernels.gemm.preshuffle_gemm import compile_preshuffle_gemm

    family, kind, M, N, K, _ = WORKLOADS[name]
    dev = torch.device("cuda:0")
    host = make_a8w8(M, N, K, kind, seed=0)
    a, b, sa, sb = host["a_q"].to(dev), host["b_shuf"].to(dev), host["sa"].to(dev), host["sb"].to(dev)
    c = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
    bias = torch.empty(0, dtype=torch.bfloat16, device=dev)
    fn = compile_preshuffle_gemm(N=N, K=K, tile_m=128, tile_n=256, tile_k=64, in_dtype=kind)
    stream = torch.cuda.current_stream()
    out = {}
    for label, call in (("fast_path", fn), ("checked_path", fn.launch_checked)):
        for _ in range(50):
            call(c, a, b, sa, sb, bias, M, N, stream)
        torch.cuda.synchronize()
        best = float("inf")
        for _ in range(3):
            t0 = time.perf_counter()
            for _i in range(calls):
                call(c, a, b, sa, sb, bias, M, N, stream)
            dt = time.perf_counter() - t0
            torch.cuda.synchronize()
            best = min(best, dt / calls)
        out[label] = best * 1e6
    # what both paths share: the C ABI call itself (ctypes + the library's checks + hipLaunchKernel) on a filled struct.
    # The struct is filled here for THESE tensors (the launcher's table may still hold entries of operands that earlier
    # workloads have freed since).
    cargs, handle = fn._prepare(c, a, b, sa, sb, bias, M, N, stream)
    ref = ctypes.byref(cargs)
    gemm = fn._gemm
    best = float("inf")
    for _ in range(3):
        t0 = time.perf_counter()
        for _i in range(calls):
            gemm(ref, handle)
        dt = time.perf_counter() - t0
        torch.cuda.synchronize()
        best = min(best, dt / calls)
    c_call = best * 1e6
    return {"workload": name, "calls": calls, "fast_path": out["fast_path"], "checked_path": out["checked_path"],
            "c_abi_call_alone": c_call, "launcher_overhead_fast": out["fast_path"] - c_call,
            "launcher_overhead_checked": out["checked_path"] - c_call,
            "unit": "us per call, host wall clock of an eager launch loop"}


def cpu_baseline(name, host, budget_s=12.0):  # budget_s bounds the CPU work of one workload
    """The reference's torch CPU path (dequantise to fp32 + torch.mm) on the same seeded operands,
    timed on this box's host cores.  For workloads whose single pass exceeds the budget a row sample of
    A is used (the weight side, which dominates the dequantisation cost, is always whole)."""
    import torch

    from oracle import psg_oracle as O

    family, kind, M, N, K, _ = WORKLOADS[name]
    cores = torch.get_num_threads()
    # bound the work: ~2*m*N*K flop at a conservative 50 GFLOP/s per 8 cores
    est = 2.0 * M * N * K / (6e9 * cores) + N * K / 2e8
    m_s = M if est <= budget_s else max(16, int(M * budget_s / est))
    if family == "a16w16":
        a, b = host["a_q"][:m_s], host["b_q"]
        f = lambda: torch.mm(a.to(torch.float32), b.to(torch.float32).T)  # noqa: E731  (run_torch without scales)
    elif family == "a8w8":
        a, b, sa, sb = host["a_q"][:m_s], host["b_q"], host["sa"][:m_s], host["sb"]
        f = lambda: O.run_torch_cpu(a, b, sa, sb)  # noqa: E731
    else:
        a, b, sa, sb = host["a_q"][:m_s], host["b_q"], host["sa"], host["sb"]
        f = lambda: O.run_torch_w4_cpu(a, b, sa, sb)  # noqa: E731
    t0 = time.perf_counter()
    f()
    first = time.perf_counter() - t0
    iters = max(1, min(10, int(budget_s / 2 / max(first, 1e-6))))
    times = []
    for _ in range(iters):
        t0 = time.perf_counter()
        f()
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    return {
        "value": 2.0 * m_s * N * K / med / 1e12, "unit": "TFLOP/s", "cores": cores, "kind": "port",
        "sample": f"run_torch (fp32 dequant + torch.mm) on rows [0,{m_s}) of A x all {N} weight rows, K={K}; "
                  f"median of {iters} runs, {med * 1e3:.1f} ms each",
    }


def load_traffic(name):
    """HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (scaled by a copy
    kernel of known size); kept as a small committed summary next to the profiles."""
    path = os.path.join(ROOT, "profiles", "pmc_traffic.json")
    try:
        with open(path) as f:
            return json.load(f).get(name, {}).get("traffic_bytes")
    except Exception:
        return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None)
    ap.add_argument("--warmup", type=int, default=None)
    ap.add_argument("--workload", default=DEFAULT_WORKLOAD, choices=sorted(WORKLOADS))
    ap.add_argument("--no-others", action="store_true", help="skip the per-config table of the other workloads")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--reference-shapes", action="store_true",
                    help="also time the shapes of the reference's tests for this path (reference_test_shapes), and its benchmark "
                         "list (scripts/run_benchmark.sh: reference_benchmark_shapes) where --no-others would leave that out")
    ap.add_argument("--next-rows", action="store_true",
                    help="also time the general MX kernel and the MoE stages (rows next to the hot path); adds a next_rows list")
    ap.add_argument("--next-rows-only", default=None, choices=("mx", "moe_fp8", "moe_mxfp4", "moe_sorting", "moe_gating"),
                    help="with --next-rows: run one section of them only (for profiler runs)")
    ap.add_argument("--quant-only", default=None, choices=("quant_pertoken_fp8_m8192", "quant_mxfp4_m4096"),
                    help="only run one of the on-device quantiser workloads (for profiler runs)")
    ap.add_argument("--host-cost", action="store_true", help="measure host_us_per_call even with --no-others")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="only run a plain 1 GiB device-to-device copy a few times (the known-size kernel that the "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE counters are scaled against)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build measures one GPU only (got --gpus {args.gpus}); "
              "the GEMM would shard over N (disjoint column panels of C, no exchange between GPUs)", file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the preshuffle GEMM has no CPU path", file=sys.stderr)
        sys.exit(3)
    from flydsl_amd import _lib

    _lib.lib()  # fail loudly if the HIP library is missing

    if args.calibrate_copy:
        src = torch.ones(1 << 30, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"calibrate_copy_bytes": 1 << 30, "launches": 5}))
        return

    if args.quant_only:
        print(json.dumps(run_quant_workload(args.quant_only)))
        return

    family, kind, M, N, K, bound = WORKLOADS[args.workload]
    small = bound == "hbm"
    steps = args.steps if args.steps is not None else (500 if small else 20)
    warmup = args.warmup if args.warmup is not None else (50 if small else 3)

    main_res, host = run_workload(args.workload, steps, warmup)
    main_res["roofline"]["traffic"] = load_traffic(args.workload)
    cpu = None if args.no_cpu else cpu_baseline(args.workload, host)
    del host

    others = []
    if not args.no_others:
        for name in ("fp8_decode_m1", "fp8_decode_m16", "fp8_decode_m32", "fp8_prefill_m8192", "int8_ffn_m4096", "mxfp4_m32",
                     "mxfp4_m4096", "bf16_m5120"):
            if name == args.workload:
                continue
            b = WORKLOADS[name][5]
            r, h = run_workload(name, 300 if b == "hbm" else (5 if name == "int8_ffn_m4096" else 20), 20 if b == "hbm" else 2)
            r["roofline"]["traffic"] = load_traffic(name)
            # the reference's CPU path beside every configuration (a bounded row sample, a few seconds each)
            r["cpu_baseline"] = None if args.no_cpu else cpu_baseline(name, h, budget_s=3.0)
            del h
            others.append(r)
        for name in ("quant_pertoken_fp8_m8192", "quant_mxfp4_m4096"):
            others.append(run_quant_workload(name))
    next_rows = run_next_row_workloads(args.next_rows_only) if args.next_rows else None
    ref_shapes = run_reference_test_shapes() if args.reference_shapes else None
    # the reference's own benchmark list rides along with the full line (nine shapes, a few seconds)
    ref_bench = run_reference_benchmark_shapes() if args.reference_shapes or not args.no_others else None
    host_cost = host_cost_per_call() if not args.no_others or args.host_cost else None

    line = {
        "metric": "TFLOPS + % roofline (HBM GB/s at M=16, MFMA util at M=8192), 1 MI355X",
        # whole-job throughput in the unit of the roofline that bounds the workload: bytes for the decode shapes
        # (algorithmic bytes per launch / time per step), flops for the prefill shapes
        "value": main_res["gb_per_s"] if bound == "hbm" else main_res["tflops"],
        "unit": "GB/s" if bound == "hbm" else "TFLOP/s",
        "tflops": main_res["tflops"],
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": main_res["us_per_step_wall"] / 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": {"fp8": "fp8_e4m3fn", "int8": "int8", "fp4": "mxfp4_e2m1", "bf16": "bf16", "fp16": "fp16"}[kind],
        "data": "synthetic (seed 0; A~N(0,1) per-token quantised, W~N(0,0.02) per-channel quantised and preshuffled; "
                f"{main_res['operand_sets']} rotating operand sets)",
        "config": {"workload": f"{args.workload}: {kind} W8A8 preshuffle GEMM M={M} N={N} K={K}, bf16 out", "M": M, "N": N, "K": K,
                   "timing": f"K steps recorded into one HIP graph, replayed {main_res['graph_replays_per_timing']}x per timing "
                             "(>= 50 ms of work); wall clock between synchronizes"},
        "gb_per_s": main_res["gb_per_s"],
        "parity_ok": main_res["parity_ok"],
        "us_per_launch_events": main_res["us_per_launch_events"],
        "us_per_launch_hot_cache": main_res["us_per_launch_hot_cache"],
        "roofline": main_res["roofline"],
        "cpu_baseline": cpu,
        "per_config": others,
    }
    if next_rows is not None:
        line["next_rows"] = next_rows
    if ref_shapes is not None:
        line["reference_test_shapes"] = ref_shapes
    if ref_bench is not None:
        line["reference_benchmark_shapes"] = ref_bench
    if host_cost is not None:
        line["host_us_per_call"] = host_cost
    # the metric names two operating points; the second one (MFMA-bound prefill) is lifted out of the table for convenience
    for r in others:
        if r["workload"] == "fp8_prefill_m8192":
            line["prefill_m8192"] = {"tflops": r["tflops"], "us_per_launch_events": r["us_per_launch_events"], "roofline": r["roofline"],
                                     "cpu_baseline": r.get("cpu_baseline")}
    print(json.dumps(line))


if __name__ == "__main__":
    main()
