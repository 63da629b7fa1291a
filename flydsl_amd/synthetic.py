"""Seeded synthetic operands for the preshuffle GEMM in the distributions the benchmark configs name
(activations N(0,1), weights N(0, w_std)), quantised and laid out by the package's host helpers.
Used by the benchmark and by the parity tests; everything is produced on the CPU so that the stream
of random numbers does not depend on the device."""

from __future__ import annotations

import torch

from . import layout, quant

FP8 = torch.float8_e4m3fn


def gen(seed):
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return g


def make_a8w8(M, N, K, kind, seed=0, w_std=0.02):
    """Returns dict with CPU tensors a_q [M,K], b_q [N,K] (un-shuffled), b_shuf, sa [M], sb [N]."""
    g = gen(seed)
    x = torch.randn(M, K, generator=g, dtype=torch.float32)
    w = torch.randn(N, K, generator=g, dtype=torch.float32) * w_std
    qd = torch.int8 if kind == "int8" else FP8
    a_q, sa = quant.pertoken_quant(x, quant_dtype=qd)
    b_q, sb = quant.pertoken_quant(w, quant_dtype=qd)
    b_shuf = layout.shuffle_weight(b_q.contiguous(), layout=(16, 16))
    return {
        "kind": kind,
        "a_q": a_q.contiguous(),
        "b_q": b_q.contiguous(),
        "b_shuf": b_shuf.contiguous(),
        "sa": sa.reshape(-1).contiguous(),
        "sb": sb.reshape(-1).contiguous(),
    }


def make_mxfp4(M, N, K, seed=0, w_std=0.02):
    """MXFP4 operands the way the reference's harness builds them
    (tests/kernels/test_preshuffle_gemm.py:386-414): rows padded to 32 before quantisation."""
    g = gen(seed)
    x = torch.randn(M, K, generator=g, dtype=torch.float32)
    w = torch.randn(N, K, generator=g, dtype=torch.float32) * w_std
    m32 = (M + 31) // 32 * 32
    n32 = (N + 31) // 32 * 32
    xp = torch.zeros(m32, K)
    xp[:M] = x
    wp = torch.zeros(n32, K)
    wp[:N] = w
    a_q, sa, _ = quant.per_1x32_f4_quant(xp)
    b_q, sb, _ = quant.per_1x32_f4_quant(wp)
    a_q = a_q.view(torch.uint8)[:M].contiguous()
    b_q = b_q.view(torch.uint8)[:N].contiguous()
    sa = sa.view(torch.uint8).contiguous()
    sb = sb.view(torch.uint8).contiguous()
    return {
        "a_q": a_q,
        "b_q": b_q,
        "sa": sa,
        "sb": sb,
        "b_shuf": layout.shuffle_weight_w4(b_q, 16, False, False).contiguous(),
        "sa_shuf": layout.shuffle_scale_w4(sa, 1, False).contiguous(),
        "sb_shuf": layout.shuffle_scale_w4(sb, 1, False).contiguous(),
    }


def make_mx(M, N, K, a_dtype="fp4", b_dtype="fp4", seed=0, w_std=0.02):
    """MX operands in any supported format pair, built like the reference's harnesses
    (tests/kernels/test_preshuffle_gemm.py:386-414 fp4, :507-527 fp6 x fp4, :630-647 fp8 x fp8): rows padded to 32
    before quantisation, W and both scale arrays shuffled.  ``a_q`` / ``b_q`` are uint8 in the layout the GEMM reads
    (fp4 packed nibbles, fp6 24+8-byte groups, fp8 bytes)."""
    g = gen(seed)
    x = torch.randn(M, K, generator=g, dtype=torch.float32)
    w = torch.randn(N, K, generator=g, dtype=torch.float32) * w_std
    xp = torch.zeros((M + 31) // 32 * 32, K)
    xp[:M] = x
    wp = torch.zeros((N + 31) // 32 * 32, K)
    wp[:N] = w

    def q(t, fmt):
        if fmt == "fp4":
            v, s, _ = quant.per_1x32_f4_quant(t)
        elif fmt == "fp6":
            v, s, _ = quant.per_1x32_f6_quant(t)
        elif fmt == "fp8":
            v, s = quant.per_1x32_f8_quant(t)
        else:
            raise ValueError(fmt)
        return v.view(torch.uint8).contiguous(), s.view(torch.uint8).contiguous()

    a_q, sa = q(xp, a_dtype)
    b_q, sb = q(wp, b_dtype)
    a_q, b_q = a_q[:M].contiguous(), b_q[:N].contiguous()
    return {
        "a_dtype": a_dtype,
        "b_dtype": b_dtype,
        "a_q": a_q,
        "b_q": b_q,
        "sa": sa,
        "sb": sb,
        "b_shuf": layout.shuffle_weight_w4(b_q, 16, False, False).contiguous(),
        "sa_shuf": layout.shuffle_scale_w4(sa, 1, False).contiguous(),
        "sb_shuf": layout.shuffle_scale_w4(sb, 1, False).contiguous(),
    }


def make_a16w16(M, N, K, kind, seed=0, w_std=1.0):
    """fp16 / bf16 operands (no quantisation, no scales), W preshuffled with the 2-byte layout."""
    g = gen(seed)
    dt = torch.float16 if kind == "fp16" else torch.bfloat16
    a = torch.randn(M, K, generator=g, dtype=torch.float32).to(dt)
    w = (torch.randn(N, K, generator=g, dtype=torch.float32) * w_std).to(dt)
    return {"kind": kind, "a_q": a.contiguous(), "b_q": w.contiguous(), "b_shuf": layout.shuffle_weight(w.contiguous(), layout=(16, 16)).contiguous()}
