#!/usr/bin/env python3
"""Writes the golden fixtures next to this script.

The reference keeps no recorded vectors for the preshuffle GEMM, and none of its Python is imported
here: the vectors come from THIS repository's oracle (``oracle/psg_oracle.py``) after its functions
have been pinned by tests/test_oracle_*.py.  They freeze the oracle's behaviour so that a later edit
of the oracle (or of the package's host helpers) that changes a single byte is caught, and they give
the GPU tests fixed known-answer cases.

    python tests/golden/gen_golden.py          # rewrites tests/golden/*.npz
"""

import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import psg_oracle as O  # noqa: E402


def a8w8_case(kind, m, n, k, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((m, k)).astype(np.float32)
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    aq, sa = O.pertoken_quant(x, kind)
    bq, sb = O.pertoken_quant(w, kind)
    out = {
        "x": x.astype(np.float16).astype(np.float32), "w": w.astype(np.float16).astype(np.float32),
    }
    # inputs are stored rounded to fp16 to halve the fixture; everything is recomputed from the stored values
    aq, sa = O.pertoken_quant(out["x"], kind)
    bq, sb = O.pertoken_quant(out["w"], kind)
    out.update(a_q=aq.view(np.uint8), b_q=bq.view(np.uint8), sa=sa, sb=sb, b_shuf=O.shuffle_weight(bq.view(np.uint8)),
               c_ref=O.run_torch(aq, bq, sa, sb, kind))
    if kind == "int8":
        acc = O.int32_accumulators(aq, bq)
        out["acc"] = acc
        out["c_bf16_bits"] = O.f32_to_bf16_bits(O.epilogue_a8w8(acc, sa, sb))
    out["x"] = out["x"].astype(np.float16)
    out["w"] = out["w"].astype(np.float16)
    return out


def mx_case(m, n, k, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((m, k)).astype(np.float16).astype(np.float32)
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float16).astype(np.float32)
    m32 = (m + 31) // 32 * 32
    xp = np.zeros((m32, k), np.float32)
    xp[:m] = x
    ap, sa = O.per_1x32_f4_quant(xp)
    bp, sb = O.per_1x32_f4_quant(w)
    return dict(x=x.astype(np.float16), w=w.astype(np.float16), a_q=ap[:m], b_q=bp, sa=sa, sb=sb, b_shuf=O.shuffle_weight_w4(bp),
                sa_shuf=O.shuffle_scale_w4(sa), sb_shuf=O.shuffle_scale_w4(sb), c_ref=O.run_torch_w4(ap[:m], bp, sa, sb))


def main():
    np.savez_compressed(os.path.join(HERE, "a8w8_int8_m20_n48_k192.npz"), **a8w8_case("int8", 20, 48, 192, 0))
    np.savez_compressed(os.path.join(HERE, "a8w8_fp8_m33_n64_k128.npz"), **a8w8_case("fp8", 33, 64, 128, 1))
    np.savez_compressed(os.path.join(HERE, "mxfp4_m40_n64_k512.npz"), **mx_case(40, 64, 512, 2))


if __name__ == "__main__":
    main()
