"""GPU parity of the compile_fp4_gemm_4w call shape (kernels/gemm/fp4_gemm_4wave.py:634) against the CPU oracle.
Mirrors tests/kernels/test_fp4_gemm_4wave.py:57-118 at sizes the oracle finishes in seconds (the reference runs
8192^3 and 16384^3); same operand construction, argument order and flattened views."""

import numpy as np
import pytest
import torch

from helpers import make_mxfp4
from oracle import psg_oracle as O

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("M,N,K", [(256, 512, 1024), (512, 256, 2048), (1024, 1024, 1024), (256, 256, 512)])
@pytest.mark.parametrize("bake_mn", [True, False])
def test_fp4_gemm_4wave(M, N, K, bake_mn):
    from kernels.gemm.fp4_gemm_4wave import compile_fp4_gemm_4w

    d = make_mxfp4(M, N, K, seed=3, w_std=1.0)
    ref = O.run_torch_w4(d["a_q"].numpy(), d["b_q"].numpy(), d["sa"].numpy(), d["sb"].numpy())
    dev = torch.device("cuda")
    launch = compile_fp4_gemm_4w(K=K, MN=(M, N)) if bake_mn else compile_fp4_gemm_4w(K=K, use_xcd_remap=False)
    c = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
    flat = lambda t: t.to(dev).contiguous().view(-1)  # noqa: E731
    launch(flat(d["a_q"]), flat(d["b_shuf"]), c.view(-1), flat(d["sa_shuf"]), flat(d["sb_shuf"]), M, N, torch.cuda.current_stream())
    torch.cuda.synchronize()
    out = c.float().cpu().numpy()
    ok, ratio = O.within_north_star_tolerance(out, ref, 1e-2)
    assert ok, f"outside tolerance (worst ratio {ratio:.3f})"
    assert O.verify_output(out, ref, rtol=0.1, atol=0.1)  # the reference's own bar


def test_shape_baked_in_must_match_the_call():
    from kernels.gemm.fp4_gemm_4wave import compile_fp4_gemm_4w

    launch = compile_fp4_gemm_4w(K=1024, MN=(256, 256))
    z = torch.zeros(1, device="cuda")
    with pytest.raises(ValueError, match="built for"):
        launch(z, z, z, z, z, 512, 256, None)
