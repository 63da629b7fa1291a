"""MXFP4 GEMM entry point with the call shape of the reference's ``compile_fp4_gemm_4w``
(kernels/gemm/fp4_gemm_4wave.py:634-639):

    launch = compile_fp4_gemm_4w(K=K, MN=(M, N))
    launch(A, B_T, C, A_scale, B_scale, c_m, c_n, stream)

``A`` is ``[c_m, K/2]`` packed e2m1 (two codes per byte, even k in the low nibble), ``B_T`` the weight ``[c_n, K/2]`` in
the ``shuffle_weight_w4`` layout, both scale arrays e8m0 in the ``shuffle_scale_w4`` layout, ``C`` bf16 ``[c_m, c_n]``
(tests/kernels/test_fp4_gemm_4wave.py:57-107).  These are the wire formats of ``launch_gemm`` in
``mxfp4_preshuffle.py``, so the call runs on the same native kernels (``psg_gemm_mxfp4``).  The reference's kernel is
fixed to a 256x256 block with an all-in-bounds epilogue and so needs ``c_m`` and ``c_n`` to be multiples of 256; this
library keeps its own bounds (``c_n % 32 == 0``, any ``c_m``) and takes the multiples of 256 as the common case.
"""

from __future__ import annotations

from .mxfp4_preshuffle import launch_gemm


class Fp4Gemm4Wave:
    """Launcher returned by :func:`compile_fp4_gemm_4w`.  Holds no tensor references."""

    def __init__(self, K: int, use_xcd_remap: bool, MN):
        self.K = int(K)
        self.use_xcd_remap = bool(use_xcd_remap)
        self.MN = None if MN is None else (int(MN[0]), int(MN[1]))

    def __call__(self, A, B_T, C, A_scale, B_scale, c_m, c_n, stream=None):
        M, N = int(c_m), int(c_n)
        if self.MN is not None and (M, N) != self.MN:
            raise ValueError(f"launcher was built for MN={self.MN}, called with c_m={M}, c_n={N}")
        if N < 32 or N % 32:
            raise ValueError(f"c_n={N} must be a positive multiple of 32")
        # xcd_swizzle = 0 is the library's default tile order; results do not depend on it
        launch_gemm(C, A, B_T, A_scale, B_scale, M, N, stream, N, self.K, 256, 256, 256, "fp4", "bf16", "fp4", 1, -1, -1, -1, -1, -1, -1, 0, 0)


def compile_fp4_gemm_4w(*, K: int, use_xcd_remap: bool = True, MN: tuple = None):
    """kernels/gemm/fp4_gemm_4wave.py:634-655: same keyword-only signature, defaults and assertions (K a multiple of
    the 256-element K block, and a K-step count the reference's partly unrolled loop can cover: ``(K/256 - 4)`` a
    multiple of 4 or 2)."""
    BLOCK_K = 256
    assert K % BLOCK_K == 0
    K_ITERS = K // BLOCK_K
    UNROLL = 4 if (K_ITERS - 4) % 4 == 0 else 2
    assert (K_ITERS - 4) % UNROLL == 0, K_ITERS
    return Fp4Gemm4Wave(K, use_xcd_remap, MN)
