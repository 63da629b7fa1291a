"""Row-scale fp8 GEMM entry points with the call shapes of the reference's ``compile_fp8_gemm_8w``
(kernels/gemm/fp8_gemm_8wave.py:148) and ``compile_fp8_gemm_4w`` (kernels/gemm/fp8_gemm_4wave.py:162):

    launch = compile_fp8_gemm_8w(K=K, BLOCK_M=256, BLOCK_N=256, b_preshuffled=False)
    launch(A, B_T, C, A_scale, B_scale, c_m, c_n, stream)

``A`` is ``[c_m, K]`` e4m3fn (passed flattened, viewed as int8), ``B_T`` is the weight ``[c_n, K]`` either plain row-major
or in the preshuffled fragment layout (``preshuffle_b``, kernels/gemm/fp8_gemm_utils.py:24-28, the same byte map as
``shuffle_weight``), ``C`` is bf16 ``[c_m, c_n]``, the scales are fp32 per row of A and per row of B_T.  ``c_m`` and
``c_n`` are run-time arguments; only ``K`` is fixed when the launcher is built.

Both names run the same native kernels as ``compile_preshuffle_gemm`` (``psg_gemm_a8w8``); ``BLOCK_M`` / ``BLOCK_N`` /
``use_xcd_remap`` are checked with the reference's own assertions and then treated as hints.  The reference's epilogue
multiplies ``acc * (scale_a * scale_b)`` (fp8_gemm_utils.py:149-198); this library keeps ``(acc * scale_a) * scale_b``,
which differs by at most one fp32 ulp before the bf16 rounding.
"""

from __future__ import annotations

import ctypes

from ... import _lib


class RowScaleFp8Gemm:
    """Launcher returned by :func:`compile_fp8_gemm_8w` / :func:`compile_fp8_gemm_4w`.  Holds no tensor references."""

    def __init__(self, K: int, b_preshuffled: bool):
        self.K = int(K)
        self.b_preshuffled = bool(b_preshuffled)
        self._lib = _lib.lib()

    def __call__(self, A, B_T, C, A_scale, B_scale, c_m, c_n, stream=None):
        M, N, K = int(c_m), int(c_n), self.K
        if M < 1 or M > 65536:
            raise ValueError(f"c_m={M} outside [1, 65536]")
        if N < 16 or N % 16:
            raise ValueError(f"c_n={N} must be a positive multiple of 16")
        dev = _lib.check_operand("C", C, min_elems=M * N, elem_sizes=(2,))
        _lib.check_operand("A", A, min_elems=M * K, elem_sizes=(1,), device=dev)
        _lib.check_operand("B_T", B_T, min_elems=N * K, elem_sizes=(1,), device=dev)
        _lib.check_operand("A_scale", A_scale, min_elems=M, elem_sizes=(4,), device=dev)
        _lib.check_operand("B_scale", B_scale, min_elems=N, elem_sizes=(4,), device=dev)
        args = _lib.A8W8Args()
        args.c, args.a, args.b = C.data_ptr(), A.data_ptr(), B_T.data_ptr()
        args.scale_a, args.scale_b = A_scale.data_ptr(), B_scale.data_ptr()
        args.M, args.N, args.K = M, N, K
        args.in_dtype = _lib.IN_DTYPE["fp8"]
        args.out_dtype = _lib.OUT_DTYPE["bf16"]
        args.b_layout = 0 if self.b_preshuffled else 1
        h = _lib.stream_handle(stream)
        need = self._lib.psg_workspace_bytes(M, N, K, args.in_dtype)
        if need:
            ws = _lib.workspace(dev, need, h, owner=id(self))
            args.workspace, args.workspace_bytes = ws.data_ptr(), ws.numel()
        rc = self._lib.psg_gemm_a8w8(ctypes.byref(args), h)
        if rc:
            _lib.check(rc, "psg_gemm_a8w8")


def compile_fp8_gemm_8w(*, K: int, BLOCK_M: int = 256, BLOCK_N: int = 256, b_preshuffled: bool = False):
    """kernels/gemm/fp8_gemm_8wave.py:148-153: same keyword-only signature, defaults and assertions."""
    BLOCK_K = 128
    assert BLOCK_M >= 128 and BLOCK_N >= 256 and BLOCK_M % 128 == 0 and BLOCK_N % 256 == 0
    assert K % BLOCK_K == 0
    return RowScaleFp8Gemm(K, b_preshuffled)


def compile_fp8_gemm_4w(*, K: int, BLOCK_M: int = 256, BLOCK_N: int = 256, use_xcd_remap: bool = True,
                        b_preshuffled: bool = False):
    """kernels/gemm/fp8_gemm_4wave.py:162-176: same keyword-only signature, defaults and assertions."""
    BLOCK_K = 128
    assert BLOCK_M >= 64 and BLOCK_M % 64 == 0 and BLOCK_N >= 64 and BLOCK_N % 64 == 0
    assert K % BLOCK_K == 0
    return RowScaleFp8Gemm(K, b_preshuffled)
