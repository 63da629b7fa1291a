"""On-device activation quantisers (HIP kernels behind the C ABI): the same bytes as the host helpers in
``flydsl_amd.quant`` (and therefore as the reference's ``pertoken_quant`` tests/utils.py:29-73 and
``per_1x32_f4_quant`` + ``shuffle_scale_w4`` tests/kernels/utils/gemm_common_utils.py:675-704, 645-672), produced
without leaving the GPU.  torch is used for the output allocations only."""

from __future__ import annotations

import torch

from . import _lib
from .quant import fp4x2, fp8_e8m0

_X_DTYPE = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}


def _x_code(x):
    if x.dtype not in _X_DTYPE:
        raise TypeError(f"input dtype {x.dtype} is not supported (fp32 / bf16 / fp16)")
    if not x.is_cuda or x.dim() != 2 or not x.is_contiguous():
        raise ValueError("x must be a contiguous 2-D device tensor")
    return _X_DTYPE[x.dtype]


def _check_out(x, *outs):
    for t in outs:
        if not t.is_cuda or t.device != x.device or not t.is_contiguous():
            raise ValueError("out tensors must be contiguous and on the same device as x")


def pertoken_quant(x: torch.Tensor, quant_dtype=torch.int8, stream=None, out=None):
    """Per-row symmetric quantisation on the device.  Returns ``(y [M,K] quant_dtype, scale [M,1] fp32)``.
    ``out=(y, scale)`` reuses caller-owned outputs (1-byte ``[M,K]`` and fp32 ``[M]`` / ``[M,1]``): no allocation, so the
    call can be recorded into a HIP graph."""
    code = _x_code(x)
    if quant_dtype == torch.int8:
        out_code = 0
    elif quant_dtype == torch.float8_e4m3fn:
        out_code = 1
    else:
        raise ValueError(f"quant_dtype must be torch.int8 or torch.float8_e4m3fn, got {quant_dtype}")
    m, k = x.shape
    if out is None:
        y = torch.empty((m, k), dtype=torch.uint8, device=x.device)
        scale = torch.empty((m, 1), dtype=torch.float32, device=x.device)
    else:
        y, scale = out
        _check_out(x, y, scale)
        if y.numel() != m * k or y.element_size() != 1 or scale.numel() != m or scale.dtype != torch.float32:
            raise ValueError("out must be (1-byte [M,K], fp32 [M]) tensors")
        y = y.view(torch.uint8)
    rc = _lib.lib().psg_quant_pertoken(x.data_ptr(), code, y.data_ptr(), scale.data_ptr(), m, k, out_code, _lib.stream_handle(stream))
    if rc:
        _lib.check(rc, "psg_quant_pertoken")
    return y.view(quant_dtype), scale.view(m, 1)


def per_1x32_f4_quant(x: torch.Tensor, shuffle: bool = True, stream=None, out=None):
    """OCP-MX fp4 quantisation on the device.  Returns ``(packed [M,K/2], scales)`` where ``scales`` are e8m0 bytes over
    ``ceil(M/32)*32`` rows x ``K/32``: in the GEMM's shuffled layout when ``shuffle`` (default), row-major otherwise.
    Finite inputs only: a NaN / Inf in a block does not give the reference's 0xFF scale byte (the block maximum drops
    NaN)."""
    code = _x_code(x)
    m, k = x.shape
    r = (m + 31) // 32 * 32
    if out is None:
        packed = torch.empty((m, k // 2), dtype=torch.uint8, device=x.device)
        scales = torch.empty((r, k // 32), dtype=torch.uint8, device=x.device)
    else:  # caller-owned outputs: no allocation, graph-capturable
        _check_out(x, *out)
        packed, scales = (t.view(torch.uint8) for t in out)
        if packed.numel() != m * (k // 2) or scales.numel() != r * (k // 32):
            raise ValueError("out must be (packed [M,K/2], scales [ceil(M/32)*32, K/32]) byte tensors")
    rc = _lib.lib().psg_quant_mxfp4(x.data_ptr(), code, packed.data_ptr(), scales.data_ptr(), m, k, 1 if shuffle else 0,
                                    _lib.stream_handle(stream))
    if rc:
        _lib.check(rc, "psg_quant_mxfp4")
    return packed.view(fp4x2), scales.view(fp8_e8m0)
