"""Host-side quantisers that feed the preshuffle GEMM (torch, any device).

Same results as the reference's host utilities (``pertoken_quant`` tests/utils.py:29-73;
``per_1x32_f4_quant`` and its codecs tests/kernels/utils/gemm_common_utils.py:14-71,142-275,675-704;
``per_1x32_f6_quant`` / ``per_1x32_f8_quant`` / ``pack_fp6_e2m3`` / ``fp6_e2m3_to_f32`` :708-790),
written independently: the e2m1 rounding is a chain of threshold tests and the e2m3 rounding a per-binade
round-half-even instead of fp32 bit tricks.
"""

from __future__ import annotations

import torch

fp8_e8m0 = getattr(torch, "float8_e8m0fnu", torch.uint8)
fp4x2 = getattr(torch, "float4_e2m1fn_x2", torch.uint8)


def get_dtype_max(dtype) -> float:
    return float(torch.finfo(dtype).max) if dtype.is_floating_point else float(torch.iinfo(dtype).max)


def pertoken_quant(x, scale=None, x_scale=None, scale_dtype=torch.float32, quant_dtype=torch.int8, dtypeMax=None):
    """Symmetric per-row quantisation: ``scale = max|row| / dtypeMax`` (1 for an all-zero row),
    ``y = (x / scale).to(quant_dtype)`` -- truncation for int8, round-to-nearest-even for fp8.
    Non-finite inputs are clamped first (NaN -> 0, +-Inf -> +-dtypeMax).  Returns ``(y, scale [R,1])``."""
    h = x.to(torch.float32)
    if x_scale is not None:
        h = h * x_scale
    if dtypeMax is None:
        dtypeMax = get_dtype_max(quant_dtype)
    h = torch.nan_to_num(h, nan=0.0, posinf=float(dtypeMax), neginf=-float(dtypeMax))
    if scale is None:
        hi = torch.amax(h, dim=-1, keepdim=True)
        lo = torch.amin(h, dim=-1, keepdim=True)
        scale = torch.maximum(hi, -lo) / dtypeMax
        scale = torch.where(scale == 0, torch.ones_like(scale), scale)
    scale = torch.nan_to_num(scale, nan=1.0, posinf=1.0, neginf=1.0)
    return (h / scale).to(quant_dtype), scale.to(scale_dtype)


def f32_to_e8m0(x: torch.Tensor) -> torch.Tensor:
    """Biased exponent of ``x``; one more when the mantissa is >= 1.5 (for subnormals only when it is
    > 0.5 of the smallest normal); 0xFF for NaN/Inf.  The increment wraps in 8 bits."""
    u = x.contiguous().view(torch.int32)
    e = (u >> 23) & 0xFF
    up = ((u & 0x400000) != 0) & (((u & 0x3FFFFF) != 0) | (e > 0))
    e = torch.where(up, (e + 1) & 0xFF, e)
    e = torch.where(((u >> 23) & 0xFF) == 0xFF, torch.full_like(e, 0xFF), e)
    return e.to(torch.uint8).view(fp8_e8m0)


def e8m0_to_f32(s: torch.Tensor) -> torch.Tensor:
    """``2^(b-127)``; byte 0 gives 2^-127 (bits 0x00400000), byte 255 gives NaN."""
    b = s.view(torch.uint8).to(torch.int32)
    bits = b << 23
    bits = torch.where(b == 0, torch.full_like(bits, 0x00400000), bits)
    bits = torch.where(b == 0xFF, torch.full_like(bits, 0x7F800001), bits)
    return bits.view(torch.float32)


_E2M1 = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]


def f32_to_e2m1_codes(y: torch.Tensor) -> torch.Tensor:
    """fp32 -> 4-bit e2m1 codes (uint8, one per element): nearest representable magnitude, ties to the
    even mantissa, saturating at 6; sign in bit 3."""
    a = y.abs()
    code = (
        (a > 0.25).to(torch.uint8)
        + (a >= 0.75).to(torch.uint8)
        + (a > 1.25).to(torch.uint8)
        + (a >= 1.75).to(torch.uint8)
        + (a > 2.5).to(torch.uint8)
        + (a >= 3.5).to(torch.uint8)
        + (a > 5.0).to(torch.uint8)
    )
    sign = (y.contiguous().view(torch.int32) < 0).to(torch.uint8) << 3
    return code | sign


def pack_uint4(codes: torch.Tensor) -> torch.Tensor:
    """Two codes per byte, even index in the low nibble."""
    assert codes.shape[-1] % 2 == 0
    pairs = codes.contiguous().view(*codes.shape[:-1], codes.shape[-1] // 2, 2)
    return (pairs[..., 0] & 0xF) | (pairs[..., 1] << 4)


def f32_to_mxfp4(x: torch.Tensor) -> torch.Tensor:
    return pack_uint4(f32_to_e2m1_codes(x.float())).view(fp4x2)


def mxfp4_to_f32(x: torch.Tensor) -> torch.Tensor:
    """Packed e2m1 bytes -> fp32, low nibble first."""
    b = x.view(torch.uint8)
    codes = torch.stack([b & 0xF, b >> 4], dim=-1).reshape(*b.shape[:-1], b.shape[-1] * 2)
    lut = torch.tensor(_E2M1 + [-v for v in _E2M1], dtype=torch.float32, device=b.device)
    return lut[codes.long()]


def per_1x32_f4_quant(x, scale=None, quant_dtype=fp4x2, shuffle=False):
    """OCP-MX fp4 quantisation, one e8m0 scale per 32 consecutive elements of the last dim:
    scale byte = ``f32_to_e8m0(amax / 4)``, codes = e2m1(x / 2^(scale-127)).
    Returns ``(packed [.., K/2], scale [R, K/32] as e8m0, scaled fp32 values)`` like the reference.  Byte-for-byte
    equal to the reference's quantiser on finite inputs; NaN / Inf elements are not pinned (the threshold chain maps
    NaN to code 0 and Inf to +-6)."""
    assert quant_dtype == fp4x2
    if shuffle:
        raise NotImplementedError("use shuffle_scale_w4 on the returned scales")
    shape = x.shape
    blocks = x.reshape(-1, 32).float()
    amax = blocks.abs().amax(dim=1)
    sc = f32_to_e8m0(amax / 4.0)
    y = blocks / e8m0_to_f32(sc).view(-1, 1)
    packed = f32_to_mxfp4(y).view(torch.uint8).reshape(*shape[:-1], shape[-1] // 2).view(fp4x2)
    rows = x.reshape(-1, shape[-1]).shape[0]
    return packed, sc.view(torch.uint8).reshape(rows, -1).view(fp8_e8m0), y


def f32_to_e2m3_codes(y: torch.Tensor) -> torch.Tensor:
    """fp32 -> 6-bit e2m3 codes (uint8, one per element): nearest representable magnitude, ties to the even
    mantissa, saturating at 7.5; sign in bit 5.  Magnitudes are spaced 1/8 below 2, 1/4 in [2, 4) and 1/2 above, and
    the 5-bit magnitude code counts them in order, so each binade is one round-half-even."""
    a = y.float().abs()
    lo = torch.round(a * 8.0)
    mid = 16.0 + torch.round((a - 2.0) * 4.0)
    hi = 24.0 + torch.round((a - 4.0) * 2.0)
    code = torch.where(a < 2.0, lo, torch.where(a < 4.0, mid, hi)).clamp(max=31.0).to(torch.uint8)
    sign = (y.float().contiguous().view(torch.int32) < 0).to(torch.uint8) << 5
    return code | sign


def pack_fp6_e2m3(x_unpacked: torch.Tensor) -> torch.Tensor:
    """uint8 codes (low 6 bits) ``[.., 4G]`` -> dense bytes ``[.., 3G]``; element j of each group of four sits at bits
    [6j, 6j+6) of the group's 24 bits, least significant byte first."""
    assert x_unpacked.dtype == torch.uint8 and x_unpacked.shape[-1] % 4 == 0
    g = x_unpacked.reshape(*x_unpacked.shape[:-1], -1, 4).to(torch.int32) & 0x3F
    word = g[..., 0] | (g[..., 1] << 6) | (g[..., 2] << 12) | (g[..., 3] << 18)
    out = torch.stack([word & 0xFF, (word >> 8) & 0xFF, (word >> 16) & 0xFF], dim=-1).to(torch.uint8)
    return out.reshape(*x_unpacked.shape[:-1], x_unpacked.shape[-1] // 4 * 3).contiguous()


def fp6_e2m3_to_f32(x_unpacked: torch.Tensor) -> torch.Tensor:
    """uint8 codes (low 6 bits: sign, 2 exponent bits with bias 1, 3 mantissa bits) -> fp32."""
    c = (x_unpacked & 0x3F).to(torch.int32)
    e, m = (c >> 3) & 3, (c & 7).float()
    mag = torch.where(e == 0, m / 8.0, torch.ldexp(1.0 + m / 8.0, e - 1))
    return torch.where((c & 0x20) != 0, -mag, mag)


def per_1x32_f6_quant(x):
    """OCP-MX fp6 (e2m3) quantisation of an A operand ``[M, K]``: scale byte = ``f32_to_e8m0(amax / 4)``, codes =
    e2m3(x / 2^(scale-127)).  Returns ``(a_pad [M, K] uint8, scale [M, K/32] uint8, codes [M, K] uint8)`` like the
    reference: ``a_pad`` holds per 32 elements the 24 packed bytes followed by 8 zero bytes, which is what the GEMM
    reads.  Finite inputs only."""
    shape = x.shape
    blocks = x.reshape(-1, 32).float()
    amax = blocks.abs().amax(dim=1)
    sc = f32_to_e8m0(amax / 4.0)
    y = blocks / e8m0_to_f32(sc).view(-1, 1)
    codes = f32_to_e2m3_codes(y).reshape(shape).contiguous()
    M, K = codes.shape[0], codes.shape[-1]
    a_pad = torch.zeros(M, K // 32, 32, dtype=torch.uint8, device=x.device)
    a_pad[:, :, :24] = pack_fp6_e2m3(codes).view(M, K // 32, 24)
    return a_pad.view(M, K), sc.view(torch.uint8).reshape(M, -1), codes


def per_1x32_f8_quant(x):
    """OCP-MX fp8 (e4m3fn) quantisation: scale byte = ``f32_to_e8m0(max(amax, 1e-30) / 448)``, codes =
    e4m3fn(clamp(x / 2^(scale-127), +-448)).  Returns ``(x_q [.., K] float8_e4m3fn, scale [.., K/32] uint8)``.
    Finite inputs only."""
    shape = x.shape
    blocks = x.contiguous().reshape(-1, 32).float()
    amax = blocks.abs().amax(dim=-1).clamp_min(1e-30)
    sc = f32_to_e8m0(amax / 448.0)
    sf = e8m0_to_f32(sc).clamp_min(1e-30)
    x_q = (blocks / sf.view(-1, 1)).clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(shape).contiguous()
    return x_q, sc.view(torch.uint8).reshape(*shape[:-1], shape[-1] // 32).contiguous()
