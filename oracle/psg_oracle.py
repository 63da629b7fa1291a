"""CPU oracle for the preshuffle quantized GEMM path.  TEST INFRASTRUCTURE ONLY.

Nothing under ``flydsl_amd/`` or ``kernels/`` may import this module; only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` use it, and only as
the checker.

Everything here is a numpy restatement of what the reference computes on the host (torch CPU)
for this path.  Each function names the reference lines it follows.  The reference keeps no
golden vectors for this path, so each function is pinned in ``tests/test_oracle_*.py`` by
independent means (closed-form index maps, exhaustive code tables, brute force on tiny inputs,
library casts, float64 cross-checks); the pin for each function is named in its docstring.

All tensors are numpy arrays.  fp8 / fp4 / e8m0 data are carried as ``uint8`` bit patterns.
"""

from __future__ import annotations

import numpy as np

# ----------------------------------------------------------------------------------------------
# Codecs
# ----------------------------------------------------------------------------------------------

#: e2m1 magnitudes by 3-bit code; bit 3 of the 4-bit code is the sign
#: (tests/kernels/utils/gemm_common_utils.py:31-48).
E2M1_LUT = np.array(
    [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0],
    dtype=np.float32,
)


def e4m3fn_to_f32(code: np.ndarray) -> np.ndarray:
    """Decode OCP e4m3fn bit patterns (bias 7, no inf, 0x7f/0xff = NaN) to fp32.

    This is what ``tensor.to(torch.float32)`` does for ``torch.float8_e4m3fn`` in the reference's
    oracle (tests/kernels/test_preshuffle_gemm.py:105-106).  Pinned by comparison with torch's own
    cast on all 256 codes.
    """
    c = np.asarray(code, dtype=np.uint8).astype(np.int32)
    s = (c >> 7) & 1
    e = (c >> 3) & 0xF
    m = c & 7
    sub = np.ldexp(m.astype(np.float32) / 8.0, -6)
    nor = np.ldexp(1.0 + m.astype(np.float32) / 8.0, e - 7)
    v = np.where(e == 0, sub, nor).astype(np.float32)
    v = np.where((e == 15) & (m == 7), np.float32(np.nan), v)
    return np.where(s == 1, -v, v).astype(np.float32)


_E4M3_TABLE = None


def _e4m3_table():
    global _E4M3_TABLE
    if _E4M3_TABLE is None:
        _E4M3_TABLE = e4m3fn_to_f32(np.arange(256, dtype=np.uint8))
    return _E4M3_TABLE


def f32_to_e4m3fn(x: np.ndarray) -> np.ndarray:
    """fp32 -> e4m3fn bit pattern, round-to-nearest-even, no saturation (|x| >= 465 -> NaN).

    Semantics of ``tensor.to(torch.float8_e4m3fn)`` used by ``pertoken_quant``
    (tests/utils.py:71).  Pinned against torch's cast on a dense sweep including every midpoint
    between adjacent codes.
    """
    x = np.asarray(x, dtype=np.float32)
    bits = x.view(np.uint32)
    sign = ((bits >> 31) & 1).astype(np.uint8)
    ax = np.abs(x).astype(np.float64)
    out = np.zeros(x.shape, dtype=np.uint8)
    nan = np.isnan(x) | (ax >= 480.0)
    # exponent of the target binade, clamped to the subnormal binade (2^-6)
    with np.errstate(divide="ignore"):
        e = np.floor(np.log2(np.where(ax > 0, ax, 1.0))).astype(np.int64)
    e = np.maximum(e, -6)
    step = np.ldexp(1.0, e - 3)  # spacing of representable values in this binade
    q = ax / step  # exact in float64 (power-of-two scaling)
    r = np.rint(q)  # numpy rint = round half to even
    val = r * step  # rounded magnitude (may carry into the next binade)
    # encode the rounded magnitude
    with np.errstate(divide="ignore"):
        e2 = np.floor(np.log2(np.where(val > 0, val, 1.0))).astype(np.int64)
    is_sub = val < 2.0**-6
    mant_sub = np.rint(val / 2.0**-9).astype(np.int64)  # m/8 * 2^-6
    mant_nor = np.rint((val / np.ldexp(1.0, e2) - 1.0) * 8.0).astype(np.int64)
    code = np.where(is_sub, mant_sub, ((e2 + 7) << 3) | mant_nor).astype(np.int64)
    nan = nan | (code >= 0x7F)
    code = np.where(nan, 0x7F, code).astype(np.uint8)
    out = code | (sign << 7).astype(np.uint8)
    return out.astype(np.uint8)


def e8m0_to_f32(b: np.ndarray) -> np.ndarray:
    """e8m0 byte -> fp32 ``2^(b-127)``; byte 0 -> bits 0x00400000 (2^-127), byte 255 -> NaN.

    tests/kernels/utils/gemm_common_utils.py:63-71.  Pinned on all 256 bytes against ``ldexp``.
    """
    b = np.asarray(b, dtype=np.uint8)
    bits = b.astype(np.uint32) << np.uint32(23)
    bits = np.where(b == 0, np.uint32(0x00400000), bits)
    bits = np.where(b == 0xFF, np.uint32(0x7F800001), bits)
    return bits.astype(np.uint32).view(np.float32)


def f32_to_e8m0(x: np.ndarray) -> np.ndarray:
    """fp32 -> e8m0 byte: biased exponent, plus one when mantissa bit 22 is set and (bit 21 or any
    lower bit is set or the exponent is non-zero); NaN/Inf exponent stays 0xFF; the increment wraps
    in uint8 like the reference's.

    tests/kernels/utils/gemm_common_utils.py:53-60.  Pinned on exponent boundaries and the
    mantissa cases (1.0, 1.25, 1.5-ulp, 1.5, 1.75, subnormals) by hand-computed expectations.
    """
    u = np.asarray(x, dtype=np.float32).view(np.uint32)
    exponent = ((u >> 23) & 0xFF).astype(np.uint8)
    nan_case = exponent == 0xFF
    round_case = ((u & 0x400000) > 0) & (((u & 0x200000) > 0) | ((u & 0x1FFFFF) > 0) | (exponent > 0))
    exponent = np.where(round_case, exponent + np.uint8(1), exponent).astype(np.uint8)
    exponent = np.where(nan_case, np.uint8(0xFF), exponent).astype(np.uint8)
    return exponent


def f32_to_floatx(x: np.ndarray, ebits: int, mbits: int) -> np.ndarray:
    """fp32 -> sign/ebits/mbits code in the low bits of a uint8, round-to-nearest-even, saturating to the largest
    magnitude (no NaN / Inf codes).

    Follows the bit-level algorithm of ``_f32_to_floatx_unpacked``
    (tests/kernels/utils/gemm_common_utils.py:162-275): saturate at >= max_normal, a denormal branch that adds and
    subtracts a magic constant below min_normal, and a normal branch that re-biases the exponent and adds a rounding
    bias with the tie bit.  Pinned for (2,1) and (2,3) against an independent nearest-value search with ties-to-even on
    dense sweeps that contain every midpoint.
    """
    x = np.asarray(x, dtype=np.float32)
    exp_bias = (1 << (ebits - 1)) - 1
    max_int = (1 << (ebits + mbits)) - 1
    magic_adder = (1 << (23 - mbits - 1)) - 1
    max_normal = 2.0 ** (((1 << ebits) - 1) - exp_bias) * (((1 << (mbits + 1)) - 1) / float(1 << mbits))
    min_normal = 2.0 ** (1 - exp_bias)
    denorm_exp = (127 - exp_bias) + (23 - mbits) + 1
    denorm_mask_int = np.int32(denorm_exp << 23)
    denorm_mask_float = np.array(denorm_mask_int, dtype=np.int32).view(np.float32)

    xi = x.view(np.int32)
    sign = xi & np.int32(-0x80000000)
    ax_i = xi ^ sign
    ax = ax_i.view(np.float32)

    saturate = ax >= max_normal
    denormal = (~saturate) & (ax < min_normal)
    normal = ~(saturate | denormal)

    with np.errstate(invalid="ignore", over="ignore"):
        den = (ax + denorm_mask_float).astype(np.float32).view(np.int32) - denorm_mask_int
    den = (den & 0xFF).astype(np.uint8)

    nor = ax_i.astype(np.int64)
    mant_odd = (nor >> (23 - mbits)) & 1
    nor = nor + (((exp_bias - 127) << 23) + magic_adder)
    nor = nor + mant_odd
    nor = (nor >> (23 - mbits)) & 0xFF
    nor = nor.astype(np.uint8)

    out = np.full(x.shape, max_int, dtype=np.uint8)
    out = np.where(denormal, den, out)
    out = np.where(normal, nor, out)
    sign_lp = ((sign.view(np.uint32) >> np.uint32(23 + 8 - mbits - ebits)) & np.uint32(1 << (ebits + mbits))).astype(
        np.uint8
    )
    return (out | sign_lp).astype(np.uint8)


def f32_to_e2m1(x: np.ndarray) -> np.ndarray:
    """fp32 -> 4-bit e2m1 code (one per uint8), RNE, saturating to +-6: ``_f32_to_floatx_unpacked(x, 2, 1)``."""
    return f32_to_floatx(x, 2, 1)


def f32_to_e2m3(x: np.ndarray) -> np.ndarray:
    """fp32 -> 6-bit e2m3 code (one per uint8), RNE, saturating to +-7.5: ``_f32_to_floatx_unpacked(x, 2, 3)``
    (tests/kernels/utils/gemm_common_utils.py:763)."""
    return f32_to_floatx(x, 2, 3)


def e2m3_to_f32(codes: np.ndarray) -> np.ndarray:
    """6-bit e2m3 code (sign, 2 exponent bits with bias 1, 3 mantissa bits) -> fp32
    (tests/kernels/utils/gemm_common_utils.py:727-741).  Pinned on all 64 codes against the format's definition
    evaluated with ``ldexp`` and against the encoder's round trip."""
    c = np.asarray(codes, dtype=np.uint8) & 0x3F
    exp = ((c >> 3) & 0x3).astype(np.int32)
    mant = (c & 0x7).astype(np.float32)
    mag = np.where(exp == 0, mant / np.float32(8.0), np.ldexp(np.float32(1.0) + mant / np.float32(8.0), exp - 1))
    return np.where((c & 0x20) != 0, -mag, mag).astype(np.float32)


def pack_fp6(codes: np.ndarray) -> np.ndarray:
    """Four 6-bit codes -> three bytes, little-endian bit order (element j of a group of four at bits [6j, 6j+6) of
    the 24-bit group): ``pack_fp6_e2m3`` (tests/kernels/utils/gemm_common_utils.py:708-721).  Pinned against a
    big-integer bit-string construction."""
    c = np.asarray(codes, dtype=np.uint8)
    assert c.shape[-1] % 4 == 0
    g = (c.reshape(c.shape[:-1] + (-1, 4)).astype(np.uint32)) & 0x3F
    word = g[..., 0] | (g[..., 1] << 6) | (g[..., 2] << 12) | (g[..., 3] << 18)
    out = np.stack([word & 0xFF, (word >> 8) & 0xFF, (word >> 16) & 0xFF], axis=-1).astype(np.uint8)
    return out.reshape(c.shape[:-1] + (c.shape[-1] // 4 * 3,))


def unpack_fp6_padded(a_pad: np.ndarray) -> np.ndarray:
    """Inverse of the A-operand layout of ``per_1x32_f6_quant``: ``[R, K]`` bytes (24 packed + 8 padding per 32
    elements) -> ``[R, K]`` 6-bit codes.  Not in the reference; pinned as the inverse of ``pack_fp6``."""
    p = np.asarray(a_pad, dtype=np.uint8)
    r, k = p.shape
    g = p.reshape(r, k // 32, 32)[:, :, :24].reshape(r, k // 32, 8, 3).astype(np.uint32)
    word = g[..., 0] | (g[..., 1] << 8) | (g[..., 2] << 16)
    codes = np.stack([(word >> (6 * j)) & 0x3F for j in range(4)], axis=-1)
    return codes.reshape(r, k).astype(np.uint8)


def pack_uint4(codes: np.ndarray) -> np.ndarray:
    """Two 4-bit codes per byte, even index in the LOW nibble
    (tests/kernels/utils/gemm_common_utils.py:142-147).  Pinned by a two-element example."""
    codes = np.asarray(codes, dtype=np.uint8)
    assert codes.shape[-1] % 2 == 0
    flat = codes.reshape(-1)
    packed = (flat[1::2] << 4) | (flat[0::2] & 0xF)
    return packed.reshape(codes.shape[:-1] + (codes.shape[-1] // 2,)).astype(np.uint8)


def mxfp4_to_f32(packed: np.ndarray) -> np.ndarray:
    """Packed e2m1 bytes -> fp32, low nibble first
    (tests/kernels/utils/gemm_common_utils.py:23-50)."""
    p = np.asarray(packed, dtype=np.uint8)
    lo = p & 0xF
    hi = p >> 4
    codes = np.stack([lo, hi], axis=-1).reshape(p.shape[:-1] + (p.shape[-1] * 2,))
    return E2M1_LUT[codes]


# ----------------------------------------------------------------------------------------------
# Host quantisers
# ----------------------------------------------------------------------------------------------


def pertoken_quant(x: np.ndarray, quant: str = "int8"):
    """Per-row symmetric quantisation (tests/utils.py:29-73).

    ``x`` fp32 ``[R, K]``; ``quant`` is ``"int8"`` (dtypeMax 127, cast truncates toward zero) or
    ``"fp8"`` (e4m3fn, dtypeMax 448, cast rounds to nearest even).  Returns ``(y, scale)`` with
    ``y`` int8 / uint8 bit patterns ``[R, K]`` and ``scale`` fp32 ``[R, 1]``.

    Pinned by closed-form invariants (row max maps to +-dtypeMax, zero rows get scale 1,
    reconstruction error bounds) and by an elementwise comparison with torch's own amax / divide /
    cast ops.
    """
    x = np.asarray(x, dtype=np.float32)
    dtype_max = np.float32(127.0 if quant == "int8" else 448.0)
    h = np.nan_to_num(x, nan=0.0, posinf=float(dtype_max), neginf=-float(dtype_max)).astype(np.float32)
    row_max = h.max(axis=-1, keepdims=True)
    row_min = h.min(axis=-1, keepdims=True)
    amax = np.maximum(row_max, -row_min).astype(np.float32)
    scale = (amax / dtype_max).astype(np.float32)
    scale[scale == 0] = 1.0
    scale = np.nan_to_num(scale, nan=1.0, posinf=1.0, neginf=1.0).astype(np.float32)
    y = (h / scale).astype(np.float32)
    if quant == "int8":
        q = np.trunc(y).astype(np.int8)  # torch float->int8 truncates toward zero
    elif quant == "fp8":
        q = f32_to_e4m3fn(y)
    else:
        raise ValueError(quant)
    return q, scale


def per_1x32_f4_quant(x: np.ndarray):
    """OCP-MX fp4 quantisation with one e8m0 scale per 32 consecutive K elements
    (tests/kernels/utils/gemm_common_utils.py:675-704).

    scale byte = ``f32_to_e8m0(amax / 4)``; ``y = x / e8m0_to_f32(scale)``; codes = e2m1 RNE with
    saturation; packed two per byte.  Returns ``(packed [R, K/2] uint8, scale [R, K/32] uint8)``.

    Pinned through its parts (each codec above is pinned on its own) plus composition invariants:
    dequantised error is at most half an e2m1 step at the chosen scale unless saturated, the
    block maximum never decodes above 6*scale, and all-zero blocks give scale byte 0 and zero codes.
    """
    x = np.asarray(x, dtype=np.float32)
    r, k = x.shape
    assert k % 32 == 0
    blocks = x.reshape(-1, 32)
    amax = np.abs(blocks).max(axis=1).astype(np.float32)
    sc = f32_to_e8m0((amax / np.float32(4.0)).astype(np.float32))
    sf = e8m0_to_f32(sc)
    with np.errstate(over="ignore", invalid="ignore"):
        y = (blocks / sf[:, None]).astype(np.float32)
    codes = f32_to_e2m1(y)
    packed = pack_uint4(codes.reshape(r, k))
    return packed, sc.reshape(r, k // 32)


def per_1x32_f6_quant(x: np.ndarray):
    """OCP-MX fp6 (e2m3) quantisation of an A operand (tests/kernels/utils/gemm_common_utils.py:744-770).

    scale byte = ``f32_to_e8m0(amax / 4)`` (4 = 2^floor(log2 7.5)); codes = e2m3 RNE with saturation.  Returns
    ``(a_pad [R, K] uint8, scale [R, K/32] uint8, codes [R, K] uint8)`` where ``a_pad`` holds per 32 elements the 24
    packed bytes followed by 8 zero bytes (the layout the kernel reads).  Pinned through its parts plus composition
    invariants (error at most half an e2m3 step at the chosen scale unless saturated; zero blocks -> scale 0, codes 0).
    """
    x = np.asarray(x, dtype=np.float32)
    r, k = x.shape
    assert k % 32 == 0
    blocks = x.reshape(-1, 32)
    amax = np.abs(blocks).max(axis=1).astype(np.float32)
    sc = f32_to_e8m0((amax / np.float32(4.0)).astype(np.float32))
    sf = e8m0_to_f32(sc)
    with np.errstate(over="ignore", invalid="ignore"):
        y = (blocks / sf[:, None]).astype(np.float32)
    codes = f32_to_e2m3(y).reshape(r, k)
    a_pad = np.zeros((r, k // 32, 32), dtype=np.uint8)
    a_pad[:, :, :24] = pack_fp6(codes).reshape(r, k // 32, 24)
    return a_pad.reshape(r, k), sc.reshape(r, k // 32), codes


def per_1x32_f8_quant(x: np.ndarray):
    """OCP-MX fp8 (e4m3fn) quantisation (tests/kernels/utils/gemm_common_utils.py:773-790).

    ``amax`` clamped to >= 1e-30; scale byte = ``f32_to_e8m0(amax / 448)``; ``y = clamp(x / max(2^(s-127), 1e-30),
    -448, 448)`` cast to e4m3fn (RNE).  Returns ``(codes [R, K] uint8, scale [R, K/32] uint8)``.  Pinned through its
    parts plus composition invariants (block maximum decodes within one e4m3 step of itself; relative error of normal
    values <= 2^-4).
    """
    x = np.asarray(x, dtype=np.float32)
    r, k = x.shape
    assert k % 32 == 0
    blocks = x.reshape(-1, 32)
    amax = np.maximum(np.abs(blocks).max(axis=1).astype(np.float32), np.float32(1e-30))
    sc = f32_to_e8m0((amax / np.float32(448.0)).astype(np.float32))
    sf = np.maximum(e8m0_to_f32(sc), np.float32(1e-30))
    with np.errstate(over="ignore", invalid="ignore"):
        y = np.clip((blocks / sf[:, None]).astype(np.float32), np.float32(-448.0), np.float32(448.0))
    return f32_to_e4m3fn(y).reshape(r, k), sc.reshape(r, k // 32)


# ----------------------------------------------------------------------------------------------
# Wire formats
# ----------------------------------------------------------------------------------------------


def shuffle_weight(w: np.ndarray) -> np.ndarray:
    """Preshuffle ``W[N, K]`` (1- or 2-byte elements) into MFMA-fragment order, layout (16, 16)
    (tests/utils.py:76-96): ``view(N/16, 16, K/32, 32/Kp, Kp).permute(0, 2, 3, 1, 4)`` with
    ``Kp = 16 / itemsize`` elements.  Shape and dtype are kept.

    Pinned by the closed-form destination offset and explicit loops on tiny inputs.
    """
    w = np.ascontiguousarray(w)
    n, k = w.shape
    kp = 16 // w.dtype.itemsize
    assert n % 16 == 0 and k % 32 == 0
    v = w.reshape(n // 16, 16, k // 32, 32 // kp, kp).transpose(0, 2, 3, 1, 4)
    return np.ascontiguousarray(v).reshape(n, k)


def shuffle_weight_w4(packed: np.ndarray) -> np.ndarray:
    """Preshuffle packed fp4 bytes ``[N, K/2]``: ``view(N/16, 16, Kpk/64, 4, 16).permute(0,2,3,1,4)``
    (tests/kernels/utils/gemm_common_utils.py:634-642, NLane=16, non-MoE)."""
    p = np.ascontiguousarray(np.asarray(packed, dtype=np.uint8))
    n, kpk = p.shape
    assert n % 16 == 0 and kpk % 64 == 0
    v = p.reshape(n // 16, 16, kpk // 64, 4, 16).transpose(0, 2, 3, 1, 4)
    return np.ascontiguousarray(v).reshape(n, kpk)


def shuffle_scale_w4(scale: np.ndarray) -> np.ndarray:
    """Permute e8m0 bytes ``[R, K/32]`` -> ``[R/32][K/256][klane 4][nlane 16][kpack 2][npack 2]``
    (tests/kernels/utils/gemm_common_utils.py:645-672, one expert, not gate_up).

    Pinned by the closed-form destination offset
    ``(r/32)*32*KB + (kb/8)*256 + (kb%4)*64 + (r%16)*4 + ((kb%8)/4)*2 + (r%32)/16``.
    """
    s = np.ascontiguousarray(np.asarray(scale, dtype=np.uint8))
    r, kb = s.shape
    assert r % 32 == 0 and kb % 8 == 0
    v = s.reshape(r // 32, 2, 16, kb // 8, 2, 4).transpose(0, 3, 5, 2, 4, 1)
    return np.ascontiguousarray(v).reshape(r, kb)


# ----------------------------------------------------------------------------------------------
# GEMM oracles
# ----------------------------------------------------------------------------------------------


def f16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return np.asarray(b).view(np.float16).astype(np.float32)


def _as_f32_operand(q: np.ndarray, kind: str) -> np.ndarray:
    if kind == "bf16":
        return bf16_bits_to_f32(np.asarray(q).view(np.uint16))
    if kind == "fp16":
        return f16_bits_to_f32(np.asarray(q).view(np.uint16))
    if kind == "int8":
        return np.asarray(q).view(np.int8).astype(np.float32)
    if kind == "fp8":
        return _e4m3_table()[np.asarray(q).view(np.uint8)]
    raise ValueError(kind)


def run_torch(a_q, b_q, scale_a, scale_b, kind: str, bias=None) -> np.ndarray:
    """The reference's parity oracle (tests/kernels/test_preshuffle_gemm.py:103-113): dequantise
    both operands to fp32 (``a * sa[:, None]``, ``b * sb[:, None]``), fp32 matmul ``a @ b.T``,
    optional ``+ bias``; fp32 ``[M, N]`` result.  ``b_q`` is the UN-shuffled weight.

    Pinned by a float64 matmul of the same dequantised operands on small shapes.
    """
    a32 = _as_f32_operand(a_q, kind)
    b32 = _as_f32_operand(b_q, kind)
    if scale_a is not None and scale_b is not None:  # fp16 / bf16 operands carry no scales (:108-109)
        a32 = a32 * np.asarray(scale_a, dtype=np.float32).reshape(-1, 1)
        b32 = b32 * np.asarray(scale_b, dtype=np.float32).reshape(-1, 1)
    c = a32 @ b32.T
    if bias is not None:
        c = c + np.asarray(bias, dtype=np.float32).reshape(1, -1)
    return c.astype(np.float32)


def int32_accumulators(a_q: np.ndarray, b_q: np.ndarray) -> np.ndarray:
    """Exact integer matmul ``sum_k int(A[m,k]) * int(B[n,k])`` as int32 ``[M, N]``.

    The reference has no int32 output; this is the accumulator the int8 kernel must hold before
    its epilogue (kernels/gemm/preshuffle_gemm.py:538,738-740).  Computed in float64 blocks of K
    small enough to be exact, summed in int64.  Pinned against a pure-integer loop on tiny inputs.
    """
    a = np.asarray(a_q).view(np.int8)
    b = np.asarray(b_q).view(np.int8)
    m, k = a.shape
    n = b.shape[0]
    acc = np.zeros((m, n), dtype=np.int64)
    step = 1 << 14  # 127*127*16384 < 2^53: each float64 partial is exact
    for k0 in range(0, k, step):
        part = a[:, k0 : k0 + step].astype(np.float64) @ b[:, k0 : k0 + step].astype(np.float64).T
        acc += part.astype(np.int64)
    assert np.abs(acc).max(initial=0) < 2**31
    return acc.astype(np.int32)


def run_torch_w4(a_packed, b_packed, scale_a, scale_b) -> np.ndarray:
    """MXFP4 parity oracle (tests/kernels/test_preshuffle_gemm.py:404-411): decode nibbles through
    the LUT, multiply each 32-element block by ``2^(e-127)``, fp32 matmul.  Operands and scales are
    UN-shuffled; scale arrays may have more rows than the operands (32-row padding)."""
    x = mxfp4_to_f32(a_packed)
    w = mxfp4_to_f32(b_packed)
    xs = e8m0_to_f32(np.repeat(np.asarray(scale_a, dtype=np.uint8)[: x.shape[0]], 32, axis=1))
    ws = e8m0_to_f32(np.repeat(np.asarray(scale_b, dtype=np.uint8)[: w.shape[0]], 32, axis=1))
    return ((x * xs) @ (w * ws).T).astype(np.float32)


def mx_operand_to_f32(q: np.ndarray, fmt: str) -> np.ndarray:
    """Decode one MX operand to fp32 ``[R, K]``: ``fmt`` "fp4" (packed nibbles ``[R, K/2]``), "fp6" (the padded
    ``[R, K]`` byte layout of ``per_1x32_f6_quant``) or "fp8" (e4m3fn bytes ``[R, K]``)."""
    if fmt == "fp4":
        return mxfp4_to_f32(q)
    if fmt == "fp6":
        return e2m3_to_f32(unpack_fp6_padded(q))
    if fmt == "fp8":
        return e4m3fn_to_f32(q)
    raise ValueError(fmt)


def run_torch_mx(a_q, b_q, scale_a, scale_b, a_fmt: str = "fp4", b_fmt: str = "fp4") -> np.ndarray:
    """Parity oracle of the mixed-format MX GEMM: ``dequant(A) @ dequant(W)^T`` in fp32 with one e8m0 scale per 32 K
    elements (tests/kernels/test_preshuffle_gemm.py:530-537 for fp6 x fp4, :650-653 for fp8 x fp8).  Operands and scales
    are UN-shuffled; scale arrays may have more rows than the operands."""
    x = mx_operand_to_f32(a_q, a_fmt)
    w = mx_operand_to_f32(b_q, b_fmt)
    xs = e8m0_to_f32(np.repeat(np.asarray(scale_a, dtype=np.uint8)[: x.shape[0]], 32, axis=1))
    ws = e8m0_to_f32(np.repeat(np.asarray(scale_b, dtype=np.uint8)[: w.shape[0]], 32, axis=1))
    return ((x * xs) @ (w * ws).T).astype(np.float32)


# ----------------------------------------------------------------------------------------------
# MoE 2-stage (tests/kernels/test_moe_gemm_2stage.py, tests/kernels/test_ref.py)
# ----------------------------------------------------------------------------------------------


def moe_sorting(topk_ids: np.ndarray, topk_weights: np.ndarray, num_experts: int, block_size: int, expert_mask=None):
    """Expert sorting of routed (token, slot) pairs (tests/kernels/test_moe_gemm_2stage.py:99-137): experts in
    ascending order, each expert's pairs in row-major (token, slot) order and padded to whole blocks with
    ``(topk << 24) | tokens``; one expert id per block, -1 for unused blocks.  Returns ``(sorted_ids int32,
    sorted_weights fp32 (0 in padding rows; the reference leaves them uninitialised), sorted_expert_ids int32,
    num_tokens_post_pad int32[2])``.  With ``expert_mask`` (one flag per expert) the experts whose flag is 0 are
    dropped and the others numbered densely in ``sorted_expert_ids`` (tests/kernels/test_moe_sorting.py:74-110).
    Pinned by invariants (every pair exactly once and inside its expert's blocks, padding values, block count) and
    hand-worked examples, one of them with a mask."""
    ids = np.asarray(topk_ids)
    wts = np.asarray(topk_weights, dtype=np.float32)
    tokens, topk = ids.shape
    max_padded = int(ids.size + num_experts * block_size - topk)
    max_blocks = (max_padded + block_size - 1) // block_size
    sorted_ids = np.full(max_padded, (topk << 24) | tokens, dtype=np.int32)
    sorted_w = np.zeros(max_padded, dtype=np.float32)
    sorted_e = np.full(max_blocks, -1, dtype=np.int32)
    begin = blk = skipped = 0
    for e in range(num_experts):
        if expert_mask is not None and not int(expert_mask[e]):
            skipped += 1
            continue
        t, s = np.nonzero(ids == e)
        n = t.size
        nb = (n + block_size - 1) // block_size
        sorted_ids[begin : begin + n] = (s.astype(np.int32) << 24) | t.astype(np.int32)
        sorted_w[begin : begin + n] = wts[t, s]
        begin += nb * block_size
        sorted_e[blk : blk + nb] = e - skipped
        blk += nb
    return sorted_ids, sorted_w, sorted_e, np.array([begin, tokens], dtype=np.int32)


def topk_gating_softmax(gating, topk: int, renormalize: bool = True):
    """Router gating (kernels/moe/topk_gating_softmax_kernel.py:545-650): fp32 ``p = exp2((x - max) * log2 e) * (1 / sum)``;
    ``topk`` rounds of arg-max over ``p`` in which the LOWER expert index wins ties and the winner is masked with -inf
    (:585-618); ``renormalize`` multiplies the winners by ``1 / max(their sum, 1e-20)`` (:623-625).  ``gating`` ``[tokens,
    experts]`` (any float dtype; converted to fp32 as the kernel does).  Returns ``(weights fp32 [tokens, topk], indices int32
    [tokens, topk], token_expert_indices int32 [tokens, topk] = k * tokens + token)`` (:648-650).
    Pinned by ``scipy.special.softmax`` + a stable descending sort in float64, closed forms (uniform logits, one dominant
    logit, topk = experts) and shift invariance."""
    x = np.asarray(gating, dtype=np.float32)
    tokens, experts = x.shape
    mx = x.max(axis=1, keepdims=True)
    e = np.exp2((x - mx) * np.float32(1.4426950408889634)).astype(np.float32)
    p = e * (np.float32(1.0) / e.sum(axis=1, keepdims=True, dtype=np.float32))
    w = np.zeros((tokens, topk), dtype=np.float32)
    idx = np.zeros((tokens, topk), dtype=np.int32)
    rows = np.arange(tokens)
    for k in range(topk):
        j = p.argmax(axis=1)  # the first maximum: the lowest index among equals
        w[:, k] = p[rows, j]
        idx[:, k] = j
        p[rows, j] = -np.inf
    if renormalize:
        w = w * (np.float32(1.0) / np.maximum(w.sum(axis=1, keepdims=True, dtype=np.float32), np.float32(1e-20)))
    tei = (np.arange(topk, dtype=np.int32)[None, :] * np.int32(tokens) + np.arange(tokens, dtype=np.int32)[:, None]).astype(np.int32)
    return w.astype(np.float32), idx, tei


def moe_reduce(x, topk_ids=None, expert_mask=None):
    """Slot reduction behind the non-accumulating stage 2 (kernels/moe/moe_gemm_2stage/moe_reduce.py:141-150): ``y[t] =
    sum_k x[t, k]`` in fp32 in slot order; with a mask only the slots with ``expert_mask[topk_ids[t, k]] != 0`` count (the
    others are replaced by zeros before the addition, so whatever they hold, NaN included, never reaches the sum).  ``x``
    fp32 ``[tokens, topk, dim]``.  Pinned by a scalar loop on a hand-made case with poisoned masked rows."""
    x = np.asarray(x, dtype=np.float32)
    tokens, topk, dim = x.shape
    y = np.zeros((tokens, dim), dtype=np.float32)
    for k in range(topk):
        if expert_mask is None:
            y += x[:, k]
        else:
            on = np.asarray(expert_mask)[np.asarray(topk_ids)[:, k]] != 0
            y[on] += x[on, k]
    return y


def moe_gemm1(x_q, w1_q, scale_x, scale_w1, topk_ids, topk_weights, inter_dim: int, doweight_stage1: bool, kind: str = "fp8",
              x_slot_major: bool = False):
    """Stage 1 of the 2-stage MoE (tests/kernels/test_ref.py:91-161, per-row scales): for every routed (token, slot)
    with expert e, ``y = W1[e] @ x[token]`` over the dequantised operands, ``out[token, slot] = silu(y[:inter]) *
    y[inter:]`` (times the routing weight when ``doweight_stage1``).  ``x_q [tokens, model_dim]``, ``w1_q
    [experts*2*inter, model_dim]`` bit patterns (``kind`` "fp8" / "int8"), scales fp32 per row.  With ``x_slot_major`` (the
    int8smooth inputs, tests/kernels/test_moe_gemm_2stage.py:482-519) ``x_q`` / ``scale_x`` hold one row per (slot, token)
    at ``slot*tokens + token`` and the pair (token, slot) multiplies ITS row.  Returns fp32 ``[tokens, topk, inter_dim]``.
    Pinned by scalar float64 loops on tiny inputs (both layouts)."""
    x = _as_f32_operand(np.asarray(x_q), kind) * np.asarray(scale_x, dtype=np.float32).reshape(-1, 1)
    w = _as_f32_operand(np.asarray(w1_q), kind) * np.asarray(scale_w1, dtype=np.float32).reshape(-1, 1)
    ids = np.asarray(topk_ids)
    tokens, topk = ids.shape
    w = w.reshape(-1, 2 * inter_dim, x.shape[1])
    out = np.zeros((tokens, topk, inter_dim), dtype=np.float32)
    for e in range(w.shape[0]):
        t, s = np.nonzero(ids == e)
        if t.size == 0:
            continue
        y2 = (x[s * tokens + t if x_slot_major else t] @ w[e].T).astype(np.float32)
        g, u = y2[:, :inter_dim], y2[:, inter_dim:]
        with np.errstate(over="ignore"):
            y = (g / (np.float32(1.0) + np.exp(-g))).astype(np.float32) * u
        if doweight_stage1:
            y = y * np.asarray(topk_weights, dtype=np.float32)[t, s][:, None]
        out[t, s] = y
    return out


def moe_gemm2(a2_q, w2_q, scale_a2, scale_w2, topk_ids, topk_weights, model_dim: int, doweight_stage2: bool, kind: str = "fp8",
              reduce_slots: bool = True):
    """Stage 2 of the 2-stage MoE (tests/kernels/test_ref.py:164-240, per-row scales): ``y = W2[e] @ a2[token, slot]``
    (times the routing weight when ``doweight_stage2``), summed over the slots into ``[tokens, model_dim]`` fp32
    (``reduce_slots=False`` keeps ``[tokens, topk, model_dim]``, what the non-accumulating kernel writes).  ``a2_q
    [tokens, topk, inter]``, ``w2_q [experts*model_dim, inter]``.  Pinned by scalar float64 loops on tiny inputs."""
    ids = np.asarray(topk_ids)
    tokens, topk = ids.shape
    a = _as_f32_operand(np.asarray(a2_q).reshape(tokens * topk, -1), kind) * np.asarray(scale_a2, dtype=np.float32).reshape(-1, 1)
    a = a.reshape(tokens, topk, -1)
    w = _as_f32_operand(np.asarray(w2_q).reshape(-1, a.shape[2]), kind) * np.asarray(scale_w2, dtype=np.float32).reshape(-1, 1)
    w = w.reshape(-1, model_dim, a.shape[2])
    out = np.zeros((tokens, topk, model_dim), dtype=np.float32)
    for e in range(w.shape[0]):
        t, s = np.nonzero(ids == e)
        if t.size == 0:
            continue
        y = (a[t, s] @ w[e].T).astype(np.float32)
        if doweight_stage2:
            y = y * np.asarray(topk_weights, dtype=np.float32)[t, s][:, None]
        out[t, s] = y
    return out.sum(axis=1).astype(np.float32) if reduce_slots else out


# ----------------------------------------------------------------------------------------------
# Epilogue (kernels/gemm/preshuffle_gemm.py:672-714)
# ----------------------------------------------------------------------------------------------


# ----------------------------------------------------------------------------------------------
# Fused MX-FP4 MoE (kernels/moe/mxfp_moe, tests/kernels/test_moe_gemm.py:540-818)
# ----------------------------------------------------------------------------------------------


def e8m0_shuffle(scale: np.ndarray) -> np.ndarray:
    """Scale bytes ``[R, C]`` zero-padded to ``(ceil(R/256)*256, ceil(C/8)*8)``, then ``view(R/32, 2, 16, C/8, 2, 4)``
    permuted to ``(0, 3, 5, 2, 4, 1)`` (tests/kernels/utils/gemm_common_utils.py:114-136).  Pinned by explicit loops over the
    closed-form offset ``((r/32 * C/8 + c/8) * 4 + c%4) * 64 + (r%16) * 4 + ((c%8)/4) * 2 + (r%32)/16`` and by equality with
    ``shuffle_scale_w4`` on shapes that need no padding."""
    sc = np.asarray(scale, dtype=np.uint8)
    r, c = sc.shape
    pad = np.zeros(((r + 255) // 256 * 256, (c + 7) // 8 * 8), dtype=np.uint8)
    pad[:r, :c] = sc
    v = pad.reshape(pad.shape[0] // 32, 2, 16, pad.shape[1] // 8, 2, 4)
    return np.ascontiguousarray(v.transpose(0, 3, 5, 2, 4, 1)).reshape(pad.shape)


def e8m0_unshuffle(shuf: np.ndarray, rows: int, cols: int) -> np.ndarray:
    """Inverse of the permutation of ``e8m0_shuffle`` on a flat byte array holding ``rows x cols`` (multiples of 32 and 8)."""
    v = np.asarray(shuf, dtype=np.uint8).reshape(-1)[: rows * cols].reshape(rows // 32, cols // 8, 4, 16, 2, 2)
    return np.ascontiguousarray(v.transpose(0, 5, 3, 1, 4, 2)).reshape(rows, cols)


def moe_mxfp4_sort(scale: np.ndarray, sorted_ids: np.ndarray, num_valid: int, token_num: int) -> np.ndarray:
    """Scales gathered by sorted position and shuffled (tests/kernels/utils/gemm_common_utils.py:464-598): logical row ``i``
    = scale row of token ``sorted_ids[i] & 0xFFFFFF`` (2-D input) or of ``token * topk + (sorted_ids[i] >> 24)`` (3-D input)
    when the token is below ``token_num`` and ``i < num_valid``, else zero; output ``[ceil(rows/32)*32, C]`` in the 32 x 8
    blocked order (u32 ``[4][16]`` per block, byte = 16-row half + 2 * 4-column half).  Pinned by explicit loops."""
    sc = np.asarray(scale, dtype=np.uint8)
    topk = 1
    if sc.ndim == 3:
        topk = sc.shape[1]
        sc = sc.reshape(-1, sc.shape[-1])
    ids = np.asarray(sorted_ids).astype(np.int64)
    rows = (ids.size + 31) // 32 * 32
    c = sc.shape[1]
    out = np.zeros((rows, c), dtype=np.uint8)
    for i in range(min(ids.size, int(num_valid))):
        tok, slot = int(ids[i]) & 0xFFFFFF, (int(ids[i]) >> 24) & 0xFF
        if tok < token_num:
            out[i] = sc[tok if topk == 1 else tok * topk + slot]
    v = out.reshape(rows // 32, 2, 16, c // 8, 2, 4)
    return np.ascontiguousarray(v.transpose(0, 3, 5, 2, 4, 1)).reshape(rows, c)


def e8m0_roundup(amax: np.ndarray, fmt_max: float = 6.0) -> np.ndarray:
    """Scale byte of the fused kernels' on-device quantiser: biased exponent of the smallest power of two that is
    ``>= amax * (1 / fmt_max)`` (fp32 product), at most 254 (kernels/moe/mxfp_moe/mxfp4_gemm_common.py:221-224:
    ``((bits + 0x7FFFFF) >> 23) & 0xFF``).  Pinned by the defining inequality ``2^(b-128) < amax/fmt_max <= 2^(b-127)`` on
    random values, exact powers of two and zero."""
    w = (np.asarray(amax, dtype=np.float32) * np.float32(1.0 / fmt_max)).astype(np.float32).view(np.uint32)
    b = ((w.astype(np.uint64) + 0x7FFFFF) >> 23) & 0xFF
    return np.minimum(b, 254).astype(np.uint8)


def mxfp4_requant_roundup(y: np.ndarray):
    """``[R, C]`` fp32 -> (packed e2m1 ``[R, C/2]``, scale bytes ``[R, C/32]``) with ``e8m0_roundup`` scales, the
    quantiser at the end of the fused stage 1 (kernels/moe/mxfp_moe/gemm1.py:604-613; codes = nearest-even e2m1 of
    ``y / 2^(byte-127)``, saturating)."""
    y = np.asarray(y, dtype=np.float32)
    r, c = y.shape
    blocks = y.reshape(-1, 32)
    sc = e8m0_roundup(np.abs(blocks).max(axis=1))
    sf = np.ldexp(np.float32(1.0), sc.astype(np.int32) - 127).astype(np.float32)
    q = np.where(sc[:, None] == 0, np.float32(0.0), blocks / np.where(sc == 0, np.float32(1.0), sf)[:, None]).astype(np.float32)
    return pack_uint4(f32_to_e2m1(q).reshape(r, c)), sc.reshape(r, c // 32)


def moe_mx_gemm1(a_q, a_scale, w1_q, w1_scale, sorted_ids, sorted_expert_ids, num_valid: int, tokens: int, inter_dim: int, block_m: int,
                 a_fmt: str = "fp4"):
    """Fused stage 1 by sorted position (kernels/moe/mxfp_moe/host.py:87-165; reference result
    tests/kernels/test_moe_gemm.py:780-784 = ``torch_moe_gemm1`` without routing weights, then a 1x32 fp4 quantisation):
    for sorted row ``i`` of token ``t`` in a block of expert ``e``: ``g = a[t] . W1[e, :inter]``, ``u = a[t] . W1[e, inter:]``,
    ``y = silu(g) * u``.  Operands un-shuffled: ``a_q [tokens, K/2 or K]``, ``a_scale [tokens, K/32]``, ``w1_q [E*2*inter, K/2]``,
    ``w1_scale [E*2*inter, K/32]``.  Returns ``(y fp32 [rows, inter], packed [rows, inter/2], scale [rows, inter/32])`` with
    zero rows for padding; the quantiser is ``mxfp4_requant_roundup``.  Pinned against ``run_torch_mx`` per (token, expert)
    pair in token-major order."""
    ids = np.asarray(sorted_ids).astype(np.int64)
    rows = ids.size
    x = mx_operand_to_f32(a_q, a_fmt) * e8m0_to_f32(np.repeat(np.asarray(a_scale, dtype=np.uint8), 32, axis=1))
    y = np.zeros((rows, inter_dim), dtype=np.float32)
    for blk in range(min(rows, int(num_valid)) // block_m):
        e = int(sorted_expert_ids[blk])
        if e < 0:
            continue
        sl = slice(e * 2 * inter_dim, (e + 1) * 2 * inter_dim)
        w = mxfp4_to_f32(w1_q[sl]) * e8m0_to_f32(np.repeat(np.asarray(w1_scale, dtype=np.uint8)[sl], 32, axis=1))
        tok = ids[blk * block_m : (blk + 1) * block_m] & 0xFFFFFF
        live = tok < tokens
        gu = (x[tok[live]] @ w.T).astype(np.float32)
        g, u = gu[:, :inter_dim], gu[:, inter_dim:]
        y[blk * block_m : (blk + 1) * block_m][live] = (g / (1.0 + np.exp(-g.astype(np.float64)))).astype(np.float32) * u
    packed, sc = mxfp4_requant_roundup(y)
    return y, packed, sc


def moe_mx_gemm2(a2_packed, a2_scale, w2_q, w2_scale, sorted_ids, sorted_weights, sorted_expert_ids, num_valid: int, tokens: int,
                 model_dim: int, block_m: int):
    """Fused stage 2 over the sorted fp4 rows (kernels/moe/mxfp_moe/host.py:168-231; reference result
    tests/kernels/test_moe_gemm.py:785-795): ``flat[i] = a2[i] . W2[e]`` per sorted row, ``out[t] = sum_i weight[i] * flat[i]``
    over the rows of token ``t``.  Returns ``(flat fp32 [rows, model_dim], out fp32 [tokens, model_dim])``."""
    ids = np.asarray(sorted_ids).astype(np.int64)
    rows = ids.size
    a = mxfp4_to_f32(a2_packed) * e8m0_to_f32(np.repeat(np.asarray(a2_scale, dtype=np.uint8), 32, axis=1))
    flat = np.zeros((rows, model_dim), dtype=np.float32)
    out = np.zeros((tokens, model_dim), dtype=np.float32)
    for blk in range(min(rows, int(num_valid)) // block_m):
        e = int(sorted_expert_ids[blk])
        if e < 0:
            continue
        sl = slice(e * model_dim, (e + 1) * model_dim)
        w = mxfp4_to_f32(w2_q[sl]) * e8m0_to_f32(np.repeat(np.asarray(w2_scale, dtype=np.uint8)[sl], 32, axis=1))
        rs = slice(blk * block_m, (blk + 1) * block_m)
        flat[rs] = (a[rs] @ w.T).astype(np.float32)
        for i in range(blk * block_m, (blk + 1) * block_m):
            t = int(ids[i]) & 0xFFFFFF
            if t < tokens:
                out[t] += np.float32(sorted_weights[i]) * flat[i]
    return flat, out


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """fp32 -> bf16 bit pattern (uint16), round-to-nearest-even, NaN kept quiet."""
    u = np.asarray(x, dtype=np.float32).view(np.uint32)
    rounded = (u + np.uint32(0x7FFF) + ((u >> 16) & 1)) >> 16
    nan = np.isnan(np.asarray(x, dtype=np.float32))
    return np.where(nan, (u >> 16) | 0x40, rounded).astype(np.uint16)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def epilogue_a8w8(acc: np.ndarray, scale_a, scale_b, bias=None, act: str = "none") -> np.ndarray:
    """Kernel-order epilogue on raw accumulators: ``(f32(acc) * sa[m]) * sb[n]`` then ``+ bias[n]``
    then the activation, all in fp32 (kernels/gemm/preshuffle_gemm.py:694-714).  Returns fp32."""
    v = np.asarray(acc).astype(np.float32)
    v = (v * np.asarray(scale_a, dtype=np.float32).reshape(-1, 1)).astype(np.float32)
    v = (v * np.asarray(scale_b, dtype=np.float32).reshape(1, -1)).astype(np.float32)
    return apply_bias_act(v, bias, act)


def apply_bias_act(v: np.ndarray, bias=None, act: str = "none") -> np.ndarray:
    """bias / ReLU / SiLU ``x/(1+e^-x)`` / tanh-GELU in the overflow-safe form
    (kernels/gemm/preshuffle_gemm.py:672-692)."""
    v = np.asarray(v, dtype=np.float32)
    if bias is not None:
        v = (v + np.asarray(bias, dtype=np.float32).reshape(1, -1)).astype(np.float32)
    if act == "none":
        return v
    if act == "relu":
        return np.maximum(v, np.float32(0.0))
    if act == "silu":
        return (v * (np.float32(1.0) / (np.float32(1.0) + np.exp(-v)))).astype(np.float32)
    if act == "gelu":
        y = (np.float32(0.7978845608) * (v + np.float32(0.044715) * v * v * v)).astype(np.float32)
        e = np.exp(np.float32(-2.0) * np.abs(y)).astype(np.float32)
        num = np.where(y > 0, np.float32(2.0), np.float32(2.0) * e)
        return (np.float32(0.5) * v * (num * (np.float32(1.0) / (np.float32(1.0) + e)))).astype(np.float32)
    raise ValueError(act)


# ----------------------------------------------------------------------------------------------
# Verification helpers (tests/test_common.py:353-423)
# ----------------------------------------------------------------------------------------------


def violating_fraction(out: np.ndarray, ref: np.ndarray, rtol: float, atol: float) -> float:
    """Fraction of elements failing ``|out-ref| <= atol + rtol*|ref|`` (``checkAllclose``)."""
    out = np.asarray(out, dtype=np.float32)
    ref = np.asarray(ref, dtype=np.float32)
    close = np.isclose(out, ref, rtol=rtol, atol=atol)
    return float((~close).sum()) / max(1, out.size)


def logits_diff(x: np.ndarray, y: np.ndarray) -> float:
    """``1 - 2*sum(xy)/sum(x^2+y^2)`` in float64 (``verify_output``'s fallback metric)."""
    x = np.asarray(x, dtype=np.float64)
    y = np.asarray(y, dtype=np.float64)
    den = (x * x + y * y).sum()
    if den == 0:
        return 0.0
    d = 1.0 - 2.0 * (x * y).sum() / den
    return 1.0 if np.isnan(d) else float(d)


def verify_output(out, ref, atol=1e-2, rtol=1e-2, logits_diff_threshold=2e-3) -> bool:
    """Reference acceptance rule: pass if fewer than 5 % of elements violate isclose, else pass if
    the logits-diff metric is within the threshold (tests/test_common.py:397-423)."""
    if violating_fraction(out, ref, rtol, atol) < 0.05:
        return True
    return logits_diff(out, ref) <= logits_diff_threshold


def within_north_star_tolerance(out, ref, rel: float = 1e-2):
    """The build's own (tighter) bar: ``|out-ref| <= rel*|ref| + rel*max|ref|`` everywhere.
    Returns ``(ok, worst_ratio)`` where ``worst_ratio`` is max of ``|out-ref| / bound``."""
    out = np.asarray(out, dtype=np.float32)
    ref = np.asarray(ref, dtype=np.float32)
    bound = rel * np.abs(ref) + rel * np.abs(ref).max(initial=0.0)
    err = np.abs(out - ref)
    if not np.all(np.isfinite(out)):
        return False, float("inf")
    ratio = float((err / np.maximum(bound, 1e-30)).max(initial=0.0))
    return bool(np.all(err <= bound)), ratio


# ----------------------------------------------------------------------------------------------
# Workgroup-id remap (kernels/common/mma/mfma_preshuffle_pipeline.py:685-729)
# ----------------------------------------------------------------------------------------------


def xcd_remap_bx_by(bx: int, by: int, m: int, *, tile_m: int, tile_n: int, n: int, xcd_swizzle: int, num_xcds: int = 8):
    """Remap ``(bx, by)`` so that workgroup ids dealt round-robin over XCDs form contiguous ranges
    per XCD, grouped ``xcd_swizzle`` M-tiles per N sweep.  Pinned by bijectivity over whole grids."""
    if xcd_swizzle <= 0:
        return bx, by
    gx = n // tile_n
    gy = (m + tile_m - 1) // tile_m
    linear = bx * gx + by
    num = gx * gy
    q, r = divmod(num, num_xcds)
    xcd = linear % num_xcds
    in_xcd = linear // num_xcds
    wgid = xcd * q + min(xcd, r) + in_xcd
    per_group = xcd_swizzle * gx
    group = wgid // per_group
    first_m = group * xcd_swizzle
    size_m = min(gy - first_m, xcd_swizzle)
    in_group = wgid % per_group
    return first_m + in_group % size_m, in_group // size_m


# ----------------------------------------------------------------------------------------------
# The reference's CPU path, literally (torch ops), for the cpu_baseline timing
# ----------------------------------------------------------------------------------------------


def run_torch_cpu(a_q, b_q, scale_a, scale_b):
    """``run_torch`` with torch CPU tensors exactly as the reference runs it on a CPU-only box
    (tests/kernels/test_preshuffle_gemm.py:103-113): ``a.to(f32) * sa[:, None]``,
    ``b.to(f32) * sb[:, None]``, ``torch.mm(a32, b32.T)``.  ``a_q`` / ``b_q`` are torch int8 or
    float8_e4m3fn CPU tensors (``b_q`` un-shuffled)."""
    import torch

    a32 = a_q.to(torch.float32) * scale_a.view(-1, 1)
    b32 = b_q.to(torch.float32) * scale_b.view(-1, 1)
    return torch.mm(a32, b32.T)


def run_torch_w4_cpu(a_packed, b_packed, scale_a, scale_b):
    """``run_torch_w4`` with torch CPU tensors (tests/kernels/test_preshuffle_gemm.py:404-411)."""
    import torch

    lut = torch.from_numpy(E2M1_LUT.copy())

    def dec(p):
        b = p.view(torch.uint8)
        codes = torch.stack([b & 0xF, b >> 4], dim=-1).reshape(b.shape[0], -1)
        return lut[codes.long()]

    def sc(s, rows):
        b = s.view(torch.uint8)[:rows].to(torch.int32)
        bits = torch.where(b == 0, torch.full_like(b, 0x00400000), b << 23)
        return bits.view(torch.float32).repeat_interleave(32, dim=1)

    x = dec(a_packed) * sc(scale_a, a_packed.shape[0])
    w = dec(b_packed) * sc(scale_b, b_packed.shape[0])
    return torch.mm(x, w.T)
