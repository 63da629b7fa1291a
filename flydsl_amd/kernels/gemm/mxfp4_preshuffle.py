"""MXFP4 preshuffle GEMM entry point (e2m1 x e2m1, e8m0 scale per 32 K elements).

Drop-in for the reference's ``launch_gemm`` (kernels/gemm/mxfp4_preshuffle.py:57-91): same positional
signature.  Operands are raw device pointers (what ``flyc.from_c_void_p(fx.Uint8, t.data_ptr())``
produces: an object with an integer ``value``, or a plain int, or a tensor).  Supported subset:
``a_dtype == b_dtype == "fp4"`` and all strides ``-1`` (the contiguous ``[B, M, *]`` layout); ``batch > 1`` runs one
launch per batch on the same stream with the reference's default batch strides (mxfp4_preshuffle.py:177-196).  The
rest raises ``NotImplementedError``.
"""

from __future__ import annotations

import ctypes

from ... import _lib


def _addr(x) -> int:
    if isinstance(x, int):
        return x
    if hasattr(x, "data_ptr"):
        return int(x.data_ptr())
    v = getattr(x, "value", None)
    if v is None:
        raise TypeError(f"cannot take a device address from {type(x).__name__}")
    return int(v)


def launch_gemm(
    arg_c,
    arg_a,
    arg_b,
    arg_scale_a,
    arg_scale_b,
    i32_m,
    i32_n,
    stream,
    N,
    K,
    tile_m,
    tile_n,
    tile_k,
    a_dtype,
    out_dtype,
    b_dtype,
    batch,
    a_row_stride,
    a_batch_stride,
    sca_row_stride,
    sca_batch_stride,
    c_row_stride,
    c_batch_stride,
    waves_per_eu,
    xcd_swizzle=0,
    *,
    _force_path=0,
    _tile=None,
    _acc=None,
    _wave_layout=0,
    _splits=0,
):
    """Launch ``C[M,N] = A_mx[M,K] @ W_mx[N,K]^T`` on ``stream``.  The reference's constraints are kept:
    ``tile_k in {128, 256}``, ``tile_n % 128 == 0``, ``K % tile_k == 0`` (mxfp4_preshuffle.py:122,316)."""
    if a_dtype != "fp4" or b_dtype != "fp4":
        raise NotImplementedError(f"only fp4 x fp4 is built (got a_dtype={a_dtype!r}, b_dtype={b_dtype!r})")
    if int(batch) < 1:
        raise ValueError(f"batch must be >= 1, got {batch}")
    if any(int(s) >= 0 for s in (a_row_stride, a_batch_stride, sca_row_stride, sca_batch_stride, c_row_stride, c_batch_stride)):
        raise NotImplementedError("caller-controlled row/batch strides are not built; pass -1")
    if out_dtype not in _lib.OUT_DTYPE:
        raise ValueError(f"out_dtype must be bf16/fp16, got {out_dtype!r}")
    if tile_k not in (128, 256):
        raise ValueError(f"tile_k must be 128 or 256, got {tile_k}")
    if tile_n % 128 != 0:
        raise ValueError(f"tile_n must be a multiple of 128, got {tile_n}")
    if K % tile_k != 0:
        raise ValueError(f"K={K} must be a multiple of tile_k={tile_k}")
    if int(i32_n) != int(N):
        raise ValueError(f"runtime N={i32_n} differs from the compile-time N={N}")
    M, Nn, Kk = int(i32_m), int(N), int(K)
    # default batch strides of the reference: A [B,M,K/2], W [B,N,K/2], scale_a over ceil(M/32) chunks, scale_b over N/32
    # chunks of (K/256)*256 bytes each, C [B,M,N]
    chunk = (Kk // 256) * 256
    strides = (M * Nn * 2, M * (Kk // 2), Nn * (Kk // 2), ((M + 31) // 32) * chunk, (Nn // 32) * chunk)
    B = int(batch)
    chunks_m = (M + 31) // 32
    # operands given as tensors are checked on the host (raw addresses cannot be): device, contiguity, extent
    for name, t, need in (("c", arg_c, B * M * Nn * 2), ("a", arg_a, B * M * (Kk // 2)), ("b", arg_b, B * Nn * (Kk // 2)),
                          ("scale_a", arg_scale_a, B * chunks_m * chunk), ("scale_b", arg_scale_b, B * (Nn // 32) * chunk)):
        if hasattr(t, "data_ptr") and hasattr(t, "is_cuda") and not (name == "c" and _acc is not None):
            if not t.is_cuda or not t.is_contiguous():
                raise ValueError(f"{name} must be a contiguous device tensor")
            if t.numel() * t.element_size() < need:
                raise ValueError(f"{name} holds {t.numel() * t.element_size()} bytes, this call needs at least {need}")
    h = _lib.stream_handle(stream)
    base = (None if _acc is not None else _addr(arg_c), _addr(arg_a), _addr(arg_b), _addr(arg_scale_a), _addr(arg_scale_b))
    lib = _lib.lib()
    for bz in range(int(batch)):
        args = _lib.MxArgs()
        args.c = None if base[0] is None else base[0] + bz * strides[0]
        args.a = base[1] + bz * strides[1]
        args.b = base[2] + bz * strides[2]
        args.scale_a = base[3] + bz * strides[3]
        args.scale_b = base[4] + bz * strides[4]
        args.M, args.N, args.K = M, Nn, Kk
        args.out_dtype = _lib.OUT_DTYPE[out_dtype]
        args.tile_m, args.tile_n, args.tile_k = int(tile_m), int(tile_n), int(tile_k)
        if _tile is not None:
            args.tile_m, args.tile_n = int(_tile[0]), int(_tile[1])
        args.xcd_swizzle = int(xcd_swizzle)
        args.force_path = int(_force_path)
        args.reserved = int(_wave_layout)
        if _tile is not None:
            args.tile_k = max(1, int(_splits))
            need = args.tile_k * args.M * args.N * 4 if args.tile_k > 1 else 0
        else:
            need = lib.psg_workspace_bytes(args.M, args.N, args.K, 4)
        if need and _acc is None and hasattr(arg_c, "device"):
            ws = _lib.workspace(arg_c.device, need, h, owner="mxfp4")
            args.workspace, args.workspace_bytes = ws.data_ptr(), ws.numel()
        if _acc is None:
            rc = lib.psg_gemm_mxfp4(ctypes.byref(args), h)
        else:
            rc = lib.psg_gemm_mxfp4_acc(ctypes.byref(args), _addr(_acc) + bz * M * Nn * 4, h)
        if rc:
            _lib.check(rc, "psg_gemm_mxfp4")
