"""MX preshuffle GEMM entry point: fp4 (e2m1), fp6 (e2m3) or fp8 (e4m3fn) A against preshuffled fp4 or fp8 W, one e8m0
scale per 32 K elements on both sides.

Drop-in for the reference's ``launch_gemm`` (kernels/gemm/mxfp4_preshuffle.py:57-91): same positional
signature.  Operands are raw device pointers (what ``flyc.from_c_void_p(fx.Uint8, t.data_ptr())``
produces: an object with an integer ``value``, or a plain int, or a tensor).  ``batch > 1`` is strided-batched in one
launch (grid.z); the ``a_`` / ``sca_`` / ``c_`` row and batch strides have the reference's meaning and units
(mxfp4_preshuffle.py:177-196, 435-444): ``a_row_stride`` and both batch strides in bytes, ``sca_row_stride`` in dwords
between 32-row scale chunks, ``c_row_stride`` in elements, ``c_batch_stride`` in bytes; a negative value keeps the
contiguous ``[B, M, *]`` default.  As in the reference, the A and scale_a ROW strides only apply when ``batch > 1``.
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
    _no_split=False,
):
    """Launch ``C[b] = A_mx[b] @ W_mx[b]^T`` (``[M,K] x [N,K]``) for every batch ``b`` on ``stream``.  The reference's
    constraints are kept: ``tile_k in {128, 256}``, ``tile_n % 128 == 0``, ``K % tile_k == 0``
    (mxfp4_preshuffle.py:122,316).  Dense unbatched fp4 x fp4 runs on the tuned fp4 kernels (``tile_*`` are hints the
    planner may override); every other combination runs on the general MX kernel, which has a fixed tile."""
    if a_dtype not in _lib.MX_DTYPE:
        raise ValueError(f"a_dtype must be fp4/fp6/fp8, got {a_dtype!r}")
    if b_dtype not in ("fp4", "fp8"):
        raise ValueError(f"b_dtype must be fp4/fp8, got {b_dtype!r}")
    B = int(batch)
    if B < 1 or B > 65535:
        raise ValueError(f"batch must be in [1, 65535], got {batch}")
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
    a_row = Kk // 2 if a_dtype == "fp4" else Kk
    b_row = Kk // 2 if b_dtype == "fp4" else Kk
    chunk = (Kk // 256) * 256  # bytes of one 32-row chunk of shuffled scales
    chunks_m = (M + 31) // 32
    # strides in bytes (C rows in elements); the row strides of A / scale_a only count when batch > 1
    a_rs = int(a_row_stride) if (B > 1 and int(a_row_stride) >= 0) else a_row
    sa_cs = int(sca_row_stride) * 4 if (B > 1 and int(sca_row_stride) >= 0) else chunk
    c_rs = int(c_row_stride) if int(c_row_stride) >= 0 else Nn
    a_bs = int(a_batch_stride) if int(a_batch_stride) >= 0 else M * a_row
    sa_bs = int(sca_batch_stride) if int(sca_batch_stride) >= 0 else chunks_m * chunk
    c_bs = int(c_batch_stride) if int(c_batch_stride) >= 0 else M * Nn * 2
    fast = a_dtype == "fp4" and b_dtype == "fp4" and B == 1 and c_rs == Nn and _force_path != 3
    # operands given as tensors are checked on the host (raw addresses cannot be): device, contiguity, extent
    for name, t, need in (("c", arg_c, (B - 1) * c_bs + ((M - 1) * c_rs + Nn) * 2), ("a", arg_a, (B - 1) * a_bs + (M - 1) * a_rs + a_row),
                          ("b", arg_b, B * Nn * b_row), ("scale_a", arg_scale_a, (B - 1) * sa_bs + (chunks_m - 1) * sa_cs + chunk),
                          ("scale_b", arg_scale_b, B * (Nn // 32) * chunk)):
        if hasattr(t, "data_ptr") and hasattr(t, "is_cuda") and not (name == "c" and _acc is not None):
            if not t.is_cuda or not t.is_contiguous():
                raise ValueError(f"{name} must be a contiguous device tensor")
            if t.numel() * t.element_size() < need:
                raise ValueError(f"{name} holds {t.numel() * t.element_size()} bytes, this call needs at least {need}")
    h = _lib.stream_handle(stream)
    lib = _lib.lib()
    args = _lib.MxArgs()
    args.c = None if _acc is not None else _addr(arg_c)
    args.a, args.b = _addr(arg_a), _addr(arg_b)
    args.scale_a, args.scale_b = _addr(arg_scale_a), _addr(arg_scale_b)
    args.M, args.N, args.K = M, Nn, Kk
    args.out_dtype = _lib.OUT_DTYPE[out_dtype]
    args.a_dtype, args.b_dtype = _lib.MX_DTYPE[a_dtype], _lib.MX_DTYPE[b_dtype]
    args.batch = B
    args.a_row_stride, args.c_row_stride, args.scale_a_chunk_stride = a_rs, c_rs, sa_cs
    args.a_batch_stride, args.c_batch_stride, args.scale_a_batch_stride = a_bs, c_bs, sa_bs
    args.tile_m, args.tile_n, args.tile_k = int(tile_m), int(tile_n), int(tile_k)
    if _tile is not None:
        args.tile_m, args.tile_n = int(_tile[0]), int(_tile[1])
    args.xcd_swizzle = int(xcd_swizzle)
    args.force_path = int(_force_path)
    args.reserved = int(_wave_layout)
    if fast:
        if _tile is not None:
            args.tile_k = max(1, int(_splits))
            need = args.tile_k * args.M * args.N * 4 if args.tile_k > 1 else 0
        else:
            need = lib.psg_workspace_bytes(args.M, args.N, args.K, 4)
    elif B == 1 and c_rs == Nn and not _no_split:
        need = lib.psg_workspace_bytes(args.M, args.N, args.K, 5)
    else:
        need = 0
    if need and _acc is None and hasattr(arg_c, "device"):
        ws = _lib.workspace(arg_c.device, need, h, owner="mxfp4")
        args.workspace, args.workspace_bytes = ws.data_ptr(), ws.numel()
    if _acc is None:
        rc = lib.psg_gemm_mxfp4(ctypes.byref(args), h)
    else:
        rc = lib.psg_gemm_mxfp4_acc(ctypes.byref(args), _addr(_acc), h)
    if rc:
        _lib.check(rc, "psg_gemm_mxfp4")
