"""ctypes binding of ``libpsgemm.so`` (the C ABI declared in ``include/psgemm.h``).

The library is the only compute path: if it is missing or fails to load, ``lib()`` raises
``RuntimeError``; nothing falls back to torch or to the CPU.
"""

from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libpsgemm.so")
ABI_VERSION = 1

IN_DTYPE = {"int8": 0, "fp8": 1, "fp16": 2, "bf16": 3}
OUT_DTYPE = {"bf16": 0, "fp16": 1}
EPILOGUE = {"none": 0, "bias": 1, "bias_relu": 2, "bias_silu": 3, "bias_gelu": 4}

EXPORTS = (
    "psg_abi_version",
    "psg_last_error",
    "psg_workspace_bytes",
    "psg_gemm_a8w8",
    "psg_gemm_a8w8_acc",
    "psg_gemm_mxfp4",
    "psg_gemm_mxfp4_acc",
    "psg_quant_pertoken",
    "psg_quant_mxfp4",
)


class A8W8Args(ctypes.Structure):
    _fields_ = [
        ("c", ctypes.c_void_p),
        ("a", ctypes.c_void_p),
        ("b", ctypes.c_void_p),
        ("scale_a", ctypes.c_void_p),
        ("scale_b", ctypes.c_void_p),
        ("bias", ctypes.c_void_p),
        ("workspace", ctypes.c_void_p),
        ("workspace_bytes", ctypes.c_uint64),
        ("M", ctypes.c_int32),
        ("N", ctypes.c_int32),
        ("K", ctypes.c_int32),
        ("in_dtype", ctypes.c_int32),
        ("out_dtype", ctypes.c_int32),
        ("epilogue", ctypes.c_int32),
        ("tile_m", ctypes.c_int32),
        ("tile_n", ctypes.c_int32),
        ("tile_k", ctypes.c_int32),
        ("xcd_swizzle", ctypes.c_int32),
        ("force_path", ctypes.c_int32),
        ("reserved", ctypes.c_int32),
    ]


class MxArgs(ctypes.Structure):
    _fields_ = [
        ("c", ctypes.c_void_p),
        ("a", ctypes.c_void_p),
        ("b", ctypes.c_void_p),
        ("scale_a", ctypes.c_void_p),
        ("scale_b", ctypes.c_void_p),
        ("workspace", ctypes.c_void_p),
        ("workspace_bytes", ctypes.c_uint64),
        ("M", ctypes.c_int32),
        ("N", ctypes.c_int32),
        ("K", ctypes.c_int32),
        ("out_dtype", ctypes.c_int32),
        ("tile_m", ctypes.c_int32),
        ("tile_n", ctypes.c_int32),
        ("tile_k", ctypes.c_int32),
        ("xcd_swizzle", ctypes.c_int32),
        ("force_path", ctypes.c_int32),
        ("reserved", ctypes.c_int32),
    ]


_lib = None


def lib() -> ctypes.CDLL:
    """Load ``libpsgemm.so`` once.  Raises ``RuntimeError`` when it is absent or has the wrong ABI."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is not built; run `make -C {os.path.join(_HERE, 'csrc')}` "
            "(there is no CPU or torch fallback for the preshuffle GEMM)"
        )
    try:
        handle = ctypes.CDLL(LIB_PATH)
    except OSError as e:  # missing libamdhip64 etc.
        raise RuntimeError(f"cannot load {LIB_PATH}: {e}") from e
    handle.psg_abi_version.restype = ctypes.c_int
    handle.psg_last_error.restype = ctypes.c_char_p
    handle.psg_workspace_bytes.restype = ctypes.c_uint64
    handle.psg_workspace_bytes.argtypes = [ctypes.c_int32] * 4
    for name in ("psg_gemm_a8w8", "psg_gemm_mxfp4"):
        fn = getattr(handle, name)
        fn.restype = ctypes.c_int
        fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
    for name in ("psg_gemm_a8w8_acc", "psg_gemm_mxfp4_acc"):
        fn = getattr(handle, name)
        fn.restype = ctypes.c_int
        fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    handle.psg_quant_pertoken.restype = ctypes.c_int
    handle.psg_quant_pertoken.argtypes = [ctypes.c_void_p, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32,
                                          ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p]
    handle.psg_quant_mxfp4.restype = ctypes.c_int
    handle.psg_quant_mxfp4.argtypes = [ctypes.c_void_p, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32,
                                       ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p]
    got = handle.psg_abi_version()
    if got != ABI_VERSION:
        raise RuntimeError(f"{LIB_PATH} has ABI version {got}, this package needs {ABI_VERSION}")
    _lib = handle
    return _lib


def check(rc: int, what: str) -> None:
    """0 -> return; negative (validation) -> ValueError; positive (hipError_t) -> RuntimeError."""
    if rc == 0:
        return
    msg = lib().psg_last_error().decode("utf-8", "replace")
    if rc < 0:
        raise ValueError(f"{what}: {msg} (code {rc})")
    raise RuntimeError(f"{what}: HIP error {rc}: {msg}")


def stream_handle(stream) -> int:
    """Accept what the reference's launchers accept as ``stream``: ``torch.cuda.Stream``, a raw integer
    handle, ``None`` (the current torch stream), or any object with a ``cuda_stream`` attribute."""
    if stream is None:
        import torch

        return int(torch.cuda.current_stream().cuda_stream)
    if isinstance(stream, int):
        return stream
    h = getattr(stream, "cuda_stream", None)
    if h is None:
        h = getattr(stream, "value", None)
    if h is None:
        raise TypeError(f"cannot use {type(stream).__name__} as a stream")
    return int(h)


_workspaces = {}


def workspace(device, nbytes: int):
    """Per-device scratch for the split-K path (one torch allocation, grown on demand, zero-size means none).
    Growing allocates, so the first call for a new largest problem must happen outside graph capture -- which the
    reference's own protocol guarantees (``flyc.compile`` runs the launcher once before any capture).  Launches
    that may overlap on one device (different streams) must not rely on this shared buffer."""
    import torch

    if nbytes <= 0:
        return None
    key = torch.device(device).index if torch.device(device).index is not None else torch.cuda.current_device()
    cur = _workspaces.get(key)
    if cur is None or cur.numel() < nbytes:
        cur = torch.empty(int(nbytes), dtype=torch.uint8, device=f"cuda:{key}")
        _workspaces[key] = cur
    return cur
