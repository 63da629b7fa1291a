"""ctypes binding of ``libpsgemm.so`` (the C ABI declared in ``include/psgemm.h``).

The library is the only compute path: if it is missing or fails to load, ``lib()`` raises
``RuntimeError``; nothing falls back to torch or to the CPU.
"""

from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libpsgemm.so")
ABI_VERSION = 7

IN_DTYPE = {"int8": 0, "fp8": 1, "fp16": 2, "bf16": 3, "int4": 6}  # "int4": the MoE stages' int8 x packed-int4 weights
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
    "psg_init",
    "psg_static_scratch_bytes",
    "psg_gemm_a8w8_static",
    "psg_tile_coords",
    "psg_debug_tile_order",
    "psg_moe_gemm",
    "psg_moe_mx_gemm",
    "psg_moe_mx_scale_sort",
    "psg_moe_reduce",
    "psg_moe_reduce_masked",
    "psg_moe_sorting",
    "psg_moe_sorting_workspace_bytes",
    "psg_moe_topk_gating",
    "psg_moe_softmax_sorting",
    "psg_moe_softmax_sorting_fused",
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
        ("b_layout", ctypes.c_int32),
        ("pad0", ctypes.c_int32),
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
        ("a_dtype", ctypes.c_int32),
        ("b_dtype", ctypes.c_int32),
        ("batch", ctypes.c_int32),
        ("pad0", ctypes.c_int32),
        ("a_row_stride", ctypes.c_int64),
        ("c_row_stride", ctypes.c_int64),
        ("scale_a_chunk_stride", ctypes.c_int64),
        ("a_batch_stride", ctypes.c_int64),
        ("c_batch_stride", ctypes.c_int64),
        ("scale_a_batch_stride", ctypes.c_int64),
    ]


MX_DTYPE = {"fp4": 0, "fp6": 1, "fp8": 2}


class MoeArgs(ctypes.Structure):
    _fields_ = [
        ("out", ctypes.c_void_p),
        ("x", ctypes.c_void_p),
        ("w", ctypes.c_void_p),
        ("scale_x", ctypes.c_void_p),
        ("scale_w", ctypes.c_void_p),
        ("sorted_token_ids", ctypes.c_void_p),
        ("sorted_expert_ids", ctypes.c_void_p),
        ("sorted_weights", ctypes.c_void_p),
        ("num_valid_ids", ctypes.c_void_p),
        ("tokens", ctypes.c_int32),
        ("topk", ctypes.c_int32),
        ("experts", ctypes.c_int32),
        ("model_dim", ctypes.c_int32),
        ("inter_dim", ctypes.c_int32),
        ("sorted_size", ctypes.c_int32),
        ("blocks", ctypes.c_int32),
        ("block_m", ctypes.c_int32),
        ("in_dtype", ctypes.c_int32),
        ("out_dtype", ctypes.c_int32),
        ("stage", ctypes.c_int32),
        ("doweight", ctypes.c_int32),
        ("accumulate", ctypes.c_int32),
        ("x_slot_major", ctypes.c_int32),
        ("no_pairing", ctypes.c_int32),
        ("pad0", ctypes.c_int32),
    ]


class MoeMxArgs(ctypes.Structure):
    _fields_ = [
        ("out", ctypes.c_void_p),
        ("out_scale", ctypes.c_void_p),
        ("a", ctypes.c_void_p),
        ("a_scale", ctypes.c_void_p),
        ("w", ctypes.c_void_p),
        ("w_scale", ctypes.c_void_p),
        ("sorted_token_ids", ctypes.c_void_p),
        ("sorted_expert_ids", ctypes.c_void_p),
        ("sorted_weights", ctypes.c_void_p),
        ("num_valid_ids", ctypes.c_void_p),
        ("tokens", ctypes.c_int32),
        ("experts", ctypes.c_int32),
        ("model_dim", ctypes.c_int32),
        ("inter_dim", ctypes.c_int32),
        ("sorted_size", ctypes.c_int32),
        ("blocks", ctypes.c_int32),
        ("block_m", ctypes.c_int32),
        ("a_dtype", ctypes.c_int32),
        ("out_dtype", ctypes.c_int32),
        ("stage", ctypes.c_int32),
        ("atomic", ctypes.c_int32),
        ("pad0", ctypes.c_int32),
    ]


class MoeSortArgs(ctypes.Structure):
    _fields_ = [
        ("topk_ids", ctypes.c_void_p),
        ("topk_weights", ctypes.c_void_p),
        ("expert_mask", ctypes.c_void_p),
        ("sorted_ids", ctypes.c_void_p),
        ("sorted_weights", ctypes.c_void_p),
        ("sorted_expert_ids", ctypes.c_void_p),
        ("num_valid_ids", ctypes.c_void_p),
        ("zero_buf", ctypes.c_void_p),
        ("zero_bytes", ctypes.c_int64),
        ("workspace", ctypes.c_void_p),
        ("workspace_bytes", ctypes.c_uint64),
        ("tokens", ctypes.c_int32),
        ("topk", ctypes.c_int32),
        ("experts", ctypes.c_int32),
        ("block_m", ctypes.c_int32),
        ("sorted_size", ctypes.c_int32),
        ("blocks", ctypes.c_int32),
    ]


class MoeGatingArgs(ctypes.Structure):
    _fields_ = [
        ("gating", ctypes.c_void_p),
        ("weights", ctypes.c_void_p),
        ("indices", ctypes.c_void_p),
        ("token_expert_indices", ctypes.c_void_p),
        ("tokens", ctypes.c_int32),
        ("experts", ctypes.c_int32),
        ("topk", ctypes.c_int32),
        ("dtype", ctypes.c_int32),
        ("renormalize", ctypes.c_int32),
        ("pad0", ctypes.c_int32),
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
    handle.psg_init.restype = ctypes.c_int
    handle.psg_init.argtypes = []
    handle.psg_static_scratch_bytes.restype = ctypes.c_uint64
    handle.psg_static_scratch_bytes.argtypes = []
    handle.psg_tile_coords.restype = None
    handle.psg_tile_coords.argtypes = [ctypes.c_int32] * 4 + [ctypes.POINTER(ctypes.c_int32)] * 2
    handle.psg_debug_tile_order.restype = ctypes.c_int
    handle.psg_debug_tile_order.argtypes = [ctypes.c_int32] * 3 + [ctypes.c_void_p, ctypes.c_void_p]
    handle.psg_moe_reduce_masked.restype = ctypes.c_int
    handle.psg_moe_reduce_masked.argtypes = [ctypes.c_void_p] * 4 + [ctypes.c_int32] * 5 + [ctypes.c_void_p]
    handle.psg_moe_sorting_workspace_bytes.restype = ctypes.c_uint64
    handle.psg_moe_sorting_workspace_bytes.argtypes = [ctypes.c_int32] * 3
    handle.psg_moe_mx_scale_sort.restype = ctypes.c_int
    handle.psg_moe_mx_scale_sort.argtypes = [ctypes.c_void_p] * 4 + [ctypes.c_int32] * 4 + [ctypes.c_void_p]
    handle.psg_moe_reduce.restype = ctypes.c_int
    handle.psg_moe_reduce.argtypes = [ctypes.c_void_p, ctypes.c_void_p] + [ctypes.c_int32] * 4 + [ctypes.c_void_p]
    handle.psg_moe_softmax_sorting.restype = ctypes.c_int
    handle.psg_moe_softmax_sorting.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    handle.psg_moe_softmax_sorting_fused.restype = ctypes.c_int
    handle.psg_moe_softmax_sorting_fused.argtypes = [ctypes.c_int32] * 3
    for name in ("psg_gemm_a8w8", "psg_gemm_mxfp4", "psg_gemm_a8w8_static", "psg_moe_gemm", "psg_moe_mx_gemm", "psg_moe_sorting", "psg_moe_topk_gating"):
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


class WorkspacePool:
    """Scratch buffers of the split-K plan, one per (owner, device, stream); an owner is one launcher object.

    Launches on one stream are ordered, so they may share a buffer; launches on different streams, or through
    different launchers, get different buffers and cannot race.  A buffer that has been handed out is never released
    while the process lives: a recorded HIP graph or a launch still in flight may hold its address, and the launches
    go through ctypes, which the caching allocator knows nothing about.  When a larger problem arrives a new buffer is
    allocated and the old one is parked.  Nothing is allocated while the stream is being captured into a graph: a
    capture on a stream that has no buffer yet borrows the buffer the same launcher got on another stream of that
    device (the warm-up run the reference's ``flyc.compile`` protocol makes before any capture), so replays of that
    graph must not overlap with launches of the same launcher on the warm-up stream; if there is none the call
    raises."""

    def __init__(self, alloc=None, capturing=None):
        import threading

        self._lock = threading.Lock()
        self._live = {}     # (owner, device index, stream handle) -> current buffer
        self._parked = []   # outgrown buffers, kept alive on purpose
        self._alloc = alloc
        self._capturing = capturing

    def get(self, owner, device_index: int, stream: int, nbytes: int):
        if nbytes <= 0:
            return None
        key = (owner, int(device_index), int(stream))
        with self._lock:
            cur = self._live.get(key)
            if cur is not None and cur.numel() >= nbytes:
                return cur
            if (self._capturing or _torch_capturing)():
                for (o, d, _), buf in self._live.items():
                    if o == owner and d == key[1] and buf.numel() >= nbytes:
                        return buf
                raise RuntimeError(
                    f"the split-K plan needs {nbytes} bytes of workspace but this launcher has none that large on device "
                    f"{key[1]} yet, and allocating during graph capture is not possible; call the launcher once (or "
                    "flyc.compile) before capturing")
            new = (self._alloc or _torch_alloc)(int(nbytes), key[1])
            if cur is not None:
                self._parked.append(cur)
            self._live[key] = new
            return new


def _torch_capturing() -> bool:
    import torch

    return bool(torch.cuda.is_current_stream_capturing())


def _torch_alloc(nbytes: int, device_index: int):
    import torch

    return torch.empty(nbytes, dtype=torch.uint8, device=f"cuda:{device_index}")


_pool = WorkspacePool()


def workspace(device, nbytes: int, stream=0, owner="shared"):
    """Scratch for the split-K path of launcher ``owner`` on ``device`` for launches on ``stream`` (raw handle);
    ``None`` when ``nbytes`` is 0."""
    import torch

    if nbytes <= 0:
        return None
    d = torch.device(device)
    index = d.index if d.index is not None else torch.cuda.current_device()
    return _pool.get(owner, index, int(stream), int(nbytes))


def check_operand(name, t, *, min_elems, elem_sizes, device=None):
    """Cheap host-side validation of a tensor operand before its raw address reaches a kernel: device tensor,
    contiguous, expected element size, at least ``min_elems`` elements.  Returns the tensor's device."""
    if not getattr(t, "is_cuda", False):
        raise ValueError(f"{name} must be a device (cuda) tensor, got {getattr(t, 'device', type(t).__name__)}")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    if t.element_size() not in elem_sizes:
        raise ValueError(f"{name} has {t.element_size()}-byte elements ({t.dtype}); expected {' or '.join(map(str, elem_sizes))}")
    if t.numel() < min_elems:
        raise ValueError(f"{name} holds {t.numel()} elements, this call needs at least {min_elems}")
    if device is not None and t.device != device:
        raise ValueError(f"{name} is on {t.device}, the output is on {device}")
    return t.device
